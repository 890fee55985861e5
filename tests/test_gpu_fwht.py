"""GPU parity: Walsh-Hadamard rotation and its fusion with quantization vs the CPU oracle.

The reference computes x @ H as a dense bf16 matmul whose accumulation order is XLA's; the kernel
uses f32 butterflies.  Hence: exact equality where every partial sum is exactly representable
(small integers), <= 1 ulp on a tiny fraction otherwise, and bit-exact quantization *given the
kernel's own rotated values*.
"""
import numpy as np
import pytest
import torch

from oracle import qwix_oracle as O
from tests import util

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('n', [2, 8, 64, 256, 1024, 2048, 4096, 8192, 16384])
def test_fwht_exact_on_small_integers(n):
  from qwix_amd.contrib import hadamard_rot as hr
  g = util.rng(n)
  x = g.integers(-4, 5, (6, n)).astype(np.float32)
  p = int(np.log2(n))
  want = x.astype(np.float64) @ O.hadamard_matrix(p).astype(np.float64)
  y = hr.fwht(torch.from_numpy(x).to(util.DEV), 1)
  assert np.array_equal(util.f32np(y), want.astype(np.float32))
  if n <= 64:  # |sums| <= 256: exact in bf16 too
    yb = hr.fwht(torch.from_numpy(x).to(torch.bfloat16).to(util.DEV), 1)
    assert np.array_equal(util.f32np(yb), want.astype(np.float32))


@pytest.mark.parametrize('rows', [3, 8, 37, 2048, 4096])
def test_matrix_core_rotation_exact_on_small_integers(rows):
  """bf16 rows of 8192 in whole trips of 2048 rows (2048, 4096: the matrix-core kernel; fewer rows: the register
  kernel) take seven of the thirteen butterfly levels on the matrix cores (products with +-1 and f32 sums:
  exact on small integers like the butterflies), one wavefront per row.  Every partial sum of integers in [-4, 4] is an
  integer below 2^24, so the result is the exact transform rounded once to bf16, for any number of rows per wavefront,
  with and without the sign vectors in front of and behind the transform and the output factor."""
  from qwix_amd.contrib import hadamard_rot as hr
  n, p = 8192, 13
  g = util.rng(rows)
  x = g.integers(-4, 5, (rows, n)).astype(np.float32)
  xt = torch.from_numpy(x).to(torch.bfloat16).to(util.DEV)
  H = O.hadamard_matrix(p).astype(np.float32)
  want = x @ H                                   # integers below 2^24: exact in f32 whatever the order
  y = hr.fwht(xt, 1)
  assert y.dtype == torch.bfloat16
  assert np.array_equal(util.f32np(y), O.round_to_bf16(want))
  pre = g.choice([-1.0, 1.0], n).astype(np.float32)
  post = g.choice([-1.0, 1.0], n).astype(np.float32)
  dev = lambda a: torch.from_numpy(a).to(torch.bfloat16).to(util.DEV)
  y2 = hr.fwht(xt, 1, pre_sign=dev(pre), post_sign=dev(post), out_scale=1.0 / n)
  want2 = O.round_to_bf16(O.round_to_bf16(((x * pre) @ H) * post) * np.float32(1.0 / n))
  assert np.array_equal(util.f32np(y2), want2)
  # an impulse in one position of a row picks out one row of H: every index bit is where it belongs
  # (8 rows: the register kernel; 2048 rows: one whole trip of the matrix-core kernel, which is what runs there)
  if rows in (8, 2048):
    places = (1, 4, 8, 32, 256, 512, 1024, 4096, 8191, 2730)
    e = np.zeros((rows, n), np.float32)
    for i in range(rows):
      e[i, places[i % len(places)]] = 3.0
    ye = util.f32np(hr.fwht(torch.from_numpy(e).to(torch.bfloat16).to(util.DEV), 1))
    for i in list(range(min(rows, 20))) + [rows - 1]:
      assert np.array_equal(ye[i], 3.0 * H[places[i % len(places)]]), i


@pytest.mark.parametrize('qtype,tile', [('int8', None), ('int8', 8), ('int4', 16), ('float8_e4m3fn', 32), ('int8', 64), ('int4', 128),
                                        ('int8', 256), ('float8_e4m3fn', 512), ('int4', None)])
def test_matrix_core_rotation_fused_quantize_group_sizes(qtype, tile):
  """Every scale-group size the fused kernel takes at n = 8192 (the group's index bits sit partly in registers and
  partly across lanes): fused == rotate, then the oracle's quantize of the rotated array, bit for bit."""
  from qwix_amd.contrib import hadamard_rot as hr
  from qwix_amd.core import qarray
  n, rows = 8192, 19
  x_np, x_t = util.make((rows, n), O.BF16, seed=tile or 1)
  x_np[3] = 0
  x_np[5, 100:300] *= 50                          # outliers inside a few groups
  x_t = util.to_gpu(O.round_to_bf16(x_np), O.BF16)
  signs = torch.from_numpy(util.rng(6).choice([-1.0, 1.0], n).astype(np.float32)).to(torch.bfloat16).to(util.DEV)
  kw = dict(qtype=qtype, channelwise_axes=[0])
  if tile:
    kw['tiled_axes'] = {1: tile}
  fused = hr.rotate_and_quantize(x_t, 1, qarray.HowToQuantize(**kw), pre_sign=signs)
  rot = hr.fwht(x_t, 1, pre_sign=signs)
  want = O.quantize(util.farr(rot), O.HowToQuantize(**kw))
  util.assert_qarray_equal(fused, want, f'fused {qtype} {tile}')


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('n', [64, 512, 8192])
def test_rotate_inputs_matches_oracle_and_preserves_product(n, dtype):
  from qwix_amd.contrib import hadamard_rot as hr
  x_np, x_t = util.make((16, n), dtype, seed=n)
  w_np, w_t = util.make((n, 24), dtype, seed=n + 1, scale=0.02)
  gen = torch.Generator().manual_seed(123)
  xr, wr, _ = hr.hadamard_rotate_inputs(x_t, w_t, gen, row_sign_flip=True, col_sign_flip=True, lhs_reduction_dim=1, rhs_reduction_dim=0)
  gen = torch.Generator().manual_seed(123)
  rs = (torch.randint(0, 2, (n,), generator=gen, dtype=torch.int32) * 2 - 1).numpy().astype(np.float64)
  cs = (torch.randint(0, 2, (n,), generator=gen, dtype=torch.int32) * 2 - 1).numpy().astype(np.float64)
  oxr, owr = O.hadamard_rotate_inputs(O.FArr(x_np, dtype), O.FArr(w_np, dtype), rs, cs, lhs_reduction_dim=1, rhs_reduction_dim=0)
  assert tuple(wr.shape) == (n, 24) and wr.stride(0) == 1
  for got, want in ((util.f32np(xr), oxr.v), (util.f32np(wr), owr.v)):
    if dtype == O.BF16:
      ulp = np.abs(want) * 2.0**-7 + 1e-30
      assert np.all(np.abs(got - want) <= ulp), 'more than one bf16 ulp away'
      assert np.mean(got != want) < 2e-3
    else:
      assert np.allclose(got, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())
  prod = util.f32np(xr).astype(np.float64) @ util.f32np(wr).astype(np.float64)
  ref = x_np.astype(np.float64) @ w_np.astype(np.float64)
  tol = 1e-4 if dtype == O.F32 else 3e-2
  assert np.allclose(prod, ref, atol=tol * np.abs(ref).max())


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('qtype,tile', [('int8', None), ('int4', 128), ('float8_e4m3fn', None), ('int8', 64)])
@pytest.mark.parametrize('n', [256, 4096, 8192, 16384])
def test_fused_rotate_quantize_equals_rotate_then_quantize(n, qtype, tile, dtype):
  from qwix_amd.contrib import hadamard_rot as hr
  from qwix_amd.core import qarray
  x_np, x_t = util.make((12, n), dtype, seed=7 * n)
  signs = torch.from_numpy(util.rng(5).choice([-1.0, 1.0], n).astype(np.float32)).to(util.TORCH_DT[dtype]).to(util.DEV)
  kw = dict(qtype=qtype, channelwise_axes=[0])
  if tile:
    kw['tiled_axes'] = {1: tile}
  how = qarray.HowToQuantize(**kw)
  fused = hr.rotate_and_quantize(x_t, 1, how, pre_sign=signs)
  rot = hr.fwht(x_t, 1, pre_sign=signs)
  want = O.quantize(util.farr(rot), O.HowToQuantize(**kw))
  util.assert_qarray_equal(fused, want, f'fused {qtype} {tile}')


def test_weight_side_fused_rotation_feeds_the_grouped_gemm():
  """The Hadamard a8w4 benchmark configuration at reduced shape: rotate both sides, act int8 per token, weight int4 g128."""
  from qwix_amd.contrib import hadamard_rot as hr
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  M, K, N = 64, 1024, 256
  x_np, x_t = util.make((M, K), O.BF16, seed=1)
  g = util.rng(2)
  out_ch = g.choice(K, 11, replace=False)
  x_np[:, out_ch] = O.round_to_bf16(x_np[:, out_ch] * 50)
  x_t = torch.from_numpy(x_np).to(torch.bfloat16).to(util.DEV)
  w_np, w_t = util.make((K, N), O.BF16, seed=3, scale=0.02)
  s_np = g.choice([-1.0, 1.0], K).astype(np.float32)
  s_t = torch.from_numpy(s_np).to(torch.bfloat16).to(util.DEV)
  xq = hr.rotate_and_quantize(x_t, 1, qarray.HowToQuantize(qtype='int8', channelwise_axes=[0]), pre_sign=s_t)
  wq = hr.rotate_and_quantize(w_t, 0, qarray.HowToQuantize(qtype='int4', channelwise_axes=[1], tiled_axes={0: 128}),
                              pre_sign=s_t, out_scale=1.0 / K)
  assert tuple(wq.shape) == (K, N) and tuple(wq.scale.shape) == (K // 128, N)
  out = dg.dot_general(xq, wq, (((1,), (0,)), ((), ())))
  # oracle on the kernel's own rotated values
  xr = hr.fwht(x_t, 1, pre_sign=s_t)
  wr = hr.fwht(w_t, 0, pre_sign=s_t, out_scale=1.0 / K)
  oxq = O.quantize(util.farr(xr), O.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  owq = O.quantize(util.farr(wr.contiguous()), O.HowToQuantize(qtype='int4', channelwise_axes=[1], tiled_axes={0: 128}))
  util.assert_qarray_equal(xq, oxq, 'rotated act')
  util.assert_qarray_equal(wq, owq, 'rotated weight')
  want, wacc = O.fast_dot_general(oxq, owq, (((1,), (0,)), ((), ())), return_acc=True)
  got = util.f32np(out)
  assert np.all(np.abs(got - want.v) <= 1e-2 * np.abs(want.v) + util.partials_envelope(wacc, oxq, owq))
  exact = dg._fast_dot_general(xq, wq, (((1,), (0,)), ((), ())), exact=True)
  assert np.array_equal(util.f32np(exact), want.v)
  # the rotation spreads the outlier channels: quantization error vs the float product stays small
  ref = x_np.astype(np.float64) @ w_np.astype(np.float64)
  assert np.abs(got - ref).mean() / np.abs(ref).mean() < 0.15


@pytest.mark.parametrize('M,K,N,wq_type,group,per_group_act,dtype', [
    (64, 1024, 256, 'int4', 128, False, torch.bfloat16), (200, 2048, 520, 'int8', 256, False, torch.bfloat16),
    (33, 512, 136, 'int4', 128, True, torch.bfloat16), (16, 1024, 128, 'int8', 128, False, torch.float32),
    (128, 4096, 1024, 'int4', 128, False, torch.bfloat16)])
def test_rotate_quantize_multiply_in_one_call(M, K, N, wq_type, group, per_group_act, dtype):
  """qwix_hip_qgemm_hadamard_act through the C ABI (hadamard_quantized_matmul) == rotate_and_quantize followed by the
  sub-channel quantized dot, bit for bit; the latter is held to the oracle by the test above.  (The last shape is one
  whose GEMM cuts K into ranges, in both: the one call takes them from the surplus of its workspace.)"""
  from qwix_amd import _lib
  from qwix_amd.contrib import hadamard_rot as hr
  if M == 128:
    assert _lib.load().qwix_hip_qgemm_grouped_workspace_bytes(M, N, K, group, _lib.INT4) > 0
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  print('case hadamard one call', M, K, N, wq_type, group, per_group_act, dtype, flush=True)
  x_np, x_t = util.make((M, K), O.BF16 if dtype == torch.bfloat16 else O.F32, seed=M + K)
  w_np, w_t = util.make((K, N), O.BF16, seed=N + K, scale=0.02)
  g = util.rng(5)
  s_t = torch.from_numpy(g.choice([-1.0, 1.0], K).astype(np.float32)).to(dtype).to(util.DEV)
  wq = hr.rotate_and_quantize(w_t, 0, qarray.HowToQuantize(qtype=wq_type, channelwise_axes=[1], tiled_axes={0: group}),
                              pre_sign=s_t.to(torch.bfloat16), out_scale=1.0 / K)
  how_x = qarray.HowToQuantize(qtype='int8', channelwise_axes=[0], tiled_axes={1: group} if per_group_act else {})
  xq = hr.rotate_and_quantize(x_t, 1, how_x, pre_sign=s_t)
  want = dg.dot_general(xq, wq, (((1,), (0,)), ((), ())))
  got = hr.hadamard_quantized_matmul(x_t, wq, pre_sign=s_t, act_tile=group if per_group_act else None,
                                     preferred_element_type=want.dtype)
  torch.cuda.synchronize()
  assert got.dtype == want.dtype and torch.equal(got, want), float((got.float() - want.float()).abs().max())
  # and the product it stands for
  ref = x_np.astype(np.float64) @ w_np.astype(np.float64)
  assert np.abs(util.f32np(got) - ref).mean() / np.abs(ref).mean() < 0.2


def test_rotate_quantize_multiply_argument_checks():
  """The one-call entry point refuses a missing or short scratch buffer and activation tiles that are neither the
  whole row nor the weight's group."""
  from qwix_amd import _lib
  L = _lib.load()
  M, N, K, G = 32, 128, 512, 128
  x = torch.zeros(M, K, dtype=torch.bfloat16, device=util.DEV)
  b = torch.zeros(N, K, dtype=torch.int8, device=util.DEV)
  sb = torch.ones(K // G, N, dtype=torch.bfloat16, device=util.DEV)
  out = torch.empty(M, N, dtype=torch.bfloat16, device=util.DEV)
  need = L.qwix_hip_qgemm_hadamard_act_workspace_bytes(M, K, K, _lib.BF16)
  assert need >= M * K + 2 * M
  assert L.qwix_hip_qgemm_hadamard_act_workspace_bytes(M, K, G, _lib.BF16) >= M * K + 2 * M * (K // G)
  assert L.qwix_hip_qgemm_hadamard_act_workspace_bytes(M, K, 96, _lib.BF16) == 0
  ws = torch.empty(need, dtype=torch.uint8, device=util.DEV)
  def call(tile=K, wsp=ws.data_ptr(), nws=need):
    return L.qwix_hip_qgemm_hadamard_act(x.data_ptr(), _lib.BF16, M, N, K, None, None, 1.0, tile, b.data_ptr(), K, _lib.INT8, G,
                                         sb.data_ptr(), _lib.BF16, out.data_ptr(), _lib.BF16, N, wsp, nws, None)
  assert call() == 0
  assert call(wsp=None, nws=0) != 0 and b'workspace' in L.qwix_hip_last_error()
  assert call(nws=need - 1) != 0
  assert call(tile=256) != 0 and b'activation tile' in L.qwix_hip_last_error()
  torch.cuda.synchronize()


def test_fwht_errors():
  from qwix_amd.contrib import hadamard_rot as hr
  with pytest.raises(ValueError, match='power of 2'):
    hr.hadamard_rotate_inputs(torch.ones(2, 6, device=util.DEV), torch.ones(6, 2, device=util.DEV), None,
                              row_sign_flip=False, col_sign_flip=False, lhs_reduction_dim=1, rhs_reduction_dim=0)
  with pytest.raises(ValueError, match='to be the same'):
    hr.hadamard_rotate_inputs(torch.ones(2, 8, device=util.DEV), torch.ones(4, 2, device=util.DEV), None,
                              row_sign_flip=False, col_sign_flip=False, lhs_reduction_dim=1, rhs_reduction_dim=0)
  with pytest.raises(ValueError, match='Key must be provided'):
    hr.hadamard_rotate_inputs(torch.ones(2, 8, device=util.DEV), torch.ones(8, 2, device=util.DEV), None,
                              row_sign_flip=True, col_sign_flip=False, lhs_reduction_dim=1, rhs_reduction_dim=0)
