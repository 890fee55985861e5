"""GPU parity: MFMA quantized GEMM vs the CPU oracle.

int8: raw int32 accumulators bit-exact; scaled outputs bit-exact (the epilogue is a deterministic
elementwise function of the exact accumulator).  fp8: f32 accumulation order differs from the
oracle's exact sum, so outputs are compared at rtol 1e-2 (+ atol for cancelling sums), the
tolerance the north-star states for bf16 outputs.  With f32 outputs the v_mfma_f32_32x32x64_f8f6f4
accumulation itself shows up: its 64-wide dot is summed with less than f32 alignment precision
(measured: up to 1e-4 of the largest output), so the f32 comparison uses rtol 1e-3.
"""
import numpy as np
import pytest
import torch

from oracle import qwix_oracle as O
from tests import util

pytestmark = pytest.mark.gpu
DN = (((1,), (0,)), ((), ()))


def _quantized_pair(M, K, N, dtype, qtype, seed):
  from qwix_amd.core import qarray
  x_np, x_t = util.make((M, K), dtype, seed=seed)
  w_np, w_t = util.make((K, N), dtype, seed=seed + 1, scale=0.02)
  xq = qarray.quantize(x_t, qarray.HowToQuantize(qtype=qtype, channelwise_axes=[0]))
  wq = qarray.quantize(w_t, qarray.HowToQuantize(qtype=qtype, channelwise_axes=[1]))
  oxq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(qtype=qtype, channelwise_axes=[0]))
  owq = O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(qtype=qtype, channelwise_axes=[1]))
  return xq, wq, oxq, owq


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('M,K,N', [(256, 1024, 512), (128, 64, 128), (100, 272, 60), (1, 4096, 1024), (1024, 512, 1024), (1300, 1024, 1100),
                                   (16, 1024, 520), (32, 512, 96), (7, 256, 12300), (33, 256, 64)])
def test_int8_gemm_bit_exact(M, K, N, dtype):
  from qwix_amd.core import dot_general as dg
  print('case int8', M, K, N, dtype, flush=True)
  xq, wq, oxq, owq = _quantized_pair(M, K, N, dtype, 'int8', seed=M + K + N)
  out, acc = dg._fast_dot_general(xq, wq, DN, return_accumulators=True)
  torch.cuda.synchronize()
  want, wacc = O.fast_dot_general(oxq, owq, DN, return_acc=True)
  assert np.array_equal(acc.cpu().numpy(), wacc), 'int32 accumulators differ'
  assert out.dtype == util.TORCH_DT[dtype]
  got = util.f32np(out)
  bad = np.flatnonzero(got.ravel() != want.v.ravel())
  assert bad.size == 0, f'{bad.size} outputs differ: {got.ravel()[bad[:5]]} vs {want.v.ravel()[bad[:5]]}'


@pytest.mark.parametrize('pref', [None, torch.float32, torch.bfloat16])
def test_int8_gemm_mixed_scale_dtypes_and_preferred_type(pref):
  """bf16 lhs scale x f32 rhs scale -> f32 (dot_general_test.py:43-54), preferred type overrides."""
  from qwix_amd.core import dot_general as dg
  xq, wq, oxq, owq = _quantized_pair(64, 256, 128, O.BF16, 'int8', seed=5)
  wq = wq.astype(torch.float32)
  owq = O.QArray(owq.qvalue, owq.scale.astype(O.F32), None, 'int8')
  out = dg.dot_general(xq, wq, DN, preferred_element_type=pref)
  want = O.dot_general(oxq, owq, DN, util.ORACLE_DT[pref] if pref else None)
  assert out.dtype == (pref or torch.float32)
  assert np.array_equal(util.f32np(out), want.v)


def test_raw_int8_operand_stays_on_fast_path():
  from qwix_amd.core import dot_general as dg
  g = util.rng(9)
  a = g.integers(-128, 128, (32, 128), dtype=np.int8)
  xq, wq, oxq, owq = _quantized_pair(32, 128, 64, O.F32, 'int8', seed=6)
  out = dg.dot_general(torch.from_numpy(a).to(util.DEV), wq, DN)
  want = O.dot_general(a, owq, DN)
  assert np.array_equal(util.f32np(out), want.v)


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('M,K,N', [(256, 1024, 512), (100, 320, 60), (1024, 2048, 1024), (16, 1024, 264), (5, 4096, 12300)])
def test_fp8_gemm_close(M, K, N, dtype):
  from qwix_amd.core import dot_general as dg
  print('case fp8', M, K, N, dtype, flush=True)
  xq, wq, oxq, owq = _quantized_pair(M, K, N, dtype, 'float8_e4m3fn', seed=M + K)
  out = dg.dot_general(xq, wq, DN)
  torch.cuda.synchronize()
  want = O.dot_general(oxq, owq, DN)
  assert out.dtype == util.TORCH_DT[dtype]
  got = util.f32np(out)
  tol = 1e-2 if dtype == O.BF16 else 1e-3
  scale = np.abs(want.v).mean()
  assert np.allclose(got, want.v, rtol=tol, atol=tol * scale), np.abs(got - want.v).max()
  if dtype == O.F32:
    assert np.abs(got - want.v).max() <= 3e-4 * np.abs(want.v).max()


def test_gemm_linearity_full_size_property():
  """Size-independent check at the benchmark shape: int32 accumulators are linear in the lhs rows
  and match a float64 product on sampled rows."""
  from qwix_amd.core import dot_general as dg
  g = util.rng(77)
  M = N = K = 4096
  a = torch.from_numpy(g.integers(-127, 128, (M, K), dtype=np.int8)).to(util.DEV)
  b = torch.from_numpy(g.integers(-127, 128, (K, N), dtype=np.int8))
  b_nk = b.t().contiguous().to(util.DEV)
  from qwix_amd import _lib
  acc = torch.empty(M, N, dtype=torch.int32, device=util.DEV)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), K, b_nk.data_ptr(), K, _lib.INT8, M, N, K, None, 0, None, 0, 0,
            acc.data_ptr(), _lib.I32, N, _lib.stream_of(a))
  torch.cuda.synchronize()
  rows = g.choice(M, 16, replace=False)
  want = a[rows].cpu().numpy().astype(np.float64) @ b.numpy().astype(np.float64)
  assert np.array_equal(acc[rows].cpu().numpy(), want.astype(np.int64))
  # checksum of checksums: sum over all outputs == (column sums of a) . (row sums of b)
  total = acc.to(torch.float64).sum().item()
  want_total = float(a.to(torch.float64).sum(0).cpu().numpy() @ b.numpy().astype(np.float64).sum(1))
  assert total == want_total


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('side', ['lhs', 'rhs'])
@pytest.mark.parametrize('M,K,N', [(256, 1024, 512), (100, 272, 60), (1100, 512, 1300), (3, 64, 5), (8, 256, 200),
                                   (48, 2048, 4608), (100, 1024, 9000), (200, 2048, 4100), (30, 640, 14000)])  # decode batches against wide weights
def test_int8_gemm_with_zero_point_operand_bit_exact(M, K, N, side, dtype):
  """One asymmetric (minmax) operand: the int32 correction dot(zp, q_other) of dot_general.py:228-253 is
  subtracted before scaling, so the output is again an elementwise function of exact integers."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  print('case zp', side, M, K, N, dtype, flush=True)
  x_np, x_t = util.make((M, K), dtype, seed=M + 3 * N)
  w_np, w_t = util.make((K, N), dtype, seed=M + 3 * N + 1, scale=0.02)
  x_np = x_np + np.float32(0.75)          # shift the ranges so that the zero points are far from 0
  x_t = x_t + 0.75
  x_np = util.f32np(x_t)
  lkw = dict(qtype='int8', channelwise_axes=[0], calibration_method='minmax' if side == 'lhs' else 'absmax')
  rkw = dict(qtype='int8', channelwise_axes=[1], calibration_method='minmax' if side == 'rhs' else 'absmax')
  xq = qarray.quantize(x_t, qarray.HowToQuantize(**lkw))
  wq = qarray.quantize(w_t, qarray.HowToQuantize(**rkw))
  oxq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(**lkw))
  owq = O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(**rkw))
  util.assert_qarray_equal(xq, oxq, 'lhs')
  util.assert_qarray_equal(wq, owq, 'rhs')
  assert (xq.zero_point is not None) == (side == 'lhs') and (wq.zero_point is not None) == (side == 'rhs')
  out = dg.dot_general(xq, wq, DN)
  torch.cuda.synchronize()
  want = O.dot_general(oxq, owq, DN)
  got = util.f32np(out)
  bad = np.flatnonzero(got.ravel() != want.v.ravel())
  assert bad.size == 0, f'{bad.size} outputs differ: {got.ravel()[bad[:5]]} vs {want.v.ravel()[bad[:5]]}'
  # and it means what it should: close to the float product
  ref = x_np.astype(np.float64) @ w_np.astype(np.float64)
  if K >= 256:
    assert np.abs(got - ref).mean() / np.abs(ref).mean() < 0.05


@pytest.mark.parametrize('tile', [None, 128])
def test_weight_k_sums_are_kept_per_weight_and_follow_in_place_updates(tile):
  """The K-sums of a static weight (the other factor of an asymmetric activation's correction term) are computed once
  per weight tensor; a weight changed in place (same tensor object, new contents) gets new sums."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  x_np, x_t = util.make((64, 256), O.BF16, seed=71)
  x_t = x_t + 0.75
  x_np = util.f32np(x_t)
  w_np, w_t = util.make((256, 136), O.BF16, seed=72, scale=0.02)
  lkw = dict(qtype='int8', channelwise_axes=[0], tiled_axes={1: tile} if tile else {}, calibration_method='minmax')
  rkw = dict(qtype='int8', channelwise_axes=[1], tiled_axes={0: tile} if tile else {})
  xq, oxq = qarray.quantize(x_t, qarray.HowToQuantize(**lkw)), O.quantize(O.FArr(x_np, O.BF16), O.HowToQuantize(**lkw))
  wq, owq = qarray.quantize(w_t, qarray.HowToQuantize(**rkw)), O.quantize(O.FArr(w_np, O.BF16), O.HowToQuantize(**rkw))
  calls = []
  real = dg._lib.call
  def counting(name, *a):
    calls.append(name)
    return real(name, *a)
  dg._lib.call = counting
  try:
    first = util.f32np(dg.dot_general(xq, wq, DN, exact=True))
    again = util.f32np(dg.dot_general(xq, wq, DN, exact=True))
    n_sums = sum(c.startswith('qwix_hip_ksum') for c in calls)
    wq.qvalue.neg_()                                          # in place: same tensor, other values
    owq2 = O.QArray(-owq.qvalue, owq.scale, None, owq.qtype)
    third = util.f32np(dg.dot_general(xq, wq, DN, exact=True))
  finally:
    dg._lib.call = real
  assert n_sums == 1, calls
  assert sum(c.startswith('qwix_hip_ksum') for c in calls) == 2
  assert np.array_equal(first, O.dot_general(oxq, owq, DN).v) and np.array_equal(again, first)
  assert np.array_equal(third, O.dot_general(oxq, owq2, DN).v)


def test_both_operands_asymmetric_is_an_error():
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  _, x_t = util.make((32, 64), O.F32, seed=1)
  _, w_t = util.make((64, 32), O.F32, seed=2)
  xq = qarray.quantize(x_t, qarray.HowToQuantize(qtype='int8', channelwise_axes=[0], calibration_method='minmax'))
  wq = qarray.quantize(w_t, qarray.HowToQuantize(qtype='int8', channelwise_axes=[1], calibration_method='minmax'))
  with pytest.raises(ValueError, match='Only one operand can be asymmetric'):
    dg.dot_general(xq, wq, DN)


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('M,K,N', [(1, 2048, 1024), (5, 128, 48), (16, 1024, 520), (17, 2048, 300), (32, 1536, 14336), (8, 640, 264)])
def test_fused_activation_quantize_gemm_bit_exact(M, K, N, dtype):
  """Activation quantization folded into the decode GEMM == quantize, then dot_general (the oracle's two steps)."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  print('case fused act', M, K, N, dtype, flush=True)
  x_np, x_t = util.make((M, K), dtype, seed=M + K)
  x_np[0, :] *= 0 if M > 4 else 1          # an all-zero row takes the scale guard
  x_t = util.to_gpu(x_np, dtype)
  w_np, w_t = util.make((K, N), dtype, seed=N, scale=0.02)
  wq = qarray.quantize(w_t, qarray.HowToQuantize(qtype='int8', channelwise_axes=[1]))
  out = dg.fused_act_dot_general(x_t, wq, DN)
  assert out is not None and out.dtype == util.TORCH_DT[dtype]
  torch.cuda.synchronize()
  oxq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  owq = O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(qtype='int8', channelwise_axes=[1]))
  want = O.fast_dot_general(oxq, owq, DN)
  got = util.f32np(out)
  bad = np.flatnonzero(got.ravel() != want.v.ravel())
  assert bad.size == 0, f'{bad.size} outputs differ: {got.ravel()[bad[:5]]} vs {want.v.ravel()[bad[:5]]}'
  # operands of another kind are handed back to the two-step route
  w4 = qarray.quantize(torch.zeros(256, 64, device=util.DEV), qarray.HowToQuantize(qtype='int4', channelwise_axes=[1]))
  assert dg.fused_act_dot_general(torch.zeros(8, 256, device=util.DEV), w4, DN) is None
  assert dg.fused_act_dot_general(x_t, wq, DN, act_qtype='float8_e4m3fn') is None   # weight is int8


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('qtype', ['int8', 'float8_e4m3fn'])
@pytest.mark.parametrize('M,K,N', [(40, 2048, 520), (8, 4096, 264), (300, 1024, 1000), (512, 4096, 250), (1024, 512, 2048),
                                   (3, 20000, 64), (2048, 2048, 2048)])
def test_dynamic_activation_gemm_in_one_call_bit_exact(M, K, N, qtype, dtype):
  """qwix_hip_qgemm_dynamic_act at sizes beyond the one-launch kernel (the quantize kernel and the GEMM back to
  back on one scratch buffer; split-K shapes and rows too long for one workgroup included) == the oracle's
  quantize followed by its fast dot_general, bit for bit with int8; with e4m3 the f32 accumulation order is the
  kernel's, so the library's own two-step result is the bit-exact reference and the oracle the tolerance one."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  print('case dynamic act', M, K, N, qtype, dtype, flush=True)
  x_np, x_t = util.make((M, K), dtype, seed=M + K + 1)
  x_np[M // 2, :] = 0                        # an all-zero row takes the scale guard
  x_t = util.to_gpu(x_np, dtype)
  w_np, w_t = util.make((K, N), dtype, seed=N + 3, scale=0.02)
  wq = qarray.quantize(w_t, qarray.HowToQuantize(qtype=qtype, channelwise_axes=[1]))
  out = dg.fused_act_dot_general(x_t, wq, DN, act_qtype=qtype)
  assert out is not None and out.dtype == util.TORCH_DT[dtype]
  xq = qarray.quantize(x_t, qarray.HowToQuantize(qtype=qtype, channelwise_axes=[0]))
  two_step = dg.dot_general(xq, wq, DN)
  assert torch.equal(out, two_step)
  oxq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(qtype=qtype, channelwise_axes=[0]))
  owq = O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(qtype=qtype, channelwise_axes=[1]))
  want = O.fast_dot_general(oxq, owq, DN)
  got = util.f32np(out)
  if qtype == 'int8':
    bad = np.flatnonzero(got.ravel() != want.v.ravel())
    assert bad.size == 0, f'{bad.size} outputs differ: {got.ravel()[bad[:5]]} vs {want.v.ravel()[bad[:5]]}'
  else:
    # e4m3 accumulates in f32 in the kernel's own order; with a bf16 result the accumulator and both scalings
    # are rounded to bf16 in turn, so a last-bit difference of the f32 sum can move the result by two bf16 steps
    # (2^-6): that bounds every element, and all but 1 in 10^4 must meet the 1e-2 bar.
    tol = 1e-2 if dtype == O.BF16 else 1e-3
    atol = tol * float(np.abs(want.v).mean())
    err = np.abs(got - want.v)
    assert np.all(err <= (2.0 ** -6 if dtype == O.BF16 else tol) * np.abs(want.v) + atol), err.max()
    assert np.mean(err <= tol * np.abs(want.v) + atol) >= 1 - 1e-4


def test_dynamic_activation_gemm_argument_checks():
  """The one-call entry point refuses a missing or short scratch buffer and strided rows with an error code and
  a message instead of launching."""
  from qwix_amd import _lib
  L = _lib.load()
  M, N, K = 64, 128, 256
  x = torch.zeros(M, K, dtype=torch.bfloat16, device=util.DEV)
  b = torch.zeros(N, K, dtype=torch.int8, device=util.DEV)
  sb = torch.ones(N, dtype=torch.bfloat16, device=util.DEV)
  out = torch.empty(M, N, dtype=torch.bfloat16, device=util.DEV)
  need = L.qwix_hip_qgemm_dynamic_act_workspace_bytes(M, N, K, _lib.BF16)
  assert need >= M * K + 2 * M
  ws = torch.empty(need, dtype=torch.uint8, device=util.DEV)
  args = lambda ldx, wsp, nws: (x.data_ptr(), _lib.BF16, ldx, b.data_ptr(), K, _lib.INT8, M, N, K, sb.data_ptr(), _lib.BF16, 0,
                                out.data_ptr(), _lib.BF16, N, wsp, nws, None)
  assert L.qwix_hip_qgemm_dynamic_act(*args(K, ws.data_ptr(), need)) == 0
  assert L.qwix_hip_qgemm_dynamic_act(*args(K, None, 0)) != 0
  assert b'workspace' in L.qwix_hip_last_error()
  assert L.qwix_hip_qgemm_dynamic_act(*args(K, ws.data_ptr(), need - 1)) != 0
  assert L.qwix_hip_qgemm_dynamic_act(*args(2 * K, ws.data_ptr(), need)) != 0
  assert b'dense' in L.qwix_hip_last_error()
  torch.cuda.synchronize()


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('M,K,N', [(512, 8192, 512), (300, 8192, 520), (384, 14336, 512), (257, 8192, 1000), (512, 16384, 250)])
def test_int8_gemm_split_k_bit_exact(M, K, N, dtype):
  """A few hundred rows against a narrow weight with a long K: the library may cut K into ranges (it reports a
  workspace size for these shapes); int32 partials add exactly, so the result is the oracle's, bit for bit,
  with and without the workspace."""
  from qwix_amd import _lib
  from qwix_amd.core import dot_general as dg
  print('case split-K', M, K, N, dtype, flush=True)
  assert _lib.load().qwix_hip_qgemm_workspace_bytes(M, N, K) > 0
  xq, wq, oxq, owq = _quantized_pair(M, K, N, dtype, 'int8', seed=M + K + N)
  want = O.fast_dot_general(oxq, owq, DN)
  out = dg.dot_general(xq, wq, DN)          # takes the workspace route
  assert np.array_equal(util.f32np(out), want.v)
  # the same call without scratch memory must give the same bits
  c = dg._Canon(xq, wq, DN)
  a, (b, _) = c.lhs_values(xq), c.rhs_values(wq)
  sa, _ = c.lhs_scale(xq)
  sb, _ = c.rhs_scale(wq)
  plain = torch.empty(M, N, dtype=out.dtype, device=util.DEV)
  tag = _lib.float_tag(out.dtype)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), _lib.INT8, M, N, K, sa.data_ptr(),
            _lib.float_tag(sa.dtype), sb.data_ptr(), _lib.float_tag(sb.dtype), 0, plain.data_ptr(), tag, N, _lib.stream_of(a))
  assert torch.equal(plain, out)
  # a workspace that is too small is ignored, not overrun
  small = torch.empty(64, dtype=torch.uint8, device=util.DEV)
  again = torch.empty_like(plain)
  _lib.call('qwix_hip_qgemm_ws', a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), _lib.INT8, M, N, K, sa.data_ptr(),
            _lib.float_tag(sa.dtype), sb.data_ptr(), _lib.float_tag(sb.dtype), 0, again.data_ptr(), tag, N,
            small.data_ptr(), 64, _lib.stream_of(a))
  assert torch.equal(again, out)


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
def test_fp8_gemm_split_k_close(dtype):
  from qwix_amd.core import dot_general as dg
  M, K, N = 512, 8192, 512
  xq, wq, oxq, owq = _quantized_pair(M, K, N, dtype, 'float8_e4m3fn', seed=77)
  out = dg.dot_general(xq, wq, DN)
  want = O.fast_dot_general(oxq, owq, DN)
  tol = 1e-2 if dtype == O.BF16 else 1e-3   # the tolerance of test_fp8_gemm_close
  got = util.f32np(out)
  # (K = 8192: the f32 partial sums of the ranges differ from one f32 sum by up to two bf16 steps of the result)
  assert np.allclose(got, want.v, rtol=tol, atol=tol * np.abs(want.v).max()), np.abs(got - want.v).max()


def test_split_k_is_not_offered_where_it_cannot_pay():
  from qwix_amd import _lib
  f = _lib.load().qwix_hip_qgemm_workspace_bytes
  assert f(4096, 4096, 4096) == 0      # the tiles already fill the chip
  assert f(16, 4096, 4096) == 0        # decode sizes stream the weight
  assert f(256, 1024, 512) == 0        # too few slabs to cut
  assert f(256, 4096, 1024) == 0       # a short K (M, N, K = 256, 4096, 1024): the second launch costs more than it saves
  assert f(256, 1024, 4096) == 0       # 64 x 64 tiles with four slab stages take it faster unsplit
  assert f(256, 256, 4096) == 0        # the weight-streaming kernel takes it
  assert f(256, 1024, 4100) == 0       # K not a multiple of 128 (M, N, K)
