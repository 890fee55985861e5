"""GPU parity: sub-channel (K-group) GEMM and the weight-only skinny GEMM vs the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import qwix_oracle as O
from tests import util

pytestmark = pytest.mark.gpu
DN = (((1,), (0,)), ((), ()))


def _pair(M, K, N, dtype, wq_type, group, seed, lhs_tile=None, layout=None):
  from qwix_amd.core import qarray
  x_np, x_t = util.make((M, K), dtype, seed=seed)
  w_np, w_t = util.make((K, N), dtype, seed=seed + 1, scale=0.02)
  lkw = dict(qtype='int8', channelwise_axes=[0])
  if lhs_tile:
    lkw['tiled_axes'] = {1: lhs_tile}
  rkw = dict(qtype=wq_type, channelwise_axes=[1])
  if group:
    rkw['tiled_axes'] = {0: group}
  xq = qarray.quantize(x_t, qarray.HowToQuantize(**lkw))
  wq = qarray.quantize(w_t, qarray.HowToQuantize(**rkw), layout=layout)
  oxq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(**lkw))
  owq = O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(**rkw))
  util.assert_qarray_equal(xq, oxq, 'lhs')
  util.assert_qarray_equal(wq, owq, 'rhs')
  return xq, wq, oxq, owq, x_np, w_np


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('wq_type', ['int4', 'int8'])
@pytest.mark.parametrize('M,K,N,group', [(64, 256, 128, 128), (200, 512, 264, 128), (128, 1024, 256, 256), (300, 384, 520, 128)])
def test_grouped_gemm_exact_mode_is_bit_exact(M, K, N, group, wq_type, dtype):
  from qwix_amd.core import dot_general as dg
  print('case grouped', M, K, N, group, wq_type, dtype, flush=True)
  xq, wq, oxq, owq, _, _ = _pair(M, K, N, dtype, wq_type, group, seed=M + N)
  out, acc = dg._fast_dot_general(xq, wq, DN, exact=True, return_accumulators=True)
  torch.cuda.synchronize()
  want, wacc = O.fast_dot_general(oxq, owq, DN, return_acc=True)
  assert np.array_equal(acc.cpu().numpy(), wacc), 'per-group int32 partials differ'
  got = util.f32np(out)
  bad = np.flatnonzero(got.ravel() != want.v.ravel())
  assert bad.size == 0, f'{bad.size} outputs differ: {got.ravel()[bad[:5]]} vs {want.v.ravel()[bad[:5]]}'


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('wq_type', ['int4', 'int8'])
@pytest.mark.parametrize('M,K,N,group', [(256, 1024, 512, 128), (200, 512, 264, 128), (130, 1024, 258, 256),
                                         (520, 768, 1000, 384), (1, 128, 2, 128)])
def test_grouped_gemm_fast_mode_within_tolerance(M, K, N, group, wq_type, dtype):
  """The fast mode keeps the partial sums in f32 (no rounding per partial): it must agree with the exact
  integer partials combined in float64 to f32 accuracy, and stay inside the envelope of the reference's
  per-partial roundings."""
  from qwix_amd.core import dot_general as dg
  print('case grouped fast', M, K, N, group, wq_type, dtype, flush=True)
  xq, wq, oxq, owq, x_np, w_np = _pair(M, K, N, dtype, wq_type, group, seed=3 + M)
  out = dg.dot_general(xq, wq, DN)
  torch.cuda.synchronize()
  want, wacc = O.fast_dot_general(oxq, owq, DN, return_acc=True)
  got = util.f32np(out)
  assert np.all(np.abs(got - want.v) <= 1e-2 * np.abs(want.v) + util.partials_envelope(wacc, oxq, owq)), np.abs(got - want.v).max()
  # closed form from the integer partials: sum_g acc_g[m,n] * sb[g,n], then * sa[m]
  sa = np.asarray(oxq.scale.v, np.float64).reshape(M, 1)
  sb = np.asarray(owq.scale.v, np.float64).reshape(K // group, 1, N)
  exact = (np.asarray(wacc, np.float64).reshape(K // group, M, N) * sb).sum(0) * sa
  tol = 2.0 ** -7 if dtype is O.BF16 else 1e-5
  scale = np.abs(np.asarray(wacc, np.float64).reshape(K // group, M, N) * sb).sum(0) * sa
  assert np.all(np.abs(got - exact) <= tol * scale + 1e-30), (np.abs(got - exact) / (scale + 1e-30)).max()
  if M >= 128:
    ref = x_np.astype(np.float64) @ w_np.astype(np.float64)
    ceil = 0.12 if wq_type == 'int4' else 0.02   # einsum_test.py ceilings for w4a8 / w8a8
    assert np.abs(got - ref).mean() / np.abs(ref).mean() < ceil * 1.1


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('wq_type', ['int4', 'int8'])
@pytest.mark.parametrize('M,K,N,group', [(256, 1024, 512, 128), (200, 512, 264, 128), (130, 1024, 258, 256), (300, 2048, 1000, 128)])
def test_grouped_gemm_fast_mode_with_per_group_activation_scales(M, K, N, group, wq_type, dtype):
  """Both operands tiled along K (what a rule with tile_size gives): the fast kernel folds group g in as
  acc_g * sa[m, g] * sb[g, n] in f32.  Checked against that closed form built from the oracle's exact integer
  partials, and against the envelope of the reference's per-partial roundings."""
  from qwix_amd.core import dot_general as dg
  print('case grouped fast, both tiled', M, K, N, group, wq_type, dtype, flush=True)
  xq, wq, oxq, owq, x_np, w_np = _pair(M, K, N, dtype, wq_type, group, seed=5 + M, lhs_tile=group)
  out = dg.dot_general(xq, wq, DN)
  torch.cuda.synchronize()
  want, wacc = O.fast_dot_general(oxq, owq, DN, return_acc=True)
  got = util.f32np(out)
  G = K // group
  sa = np.asarray(oxq.scale.v, np.float64).reshape(M, G).T.reshape(G, M, 1)
  sb = np.asarray(owq.scale.v, np.float64).reshape(G, 1, N)
  parts = np.asarray(wacc, np.float64).reshape(G, M, N) * sa * sb
  exact = parts.sum(0)
  tol = 2.0 ** -7 if dtype is O.BF16 else 1e-5
  scale = np.abs(parts).sum(0)
  assert np.all(np.abs(got - exact) <= tol * scale + 1e-30), (np.abs(got - exact) / (scale + 1e-30)).max()
  # the reference rounds every partial to the scale dtype: stay within a few roundings of it
  rt = 2.0 ** -6 if dtype is O.BF16 else 1e-5
  assert np.all(np.abs(got - want.v) <= rt * scale + 1e-30)
  if M >= 128:
    ref = x_np.astype(np.float64) @ w_np.astype(np.float64)
    ceil = 0.12 if wq_type == 'int4' else 0.02
    assert np.abs(got - ref).mean() / np.abs(ref).mean() < ceil * 1.1


def test_both_sides_tiled_and_natural_layout_weight():
  from qwix_amd.core import dot_general as dg
  xq, wq, oxq, owq, _, _ = _pair(96, 512, 128, O.F32, 'int8', 128, seed=9, lhs_tile=128, layout='natural')
  out, acc = dg._fast_dot_general(xq, wq, DN, exact=True, return_accumulators=True)
  want, wacc = O.fast_dot_general(oxq, owq, DN, return_acc=True)
  assert np.array_equal(acc.cpu().numpy(), wacc)
  assert np.array_equal(util.f32np(out), want.v)
  out = dg.dot_general(xq, wq, DN)
  assert np.allclose(util.f32np(out), want.v, rtol=1e-4, atol=1e-5)


def test_per_channel_int4_weight_and_tile_mismatch_error():
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  xq, wq, oxq, owq, _, _ = _pair(64, 256, 128, O.BF16, 'int4', None, seed=12)
  out = dg._fast_dot_general(xq, wq, DN, exact=True)
  want = O.fast_dot_general(oxq, owq, DN)
  assert np.array_equal(util.f32np(out), want.v)
  xq2, _, _, _, _, _ = _pair(64, 512, 128, O.BF16, 'int4', 128, seed=12, lhs_tile=256)
  _, wq2, _, _, _, _ = _pair(64, 512, 128, O.BF16, 'int4', 128, seed=12)
  with pytest.raises(ValueError, match='same tile size'):
    dg._fast_dot_general(xq2, wq2, DN)


@pytest.mark.parametrize('wq_type', ['int4', 'int8', 'float8_e4m3fn'])
@pytest.mark.parametrize('M', [1, 8, 16, 24, 40, 100])
@pytest.mark.parametrize('K,N,group,sdt', [(512, 256, 128, torch.float32), (4096, 1024, 128, torch.float32), (1024, 200, 1024, torch.bfloat16)])
def test_weight_only_gemv(M, K, N, group, sdt, wq_type):
  """The weight-only int4 benchmark configuration at reduced N: bf16 activations x int4 g128 weight, f32 scales, bf16 out;
  the same with int8 and e4m3 weights.  The decode kernel is the one that runs: the operator's fit accepts the pair."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  print('case gemv', M, K, N, group, wq_type, flush=True)
  x_np, x_t = util.make((M, K), O.BF16, seed=M + K)
  w_np, w_t = util.make((K, N), O.BF16, seed=M + K + 1, scale=0.02)
  tiled = {0: group} if group != K else {}
  wq = qarray.quantize_api(w_t, wq_type, channelwise_axes=[1], tiled_axes=tiled, scale_dtype=sdt)
  owq = O.quantize_api(O.FArr(w_np, O.BF16), wq_type, channelwise_axes=[1], tiled_axes=tiled, scale_dtype=util.ORACLE_DT[sdt])
  util.assert_qarray_equal(wq, owq, 'weight')
  assert dg._weight_only_fit(x_t, wq, DN) is not None
  out = dg.dot_general(x_t, wq, DN, preferred_element_type=torch.bfloat16)
  torch.cuda.synchronize()
  want = O.dot_general(O.FArr(x_np, O.BF16), owq, DN, O.BF16)
  assert out.dtype == torch.bfloat16 and tuple(out.shape) == (M, N)
  got = util.f32np(out)
  scale = np.abs(want.v).mean()
  assert np.allclose(got, want.v, rtol=1e-2, atol=1e-2 * scale), np.abs(got - want.v).max()
  # default result type follows the scale dtype (bf16 x f32 -> f32)
  out2 = dg.dot_general(x_t, wq, DN)
  assert out2.dtype == sdt


@pytest.mark.parametrize('sdt', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('wq_type', ['int8', 'float8_e4m3fn'])
@pytest.mark.parametrize('K,N', [(4096, 14336), (8192, 8192)])
def test_weight_only_gemv_large_byte_weights(K, N, wq_type, sdt):
  """Byte weights of 32 MB and more take the decode kernel's four-wavefront configuration with two row tiles (the second
  one empty up to 16 rows): symmetric int8 and e4m3, both scale dtypes, 1 to 32 rows, each against the oracle's
  dequantize-first dot on the same quantized weight.  The weight is quantized once per case; the rows vary inside."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  print('case gemv large', K, N, wq_type, sdt, flush=True)
  w_np, w_t = util.make((K, N), O.BF16, seed=K + N + 11, scale=0.02)
  wq = qarray.quantize_api(w_t, wq_type, channelwise_axes=[1], tiled_axes={0: 128}, scale_dtype=sdt)
  owq = O.quantize_api(O.FArr(w_np, O.BF16), wq_type, channelwise_axes=[1], tiled_axes={0: 128}, scale_dtype=util.ORACLE_DT[sdt])
  util.assert_qarray_equal(wq, owq, 'weight')
  del w_t
  x_np, x_t = util.make((32, K), O.BF16, seed=K + 12)
  want_all = O.dot_general(O.FArr(x_np, O.BF16), owq, DN, O.F32).v
  for M in (1, 8, 16, 32):
    print('  rows', M, flush=True)
    xm = x_t[:M].contiguous()
    assert dg._weight_only_fit(xm, wq, DN) is not None
    out = dg.dot_general(xm, wq, DN, preferred_element_type=torch.float32)
    torch.cuda.synchronize()
    got, want = util.f32np(out), want_all[:M]
    assert got.shape == (M, N)
    # f32 scales: f32 partial sums in another order than the oracle's.  bf16 scales: the oracle rounds every dequantized
    # weight to bf16 (2^-9 relative each) where the kernel keeps q * scale in f32: the tolerance of a bf16 result.
    tol = 1e-3 if sdt == torch.float32 else 1e-2
    assert np.allclose(got, want, rtol=tol, atol=tol * np.abs(want).mean()), np.abs(got - want).max()
    outb = dg.dot_general(xm, wq, DN, preferred_element_type=torch.bfloat16)
    assert np.allclose(util.f32np(outb), want, rtol=1e-2, atol=1e-2 * np.abs(want).mean())


def test_decode_plan_follows_in_place_weight_updates():
  """A natural-layout weight reaches the decode kernel through a re-laid-out copy that is kept per weight object.
  Updating qvalue, scale or zero point in place (same tensors, new contents) must not serve the old copy."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  M, K, N = 8, 512, 384
  x_np, x_t = util.make((M, K), O.BF16, seed=71)
  for wq_type, asym in (('int8', False), ('int4', False), ('int8', True)):
    kw = dict(channelwise_axes=[1], tiled_axes={0: 128})
    if asym:
      kw['calibration_method'] = 'minmax'
    w1_np, w1_t = util.make((K, N), O.BF16, seed=72, scale=0.02)
    w2_np, w2_t = util.make((K, N), O.BF16, seed=73, scale=0.05)
    if asym:
      w2_np = O.round_to_bf16(w2_np + 0.02)
      w2_t = torch.from_numpy(w2_np).to(torch.bfloat16).to(util.DEV)
    wq = qarray.quantize_api(w1_t, wq_type, scale_dtype=torch.float32, layout='natural', **kw)
    wq2 = qarray.quantize_api(w2_t, wq_type, scale_dtype=torch.float32, layout='natural', **kw)
    owq2 = O.quantize_api(O.FArr(w2_np, O.BF16), wq_type, scale_dtype=O.F32, **kw)
    first = dg.dot_general(x_t, wq, DN, preferred_element_type=torch.float32)   # builds and keeps the plan
    assert dg._DECODE_PLANS.get(id(wq)) is not None and dg._DECODE_PLANS[id(wq)][2] is not None
    store = lambda q: q.data if isinstance(q, qarray.Int4Tensor) else q
    store(wq.qvalue).copy_(store(wq2.qvalue))
    wq.scale.copy_(wq2.scale)
    if asym:
      wq.zero_point.copy_(wq2.zero_point)
    out = dg.dot_general(x_t, wq, DN, preferred_element_type=torch.float32)
    torch.cuda.synchronize()
    want = O.dot_general(O.FArr(x_np, O.BF16), owq2, DN, O.F32).v
    got = util.f32np(out)
    assert np.allclose(got, want, rtol=1e-3, atol=1e-3 * np.abs(want).mean()), (wq_type, asym, np.abs(got - want).max())
    assert not torch.allclose(out, first, rtol=1e-2, atol=1e-4)
    # each part on its own: scale only
    wq.scale.mul_(2.0)
    out2 = dg.dot_general(x_t, wq, DN, preferred_element_type=torch.float32)
    torch.cuda.synchronize()
    assert np.allclose(util.f32np(out2), 2.0 * want, rtol=1e-3, atol=2e-3 * np.abs(want).mean()), (wq_type, asym)


@pytest.mark.parametrize('wq_type', ['int4', 'int8'])
@pytest.mark.parametrize('M', [1, 16, 40, 100, 250])
@pytest.mark.parametrize('K,N,group,sdt', [(512, 256, 128, torch.float32), (4224, 1024, 128, torch.bfloat16), (1024, 200, 1024, torch.bfloat16),
                                           (4096, 14336, 128, torch.float32)])
def test_weight_only_gemv_asymmetric_weights(M, K, N, group, sdt, wq_type):
  """bf16 activations x a weight quantized with min/max calibration (zero points per group and column): the decode
  kernel takes the zero point out through the row sums of x.  Against the oracle's dequantize-first dot on the
  same quantized weight, at the tolerance of the symmetric case (250 rows run the dequantizing tile GEMM, which takes
  zero points too)."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  print('case gemv zp', M, K, N, group, wq_type, sdt, flush=True)
  x_np, x_t = util.make((M, K), O.BF16, seed=M + K + 3)
  w_np, w_t = util.make((K, N), O.BF16, seed=M + K + 4, scale=0.02)
  w_np = O.round_to_bf16(w_np + 0.013)   # off-centre, so that the zero points are not all alike
  w_t = torch.from_numpy(w_np).to(torch.bfloat16).to(util.DEV)
  tiled = {0: group} if group != K else {}
  kw = dict(channelwise_axes=[1], tiled_axes=tiled, calibration_method='minmax')
  wq = qarray.quantize_api(w_t, wq_type, scale_dtype=sdt, **kw)
  owq = O.quantize_api(O.FArr(w_np, O.BF16), wq_type, scale_dtype=util.ORACLE_DT[sdt], **kw)
  util.assert_qarray_equal(wq, owq, 'weight')
  assert wq.zero_point is not None and dg._weight_only_fit(x_t, wq, DN) is not None
  out = dg.dot_general(x_t, wq, DN, preferred_element_type=torch.float32)
  torch.cuda.synchronize()
  want = O.dot_general(O.FArr(x_np, O.BF16), owq, DN, O.F32)
  got = util.f32np(out)
  assert np.allclose(got, want.v, rtol=1e-2, atol=1e-2 * np.abs(want.v).mean()), np.abs(got - want.v).max()
  # the same through the two library kernels that dequantize first (what larger batches run)
  two = dg._dequantize_then_bf16_gemm(x_t, wq, DN, torch.float32)
  assert torch.allclose(out, two, rtol=1e-2, atol=1e-2 * float(two.abs().mean()))


@pytest.mark.parametrize('wq_type', ['int4', 'int8', 'float8_e4m3fn'])
@pytest.mark.parametrize('M', [1, 20, 40])
@pytest.mark.parametrize('K,N,group', [(384, 72, 128), (4224, 136, 128), (16384, 264, 256), (8192, 2048, 128), (128, 48, 128)])
def test_weight_only_gemv_k_splits(M, K, N, group, wq_type, monkeypatch):
  """How the wavefronts of the weight-only kernel share K: an odd number of 128-wide blocks (a last, single block
  after the pairs), one block in all, and so many blocks that a wavefront makes several trips (the next pair's
  weights are requested while this pair is multiplied); N that ends inside a column tile.  (The decode kernel at every
  row count: the operator's switch to the dequantizing tile GEMM is held off.)"""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  monkeypatch.setattr(dg, 'fused_wq_min_rows', lambda *args: dg.WEIGHT_ONLY_MAX_ROWS)
  print('case gemv k-split', M, K, N, group, wq_type, flush=True)
  x_np, x_t = util.make((M, K), O.BF16, seed=M + K + 5)
  w_np, w_t = util.make((K, N), O.BF16, seed=N + K + 6, scale=0.02)
  wq = qarray.quantize_api(w_t, wq_type, channelwise_axes=[1], tiled_axes={0: group}, scale_dtype=torch.float32)
  owq = O.quantize_api(O.FArr(w_np, O.BF16), wq_type, channelwise_axes=[1], tiled_axes={0: group}, scale_dtype=O.F32)
  util.assert_qarray_equal(wq, owq, 'weight')
  out = dg.dot_general(x_t, wq, DN, preferred_element_type=torch.float32)
  torch.cuda.synchronize()
  want = O.dot_general(O.FArr(x_np, O.BF16), owq, DN, O.F32)
  got = util.f32np(out)
  # f32 sums in another order than the oracle's: 1e-3 of the typical magnitude
  assert np.allclose(got, want.v, rtol=1e-3, atol=1e-3 * np.abs(want.v).mean()), np.abs(got - want.v).max()


@pytest.mark.parametrize('wq_type', ['int4', 'int8', 'float8_e4m3fn'])
@pytest.mark.parametrize('M,K,N', [(30, 1024, 520), (50, 4096, 14336), (130, 512, 6400)])
def test_weight_only_rows_do_not_depend_on_the_batch(M, K, N, wq_type, monkeypatch):
  """More than 16 rows share a pass over the weights (2 tiles of 16 rows per workgroup, fewer wavefronts
  along K): the f32 partial sums meet in another order, nothing else changes, so the result equals the rows
  computed 16 at a time up to that reordering.  (The decode kernel for the whole batch: the operator's switch to
  the dequantizing tile GEMM, which rounds every weight to bf16 first, is held off.)"""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  monkeypatch.setattr(dg, 'fused_wq_min_rows', lambda *args: dg.WEIGHT_ONLY_MAX_ROWS)
  print('case gemv batch', M, K, N, wq_type, flush=True)
  _, x_t = util.make((M, K), O.BF16, seed=M + K)
  _, w_t = util.make((K, N), O.BF16, seed=M + K + 1, scale=0.02)
  wq = qarray.quantize_api(w_t, wq_type, channelwise_axes=[1], tiled_axes={0: 128}, scale_dtype=torch.float32)
  out = dg.dot_general(x_t, wq, DN, preferred_element_type=torch.float32)
  parts = [dg.dot_general(x_t[i:i + 16].contiguous(), wq, DN, preferred_element_type=torch.float32)
           for i in range(0, M, 16)]
  torch.cuda.synchronize()
  want = torch.cat(parts, 0)
  assert torch.allclose(out, want, rtol=1e-5, atol=1e-5 * want.abs().mean().item())


def _close(got, true, dtype):
  """f32: the 1e-4 of the reference's test; bf16 results carry a rounding per epilogue step: 1 % mean error."""
  if dtype == O.F32:
    return np.allclose(got, true, rtol=1e-4, atol=1e-4)
  return np.abs(got - true).mean() / np.abs(true).mean() < 1e-2


def _two_dim_pair(M, K, N, lt, rt, dtype, seed):
  from qwix_amd.core import qarray
  x_np, x_t = util.make((M, K), dtype, seed=seed)
  w_np, w_t = util.make((K, N), dtype, seed=seed + 1)
  lkw = dict(qtype='int8', tiled_axes={0: lt[0], 1: lt[1]})
  rkw = dict(qtype='int8', tiled_axes={0: rt[0], 1: rt[1]})
  xq = qarray.quantize(x_t, qarray.HowToQuantize(**lkw))
  wq = qarray.quantize(w_t, qarray.HowToQuantize(**rkw))
  oxq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(**lkw))
  owq = O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(**rkw))
  util.assert_qarray_equal(xq, oxq, 'lhs')
  util.assert_qarray_equal(wq, owq, 'rhs')
  return xq, wq, oxq, owq


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
def test_two_dim_scales_small_tiles(dtype):
  """two_dim_scales_test.py:29-93: 8 x 8 tiles on both operands of a 128^3 product.  Tiles below 128 take the
  dequantize-first path; dequantize is bit-exact, and dot_general == dequant . dequant within the 1e-4 the
  reference test asks for."""
  from qwix_amd.core import dot_general as dg, qarray
  xq, wq, oxq, owq = _two_dim_pair(128, 128, 128, (8, 8), (8, 8), dtype, seed=81)
  assert tuple(xq.scale.shape) == (16, 16)
  for got, want in ((qarray.dequantize(xq), O.dequantize(oxq)), (qarray.dequantize(wq), O.dequantize(owq))):
    assert tuple(got.shape) == (128, 128)
    assert np.array_equal(util.f32np(got), want.v)
  true = O.dequantize(oxq).v.astype(np.float64) @ O.dequantize(owq).v.astype(np.float64)
  out = dg.dot_general(xq, wq, DN)
  assert _close(util.f32np(out), true, dtype)
  slow = dg._slow_dot_general(xq, wq, DN)
  assert _close(util.f32np(slow), true, dtype)


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('lt,rt', [((64, 128), (128, 128)), ((32, 128), (128, 64)), ((256, 256), (256, 32))])
def test_two_dim_scales_on_the_quantized_path(lt, rt, dtype):
  """K tiles of at least 128 stay on the quantized path: the scales of the tiled non-contracted axes are
  repeated over their tiles (the reference's generic broadcast), the per-K-tile int32 partials are exact."""
  from qwix_amd.core import dot_general as dg
  xq, wq, oxq, owq = _two_dim_pair(256, 512, 384, lt, rt, dtype, seed=83)
  out, acc = dg._fast_dot_general(xq, wq, DN, exact=True, return_accumulators=True)
  torch.cuda.synchronize()
  want, wacc = O.fast_dot_general(oxq, owq, DN, return_acc=True)
  assert np.array_equal(acc.cpu().numpy(), wacc), 'per-group int32 partials differ'
  assert np.array_equal(util.f32np(out), want.v)
  fast = dg.dot_general(xq, wq, DN)
  true = O.dequantize(oxq).v.astype(np.float64) @ O.dequantize(owq).v.astype(np.float64)
  assert _close(util.f32np(fast), true, dtype)


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('wq_type', ['int4', 'int8'])
@pytest.mark.parametrize('M,K,N,group,lhs_tile', [(256, 1024, 512, 128, None), (200, 512, 264, 128, None),
                                                  (130, 1024, 258, 256, None), (300, 2048, 1000, 128, 128)])
def test_fast_kernel_int32_partials_are_bit_exact(M, K, N, group, lhs_tile, wq_type, dtype):
  """The kernel that serves dot_general by default (global -> LDS slabs, f32 sum of the scaled partials)
  dumps its per-group int32 partials on request: they are the reference's accumulators, bit for bit, and
  the outputs of the run that dumps equal those of the run that does not."""
  from qwix_amd.core import dot_general as dg
  print('case grouped fast acc', M, K, N, group, lhs_tile, wq_type, dtype, flush=True)
  xq, wq, oxq, owq, _, _ = _pair(M, K, N, dtype, wq_type, group, seed=21 + M, lhs_tile=lhs_tile)
  out, acc = dg._fast_dot_general(xq, wq, DN, exact=False, return_accumulators=True)
  plain = dg._fast_dot_general(xq, wq, DN, exact=False)
  torch.cuda.synchronize()
  _, wacc = O.fast_dot_general(oxq, owq, DN, return_acc=True)
  assert np.array_equal(acc.cpu().numpy(), wacc), 'per-group int32 partials of the fast kernel differ'
  _assert_same_up_to_fold_rounding(out, plain, wacc, oxq, owq, dtype)


def _assert_same_up_to_fold_rounding(out, plain, wacc, oxq, owq, dtype):
  """The run that dumps its partials folds them into f32 with convert + FMA; the plain run may use the
  conversion-free fold (bf16 scales, groups of 128), whose running sums carry a constant that costs about
  2^-12 of a partial in f32 rounding.  With f32 scales both runs are the same instantiation: equal bits.
  Otherwise: within one bf16 unit of the output plus 1/16 of the reference's own rounding envelope."""
  if dtype is O.F32:
    assert torch.equal(out, plain)
    return
  a, b = util.f32np(out), util.f32np(plain)
  env = util.partials_envelope(wacc, oxq, owq)
  assert np.all(np.abs(a - b) <= 2.0 ** -7 * np.abs(a) + env / 16), np.abs(a - b).max()


def _zp_pair(M, K, N, dtype, wq_type, group, seed, side, zp_tiled):
  """One asymmetric (minmax) operand; `zp_tiled`: that operand is tiled along K, so its zero point is per group."""
  from qwix_amd.core import qarray
  x_np, x_t = util.make((M, K), dtype, seed=seed, dist='uniform')
  w_np, w_t = util.make((K, N), dtype, seed=seed + 1, scale=0.02)
  w_np = w_np + np.float32(0.01)  # off-centre weights: a zero point that matters
  w_np = O.round_to_bf16(w_np) if dtype is O.BF16 else w_np
  w_t = util.to_gpu(w_np, dtype)
  lkw = dict(qtype='int8', channelwise_axes=[0])
  rkw = dict(qtype=wq_type, channelwise_axes=[1])
  if side == 'lhs':
    lkw['calibration_method'] = 'minmax'
    if zp_tiled:
      lkw['tiled_axes'] = {1: group}
    rkw['tiled_axes'] = {0: group}
  else:
    rkw['calibration_method'] = 'minmax'
    if zp_tiled:
      rkw['tiled_axes'] = {0: group}
    else:
      lkw['tiled_axes'] = {1: group}
  xq = qarray.quantize(x_t, qarray.HowToQuantize(**lkw))
  wq = qarray.quantize(w_t, qarray.HowToQuantize(**rkw))
  oxq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(**lkw))
  owq = O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(**rkw))
  util.assert_qarray_equal(xq, oxq, 'lhs')
  util.assert_qarray_equal(wq, owq, 'rhs')
  return xq, wq, oxq, owq


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('zp_tiled', [True, False])
@pytest.mark.parametrize('side', ['lhs', 'rhs'])
@pytest.mark.parametrize('wq_type', ['int4', 'int8'])
@pytest.mark.parametrize('M,K,N,group', [(200, 512, 264, 128), (130, 1024, 258, 256)])
def test_sub_channel_zero_points_bit_exact(M, K, N, group, wq_type, side, zp_tiled, dtype):
  """A tiled contraction with one asymmetric operand (dot_general.py:196-203, 228-253): the zero point is split
  with the tiles and zero_point x K-sum is subtracted from every tile's partial.  Corrected int32 partials and
  (exact mode) outputs equal the oracle's bit for bit, from both kernels; the default mode stays within the
  envelope of the reference's own per-partial roundings."""
  from qwix_amd.core import dot_general as dg
  print('case grouped zp', M, K, N, group, wq_type, side, zp_tiled, dtype, flush=True)
  xq, wq, oxq, owq = _zp_pair(M, K, N, dtype, wq_type, group, 31 + M, side, zp_tiled)
  want, wacc = O.fast_dot_general(oxq, owq, DN, return_acc=True)
  out, acc = dg._fast_dot_general(xq, wq, DN, exact=True, return_accumulators=True)
  torch.cuda.synchronize()
  assert np.array_equal(acc.cpu().numpy(), wacc), 'corrected partials differ (register-staged kernel)'
  got = util.f32np(out)
  bad = np.flatnonzero(got.ravel() != want.v.ravel())
  assert bad.size == 0, f'{bad.size} outputs differ: {got.ravel()[bad[:5]]} vs {want.v.ravel()[bad[:5]]}'
  out, acc = dg._fast_dot_general(xq, wq, DN, exact=False, return_accumulators=True)
  plain = dg.dot_general(xq, wq, DN)   # the dispatcher sends the pair to the quantized path, as the reference does
  torch.cuda.synchronize()
  assert np.array_equal(acc.cpu().numpy(), wacc), 'corrected partials differ (global -> LDS kernel)'
  assert torch.equal(out, plain)   # asymmetric operands: one instantiation serves both runs
  G = K // group
  sa = np.asarray(oxq.scale.v, np.float64)
  sa = sa.reshape(M, -1).T.reshape(-1, M, 1)               # (1 or G, M, 1)
  sb = np.asarray(owq.scale.v, np.float64).reshape(-1, 1, N)  # (1 or G, 1, N)
  parts = np.asarray(wacc, np.float64).reshape(G, M, N) * sa * sb
  rt = 2.0 ** -6 if dtype is O.BF16 else 1e-5
  assert np.all(np.abs(util.f32np(plain) - want.v) <= rt * np.abs(parts).sum(0) + 1e-30)


@pytest.mark.parametrize('out_dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('M,K,N', [(64, 64, 64), (300, 448, 200), (512, 2048, 1024), (4096, 512, 4096), (2048, 256, 14336)])
def test_bf16_gemm_against_float64(M, K, N, out_dtype):
  """qwix_hip_gemm_bf16 through the C ABI: bf16 operands are exact in f64, so the product against numpy's f64
  matmul bounds the kernel's f32 accumulation (and the one bf16 rounding of the result)."""
  from qwix_amd import _lib
  print('case bf16 gemm', M, K, N, out_dtype, flush=True)
  a_np, a = util.make((M, K), O.BF16, seed=M + N)
  b_np, b = util.make((N, K), O.BF16, seed=M + N + 1)
  out = torch.full((M, N), float('nan'), dtype=out_dtype, device=util.DEV)
  _lib.call('qwix_hip_gemm_bf16', a.data_ptr(), K, b.data_ptr(), K, M, N, K, out.data_ptr(), _lib.float_tag(out_dtype),
            N, _lib.stream_of(a))
  torch.cuda.synchronize()
  want = a_np.astype(np.float64) @ b_np.astype(np.float64).T
  got = util.f32np(out).astype(np.float64)
  mag = np.abs(a_np).astype(np.float64) @ np.abs(b_np).astype(np.float64).T   # sum of |products|
  tol = 2.0 ** -18 * mag + (2.0 ** -8 * np.abs(want) if out_dtype == torch.bfloat16 else 0)
  assert np.all(np.abs(got - want) <= tol + 1e-30), (np.abs(got - want) / (tol + 1e-30)).max()


@pytest.mark.parametrize('sdt', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('out_dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('wq_type,asym', [('int4', False), ('int4', True), ('int8', False), ('int8', True),
                                          ('float8_e4m3fn', False)])
@pytest.mark.parametrize('M,K,N,group', [(300, 256, 136, 128), (512, 1024, 1000, 256), (257, 2048, 520, 64), (2048, 4096, 1536, 128),
                                         (1, 512, 64, 512), (600, 512, 8400, 128), (1100, 256, 4100, 64), (100, 1024, 520, 128),
                                         (128, 512, 200, 64), (130, 512, 40, 128), (7, 768, 24, 256),
                                         (64, 256, 72, 64), (96, 4096, 200, 128), (33, 1280, 64, 128)])
def test_prefill_gemm_dequantizes_in_the_kernel(M, K, N, group, asym, wq_type, out_dtype, sdt):
  """qwix_hip_gemm_bf16_wq through the C ABI == qwix_hip_dequantize_rm (to bf16) + qwix_hip_gemm_bf16, bit for bit: the
  same bf16 weights, the same MFMA, K walked in the same order; int4, int8 (with and without zero points) and e4m3 weights,
  edges in M and N, one slab group (64), several; the last two shapes have more than 128 tiles of 256 x 128 and run those, the others tiles of
  256 x 64."""
  from qwix_amd import _lib
  from qwix_amd.core import qarray
  print('case wq prefill', M, K, N, group, asym, wq_type, out_dtype, sdt, flush=True)
  x_np, x_t = util.make((M, K), O.BF16, seed=M + K + 21)
  w_np, w_t = util.make((K, N), O.BF16, seed=N + K + 22, scale=0.02)
  kw = dict(calibration_method='minmax') if asym else {}
  if asym:
    w_t = (w_t.float() + 0.013).to(torch.bfloat16)  # off-centre: zero points that differ
  wq = qarray.quantize_api(w_t, wq_type, channelwise_axes=[1], tiled_axes={0: group}, scale_dtype=sdt, **kw)
  from qwix_amd.core import dot_general as dg
  c = dg._Canon(x_t, wq, DN)
  b, is4 = c.rhs_values(wq)
  sb, gb = c.rhs_scale(wq)
  assert is4 == (wq_type == 'int4') and gb == K // group
  from qwix_amd.core import numerics
  tag = numerics.qtype_tag(wq_type)
  st = _lib.stream_of(x_t)
  zp = dg._rhs_zero_point_i8(c, wq)[0] if asym else None
  assert (wq.zero_point is not None) == asym
  w = torch.empty(N, K, dtype=torch.bfloat16, device=util.DEV)
  _lib.call('qwix_hip_dequantize_rm', b.data_ptr(), tag, 1, K, N, group, sb.data_ptr(), _lib.ptr(zp), _lib.float_tag(sb.dtype),
            w.data_ptr(), _lib.BF16, st)
  want = torch.empty(M, N, dtype=out_dtype, device=util.DEV)
  _lib.call('qwix_hip_gemm_bf16', x_t.data_ptr(), K, w.data_ptr(), K, M, N, K, want.data_ptr(), _lib.float_tag(out_dtype), N, st)
  got = torch.full((M, N), float('nan'), dtype=out_dtype, device=util.DEV)
  _lib.call('qwix_hip_gemm_bf16_wq', x_t.data_ptr(), K, b.data_ptr(), b.stride(0), tag, M, N, K, group, sb.data_ptr(),
            _lib.float_tag(sb.dtype), _lib.ptr(zp), got.data_ptr(), _lib.float_tag(out_dtype), N, st)
  torch.cuda.synchronize()
  assert torch.equal(got, want), float((got.float() - want.float()).abs().max())
  # and against float64 on the dequantized weight
  ref = x_t.double() @ w.double().T
  assert torch.allclose(got.double(), ref, rtol=1e-2 if out_dtype == torch.bfloat16 else 1e-4, atol=1e-2 * float(ref.abs().mean()))


@pytest.mark.parametrize('wq_type', ['int4', 'int8', 'float8_e4m3fn'])
@pytest.mark.parametrize('M', [512, 2048])
def test_prefill_with_f32_scales_stays_within_a_bf16_rounding_of_the_f32_contraction(M, wq_type):
  """bf16 activations x weight with f32 scales, f32 result, above the decode batch: the reference contracts the
  dequantized weight in f32 (dot_general.py:264-275); here the dequantized weight is rounded to bf16 for the bf16
  matrix cores (512 rows: inside the GEMM; 2048 rows: dequantize + GEMM).  One rounding of 2^-9 relative per weight, K
  = 4096 of them per output with independent signs: the mean deviation must stay below 2^-9 of the mean magnitude
  and every element inside the 1e-2 of a bf16 result."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  K, N = 4096, 1024
  print('case prefill f32 scales', M, wq_type, flush=True)
  x_np, x_t = util.make((M, K), O.BF16, seed=M + 31)
  w_np, w_t = util.make((K, N), O.BF16, seed=M + 32, scale=0.02)
  wq = qarray.quantize_api(w_t, wq_type, channelwise_axes=[1], tiled_axes={0: 128}, scale_dtype=torch.float32)
  owq = O.quantize_api(O.FArr(w_np, O.BF16), wq_type, channelwise_axes=[1], tiled_axes={0: 128}, scale_dtype=O.F32)
  util.assert_qarray_equal(wq, owq, 'weight')
  out = dg.dot_general(x_t, wq, DN, preferred_element_type=torch.float32)
  torch.cuda.synchronize()
  assert out.dtype == torch.float32
  want = O.dot_general(O.FArr(x_np, O.BF16), owq, DN, O.F32).v
  got = util.f32np(out)
  mag = np.abs(want).mean()
  assert np.abs(got - want).mean() < 2.0 ** -9 * mag, np.abs(got - want).mean() / mag
  assert np.allclose(got, want, rtol=1e-2, atol=1e-2 * mag), np.abs(got - want).max() / mag


@pytest.mark.parametrize('sdt', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('out_dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('wq_type,asym', [('int4', False), ('int4', True), ('int8', False), ('int8', True),
                                          ('float8_e4m3fn', False)])
@pytest.mark.parametrize('M,K,N,group,splits', [(128, 4096, 1024, 128, 4), (96, 14336, 520, 128, 14), (300, 2048, 136, 64, 2),
                                                (512, 4096, 1000, 256, 4), (64, 8192, 264, 512, 8), (130, 3072, 72, 1024, 3),
                                                (128, 4096, 1024, 4096, 4), (64, 4096, 520, 2048, 4), (200, 6144, 136, 3072, 6),
                                                (2048, 4096, 1536, 128, 0), (64, 1024, 64, 128, 0)])
def test_prefill_gemm_k_ranges(M, K, N, group, splits, asym, wq_type, out_dtype, sdt):
  """qwix_hip_gemm_bf16_wq_ws: K in `splits` ranges with f32 partials in a workspace while the tiles are few (edges in
  M and N, groups of 64 to 1024 in whole numbers per range, groups of 2048 to K (one scale per column) that hold several
  ranges, ranges of 1024 elements and more).  Against the unsplit kernel: another order of the
  f32 sums, so equal to 2^-18 of the mean magnitude (plus one bf16 step, 2^-7 relative, for bf16 results); with no workspace, and
  for shapes that are not split (workspace size 0), the very same bits."""
  from qwix_amd import _lib
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import numerics
  from qwix_amd.core import qarray
  print('case wq k ranges', M, K, N, group, splits, asym, wq_type, out_dtype, sdt, flush=True)
  x_np, x_t = util.make((M, K), O.BF16, seed=M + K + 41)
  w_np, w_t = util.make((K, N), O.BF16, seed=N + K + 42, scale=0.02)
  kw = dict(calibration_method='minmax') if asym else {}
  if asym:
    w_t = (w_t.float() + 0.013).to(torch.bfloat16)
  wq = qarray.quantize_api(w_t, wq_type, channelwise_axes=[1], tiled_axes={0: group}, scale_dtype=sdt, **kw)
  c = dg._Canon(x_t, wq, DN)
  b, _ = c.rhs_values(wq)
  sb, gb = c.rhs_scale(wq)
  assert gb == K // group
  tag = numerics.qtype_tag(wq_type)
  st = _lib.stream_of(x_t)
  zp = dg._rhs_zero_point_i8(c, wq)[0] if asym else None
  nws = int(_lib.load().qwix_hip_gemm_bf16_wq_workspace_bytes(M, N, K, group))
  assert nws == splits * M * N * 4
  want = torch.empty(M, N, dtype=out_dtype, device=util.DEV)
  _lib.call('qwix_hip_gemm_bf16_wq', x_t.data_ptr(), K, b.data_ptr(), b.stride(0), tag, M, N, K, group, sb.data_ptr(),
            _lib.float_tag(sb.dtype), _lib.ptr(zp), want.data_ptr(), _lib.float_tag(out_dtype), N, st)

  def run(ws, n):
    got = torch.full((M, N), float('nan'), dtype=out_dtype, device=util.DEV)
    _lib.call('qwix_hip_gemm_bf16_wq_ws', x_t.data_ptr(), K, b.data_ptr(), b.stride(0), tag, M, N, K, group,
              sb.data_ptr(), _lib.float_tag(sb.dtype), _lib.ptr(zp), got.data_ptr(), _lib.float_tag(out_dtype), N,
              _lib.ptr(ws), n, st)
    torch.cuda.synchronize()
    return got

  assert torch.equal(run(None, 0), want)
  if not splits:
    return
  ws = torch.full((nws,), 0xFF, dtype=torch.uint8, device=util.DEV)  # NaN patterns: every partial must be written
  assert torch.equal(run(ws, nws - 1), want)  # too small a workspace: not split
  got = util.f32np(run(ws, nws))
  ref = util.f32np(want)
  mag = np.abs(ref).mean()
  tol = 2.0 ** -18 * mag * np.sqrt(K / 1024) + (2.0 ** -7 * np.abs(ref) if out_dtype == torch.bfloat16 else 0)
  assert np.all(np.abs(got - ref) <= tol + 1e-30), (np.abs(got - ref) / (tol + 1e-30)).max()
  # and through the operator, which passes the workspace
  res = dg._dequantize_then_bf16_gemm(x_t, wq, DN, out_dtype, fused_only=True)
  assert res is not None and np.array_equal(util.f32np(res), got)


def test_dequantizing_gemm_argument_checks():
  """qwix_hip_gemm_bf16_wq refuses what its tile loop cannot walk (K not in whole groups of four slabs, groups that
  are not whole slabs, unaligned rows, other weight types) with an error code and a message instead of launching."""
  from qwix_amd import _lib
  L = _lib.load()
  M, N, K = 64, 128, 512
  x = torch.zeros(M, K, dtype=torch.bfloat16, device=util.DEV)
  q = torch.zeros(N, K, dtype=torch.int8, device=util.DEV)
  s = torch.ones(K // 128, N, dtype=torch.bfloat16, device=util.DEV)
  out = torch.empty(M, N, dtype=torch.bfloat16, device=util.DEV)
  def call(lda=K, ldq=K, qt=_lib.INT8, k=K, group=128, sd=_lib.BF16, od=_lib.BF16, ldo=N):
    return L.qwix_hip_gemm_bf16_wq(x.data_ptr(), lda, q.data_ptr(), ldq, qt, M, N, k, group, s.data_ptr(), sd, None,
                                   out.data_ptr(), od, ldo, None)
  assert call() == 0
  assert call(qt=_lib.INT4, ldq=K // 2) == 0
  assert call(qt=_lib.E4M3) == 0 and call(qt=7) != 0 and b'int4, int8 or e4m3' in L.qwix_hip_last_error()
  assert call(k=384) != 0 and b'multiple of 256' in L.qwix_hip_last_error()
  assert call(group=96) != 0 and b'multiple of 64' in L.qwix_hip_last_error()
  assert call(ldq=K // 2) != 0 and b'aligned' in L.qwix_hip_last_error()       # int8 rows need K bytes
  assert call(lda=K + 4) != 0
  assert call(ldo=N - 8) != 0 and b'leading dimension' in L.qwix_hip_last_error()
  assert call(od=99) != 0 and call(sd=99) != 0
  torch.cuda.synchronize()


def test_decode_kernel_argument_checks():
  """qwix_hip_gemv_wq / qwix_hip_gemv_wq_zp refuse other weight types, zero points for float weights, K or groups that
  are not whole 128-wide blocks and unaligned rows, with an error code and a message instead of launching."""
  from qwix_amd import _lib
  L = _lib.load()
  M, N, K = 8, 64, 512
  x = torch.zeros(M, K, dtype=torch.bfloat16, device=util.DEV)
  q = torch.zeros(N, K, dtype=torch.int8, device=util.DEV)
  s = torch.ones(K // 128, N, dtype=torch.bfloat16, device=util.DEV)
  z = torch.zeros(K // 128, N, dtype=torch.int8, device=util.DEV)
  out = torch.empty(M, N, dtype=torch.bfloat16, device=util.DEV)
  def call(qt=_lib.INT8, k=K, group=128, ldb=K, zp=False):
    if zp:
      return L.qwix_hip_gemv_wq_zp(x.data_ptr(), K, q.data_ptr(), ldb, qt, M, N, k, group, s.data_ptr(), _lib.BF16,
                                   z.data_ptr(), out.data_ptr(), _lib.BF16, N, None)
    return L.qwix_hip_gemv_wq(x.data_ptr(), K, q.data_ptr(), ldb, qt, M, N, k, group, s.data_ptr(), _lib.BF16,
                              out.data_ptr(), _lib.BF16, N, None)
  assert call() == 0 and call(qt=_lib.E4M3) == 0 and call(qt=_lib.INT4, ldb=K // 2) == 0 and call(zp=True) == 0
  assert call(qt=7) != 0 and b'int4, int8 or e4m3' in L.qwix_hip_last_error()
  assert call(qt=_lib.E4M3, zp=True) != 0 and b'no zero point' in L.qwix_hip_last_error()
  assert call(k=448) != 0 and b'multiples of 128' in L.qwix_hip_last_error()
  assert call(group=192) != 0
  assert call(ldb=K - 16) != 0 and b'aligned' in L.qwix_hip_last_error()
  torch.cuda.synchronize()


@pytest.mark.parametrize('case', [('int4', 128, False, torch.float32), ('int8', 128, False, torch.bfloat16),
                                  ('int4', 256, True, torch.bfloat16), ('int8', None, True, torch.float32),
                                  ('float8_e4m3fn', None, False, torch.bfloat16)])
@pytest.mark.parametrize('M,K,N', [(64, 512, 384), (208, 512, 384), (512, 1024, 1024), (2048, 4096, 1536)])
def test_weight_only_prefill_on_hip_kernels(M, K, N, case):
  """bf16 activations x quantized weight beyond the decode batch: dequantize into a K-contiguous bf16 array, then
  the bf16 MFMA GEMM -- both this library's kernels.  The dequantized operand equals the oracle's dequantize bit
  for bit (bf16 scales) or after one bf16 rounding (f32 scales); the result is compared with the oracle's
  dequantize-first dot (f64 accumulate) at the tolerance of the weight-only configuration, rtol 1e-2."""
  from qwix_amd import _lib
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  wq_type, group, asym, sdt = case
  print('case weight-only prefill', M, K, N, case, flush=True)
  x_np, x_t = util.make((M, K), O.BF16, seed=M + K)
  w_np, w_t = util.make((K, N), O.BF16, seed=M + K + 1, scale=0.02)
  kw = dict(channelwise_axes=[1], tiled_axes={0: group} if group else {}, scale_dtype=sdt)
  okw = dict(channelwise_axes=[1], tiled_axes={0: group} if group else {}, scale_dtype=util.ORACLE_DT[sdt])
  if asym:
    kw['calibration_method'] = okw['calibration_method'] = 'minmax'
  wq = qarray.quantize_api(w_t, wq_type, **kw)
  owq = O.quantize_api(O.FArr(w_np, O.BF16), wq_type, **okw)
  util.assert_qarray_equal(wq, owq, 'weight')
  # every one of these pairs is of the decode kernel's kind; it is bypassed by the row count
  assert dg._weight_only_fit(x_t, wq, DN) is not None
  out = dg._dequantize_then_bf16_gemm(x_t, wq, DN, torch.bfloat16)
  assert out is not None and out.dtype == torch.bfloat16
  torch.cuda.synchronize()
  want = O.dot_general(O.FArr(x_np, O.BF16), owq, DN, O.BF16)
  got = util.f32np(out)
  assert np.allclose(got, want.v, rtol=1e-2, atol=1e-2 * np.abs(want.v).mean()), np.abs(got - want.v).max()
  # the operator takes this path from the row count on at which the dequantizing tile GEMM beats the decode kernel
  if M > dg.fused_wq_min_rows(N, wq_type == 'int4', K, group or K):
    assert torch.equal(dg.dot_general(x_t, wq, DN, preferred_element_type=torch.bfloat16), out)
  # the dequantized operand itself, against the oracle's dequantize
  c = dg._Canon(x_t, wq, DN)
  b, _ = c.rhs_values(wq)
  sb, gb = c.rhs_scale(wq)
  zp = None if wq.zero_point is None else c.rhs_zero_point(wq)[0].to(torch.int8)
  w = torch.empty(N, K, dtype=torch.bfloat16, device=util.DEV)
  from qwix_amd.core import numerics
  _lib.call('qwix_hip_dequantize_rm', b.data_ptr(), numerics.qtype_tag(wq.qtype), 1, K, N, K // gb, sb.data_ptr(),
            _lib.ptr(zp), _lib.float_tag(sb.dtype), w.data_ptr(), _lib.BF16, _lib.stream_of(w))
  deq = O.dequantize(owq)
  want_w = O.round_to_bf16(deq.v) if sdt == torch.float32 else deq.v
  assert np.array_equal(util.f32np(w).T, want_w)


@pytest.mark.parametrize('col0', [0, 8, 1])
@pytest.mark.parametrize('wq_type', ['int4', 'int8'])
def test_decode_call_on_one_row_of_a_wider_matrix(wq_type, col0):
  """A single-row view keeps the pitch and the base of its parent (torch calls it contiguous whatever they are): the
  decode kernel gets a 16-byte aligned row with a valid pitch, by restating the pitch or by one copy."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  g = torch.Generator().manual_seed(5)
  big = torch.randn(7, 1100, generator=g).to(torch.bfloat16).to(util.DEV)   # rows 2200 bytes apart
  w = (torch.randn(1024, 520, generator=g) * 0.05).to(torch.bfloat16).to(util.DEV)
  wq = qarray.quantize(w, qarray.HowToQuantize(qtype=wq_type, channelwise_axes=[1], tiled_axes={0: 128}))
  dn = (((1,), (0,)), ((), ()))
  row = big[3:4, col0:col0 + 1024]
  assert row.is_contiguous() and row.stride(0) == 1100
  assert torch.equal(dg.dot_general(row, wq, dn), dg.dot_general(row.clone(), wq, dn))


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('wq_type', ['int4', 'int8'])
@pytest.mark.parametrize('M,K,N', [(1, 512, 40), (5, 1024, 72), (16, 4096, 264), (32, 4224, 520), (17, 640, 32), (31, 896, 1000)])
def test_grouped_gemm_decode_batches(M, K, N, wq_type, dtype):
  """At most 32 rows against groups of 128 with one scale per token: the kernel whose four wavefronts split K by
  groups (K / 128 = 4, 5, 7, 8, 32, 33 groups: every remainder of the split; column tiles that end inside the last
  32).  Its outputs are the exact integer partials combined in f32: compared with their float64 combination."""
  from qwix_amd.core import dot_general as dg
  print('case grouped decode', M, K, N, wq_type, dtype, flush=True)
  group = 128
  xq, wq, oxq, owq, x_np, w_np = _pair(M, K, N, dtype, wq_type, group, seed=7 + M + N)
  out = dg.dot_general(xq, wq, DN)
  torch.cuda.synchronize()
  want, wacc = O.fast_dot_general(oxq, owq, DN, return_acc=True)
  got = util.f32np(out)
  assert got.shape == (M, N)
  assert np.all(np.abs(got - want.v) <= 1e-2 * np.abs(want.v) + util.partials_envelope(wacc, oxq, owq)), np.abs(got - want.v).max()
  sa = np.asarray(oxq.scale.v, np.float64).reshape(M, 1)
  sb = np.asarray(owq.scale.v, np.float64).reshape(K // group, 1, N)
  parts = np.asarray(wacc, np.float64).reshape(K // group, M, N) * sb
  exact, scale = parts.sum(0) * sa, np.abs(parts).sum(0) * sa
  tol = 2.0 ** -7 if dtype is O.BF16 else 1e-5
  assert np.all(np.abs(got - exact) <= tol * scale + 1e-30), (np.abs(got - exact) / (scale + 1e-30)).max()
  # the same rows inside a larger batch go through the tile kernel: equal up to the order of the f32 additions
  big_x = torch.cat([xq.qvalue, xq.qvalue.flip(0), xq.qvalue, xq.qvalue], 0)[:max(40, M)]
  if big_x.shape[0] >= 40:
    from qwix_amd.core.qarray import QArray
    big_s = torch.cat([xq.scale, xq.scale.flip(0), xq.scale, xq.scale], 0)[:big_x.shape[0]]
    if big_x.shape[0] == 40 and 4 * M >= 40:
      tiled = util.f32np(dg.dot_general(QArray(big_x.contiguous(), big_s.contiguous(), None, 'int8'), wq, DN))[:M]
      assert np.all(np.abs(tiled - got) <= tol * scale + 1e-30)


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('wq_type', ['int4', 'int8'])
@pytest.mark.parametrize('M,K,N,group,split', [(128, 4096, 1024, 128, True), (64, 8192, 520, 128, True), (200, 4096, 264, 256, True),
                                               (40, 3072, 72, 1024, True), (512, 8192, 1024, 128, True), (33, 4096, 64, 128, True),
                                               (16, 4096, 1024, 128, False), (2048, 4096, 4096, 128, False),
                                               (128, 1024, 1024, 128, False)])
def test_grouped_gemm_k_ranges(M, K, N, group, split, wq_type, dtype):
  """The sub-channel GEMM with K in ranges (qwix_hip_qgemm_grouped_ws, what the operator calls without `exact`): above
  the decode kernel's 32 rows, where the narrow tiles are few, every range's f32 sums go through a workspace and a
  second kernel adds them, applies the token scale and rounds.  The outputs are the exact integer partials combined in
  f32 in another order: compared with their float64 combination, and with the unsplit kernel through the C ABI (same
  bound); shapes that are not split report a workspace of 0 bytes and give the unsplit kernel's bits."""
  from qwix_amd import _lib
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import numerics
  print('case grouped k ranges', M, K, N, group, split, wq_type, dtype, flush=True)
  xq, wq, oxq, owq, x_np, w_np = _pair(M, K, N, dtype, wq_type, group, seed=11 + M + N)
  bq = numerics.qtype_tag(wq_type)
  nws = int(_lib.load().qwix_hip_qgemm_grouped_workspace_bytes(M, N, K, group, bq))
  assert (nws > 0) == split and nws % (M * N * 4) == 0
  out = dg.dot_general(xq, wq, DN)
  torch.cuda.synchronize()
  got = util.f32np(out)
  assert got.shape == (M, N)
  want, wacc = O.fast_dot_general(oxq, owq, DN, return_acc=True)
  sa = np.asarray(oxq.scale.v, np.float64).reshape(M, 1)
  sb = np.asarray(owq.scale.v, np.float64).reshape(K // group, 1, N)
  parts = np.asarray(wacc, np.float64).reshape(K // group, M, N) * sb
  exact, scale = parts.sum(0) * sa, np.abs(parts).sum(0) * sa
  tol = 2.0 ** -7 if dtype is O.BF16 else 1e-5
  assert np.all(np.abs(got - exact) <= tol * scale + 1e-30), (np.abs(got - exact) / (scale + 1e-30)).max()
  # through the C ABI: without a workspace the unsplit kernel runs; with one the result stays inside the same bound
  c = dg._Canon(xq, wq, DN)
  a = c.lhs_values(xq)
  b, _ = c.rhs_values(wq)
  sa_t, _ = c.lhs_scale(xq)
  sb_t, _ = c.rhs_scale(wq)
  st = _lib.stream_of(a)
  res_t = out.dtype

  def run(ws, n):
    o = torch.full((M, N), float('nan'), dtype=res_t, device=util.DEV)
    _lib.call('qwix_hip_qgemm_grouped_ws', a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), bq, M, N, K, group,
              sa_t.data_ptr(), _lib.float_tag(sa_t.dtype), 1, sb_t.data_ptr(), _lib.float_tag(sb_t.dtype), o.data_ptr(),
              _lib.float_tag(res_t), N, 0, None, _lib.ptr(ws), n, st)
    torch.cuda.synchronize()
    return o

  plain = torch.empty(M, N, dtype=res_t, device=util.DEV)
  _lib.call('qwix_hip_qgemm_grouped', a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), bq, M, N, K, group,
            sa_t.data_ptr(), _lib.float_tag(sa_t.dtype), 1, sb_t.data_ptr(), _lib.float_tag(sb_t.dtype), plain.data_ptr(),
            _lib.float_tag(res_t), N, 0, None, st)
  torch.cuda.synchronize()
  assert torch.equal(run(None, 0), plain)
  if not split:
    assert torch.equal(out, plain)
    return
  ws = torch.full((nws,), 0xFF, dtype=torch.uint8, device=util.DEV)  # NaN patterns: every partial sum must be written
  assert torch.equal(run(ws, nws - 1), plain)   # too small a workspace: not split
  assert torch.equal(run(ws, nws), out)         # what the operator ran
  assert np.all(np.abs(util.f32np(plain) - exact) <= tol * scale + 1e-30)
