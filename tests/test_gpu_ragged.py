"""GPU parity: ragged (mixture-of-experts) quantized GEMM through qwix_amd.ragged_dot vs the CPU oracle.

int8 x int8: the int32 sums are exact and the epilogue is elementwise, so outputs are compared bit for
bit.  e4m3 x e4m3: the matrix instruction's internal accumulation differs from the oracle's single
rounding of an exact sum (up to 1e-4 of the largest output), so outputs are compared at rtol 1e-2 for
bf16 results and 1e-3 for f32 results, the tolerances of the dense fp8 GEMM tests."""
import numpy as np
import pytest
import torch

from oracle import qwix_oracle as O
from tests import util

pytestmark = pytest.mark.gpu


def _how(qtype, channelwise, tiled=None):
  from qwix_amd.core import qarray
  return (qarray.HowToQuantize(qtype=qtype, channelwise_axes=list(channelwise), tiled_axes=dict(tiled or {})),
          O.HowToQuantize(qtype=qtype, channelwise_axes=list(channelwise), tiled_axes=dict(tiled or {})))


def _quantized(shape, dtype, seed, how, scale=1.0):
  from qwix_amd.core import qarray
  x_np, x_t = util.make(shape, dtype, seed=seed, scale=scale)
  q = qarray.quantize(x_t, how[0])
  oq = O.quantize(O.FArr(x_np, dtype), how[1])
  util.assert_qarray_equal(q, oq, 'operand')
  return q, oq


def _sizes(t):
  return torch.tensor(t, dtype=torch.int32, device=util.DEV)


def _check_exact(out, want):
  got = util.f32np(out)
  assert tuple(got.shape) == tuple(want.v.shape)
  bad = np.flatnonzero(got.ravel() != want.v.ravel())
  assert bad.size == 0, f'{bad.size} outputs differ: {got.ravel()[bad[:5]]} vs {want.v.ravel()[bad[:5]]}'


INT8_CASES = [
    # name, (M, K, G, N), group sizes, lhs channelwise, rhs channelwise, rhs tiled
    ('per-tensor', (128, 256, 4, 64), (64, 32, 16, 16), (), (), None),
    ('channelwise', (128, 256, 4, 64), (128, 100, 0, 28), (0,), (2,), None),
    ('group+channel', (128, 256, 4, 64), (50, 50, 28, 0), (0,), (0, 2), None),
    ('group only', (128, 256, 4, 64), (128, 0, 0, 0), (), (0,), None),
    ('short of M', (300, 384, 5, 200), (10, 0, 130, 1, 70), (0,), (0, 2), None),
    ('tile edges', (700, 128, 3, 260), (128, 129, 256), (0,), (0, 2), None),
    ('K not a multiple of 128', (200, 80, 3, 72), (60, 0, 100), (0,), (0, 2), None),
    ('many groups', (1000, 256, 64, 136), tuple((i * 7) % 31 for i in range(64)), (0,), (0, 2), None),
    ('k tiled', (128, 256, 4, 512), (10, 20, 30, 68), (0,), (0, 2), {1: 128}),
    ('k tiled, shared over groups', (128, 256, 4, 512), (10, 20, 30, 68), (0,), (2,), {1: 128}),
    ('k and n tiled', (128, 256, 4, 512), (10, 20, 30, 68), (0,), (0,), {1: 128, 2: 128}),
    ('decode: a few rows per group (weight-streaming kernel), empty groups, rows of no group', (40, 256, 12, 200),
     (0, 3, 16, 1, 0, 7, 2, 0, 5, 2, 1, 1), (0,), (0, 2), None),
    ('decode: one group takes several 16-row passes', (60, 384, 6, 72), (0, 40, 1, 0, 9, 3), (0,), (0, 2), None),
    ('decode: one row per group, shared weight scale', (16, 128, 16, 48), (1,) * 16, (0,), (2,), None),
    ('a few dozen rows per group (64-row tiles, deep weight prefetch), some groups empty or taller than a tile',
     (1700, 1024, 40, 520), tuple((i * 37) % 60 if i % 9 else (0 if i % 2 else 130) for i in range(40)), (0,), (0, 2), None),
    ('big groups', (2100, 512, 2, 2304), (1100, 900), (0,), (0, 2), None),
    ('big groups on a full chip (256-row tiles, ping-pong schedule)', (4096, 384, 4, 3072), (1000, 1100, 900, 1000), (0,), (0, 2), None),
]


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('name,shape,sizes,lcw,rcw,rtiled', INT8_CASES)
def test_ragged_dot_int8_bit_exact(name, shape, sizes, lcw, rcw, rtiled, dtype):
  import qwix_amd
  print('case ragged int8', name, shape, sizes, dtype, flush=True)
  M, K, G, N = shape
  xq, oxq = _quantized((M, K), dtype, 100 + M, _how('int8', lcw))
  wq, owq = _quantized((G, K, N), dtype, 200 + N, _how('int8', rcw, rtiled), scale=0.05)
  out = qwix_amd.ragged_dot(xq, wq, _sizes(sizes))
  torch.cuda.synchronize()
  _check_exact(out, O.ragged_dot(oxq, owq, sizes))


def test_ragged_dot_both_sides_k_tiled():
  import qwix_amd
  xq, oxq = _quantized((128, 256), O.BF16, 7, _how('int8', (0,), {1: 128}))
  wq, owq = _quantized((4, 256, 512), O.BF16, 8, _how('int8', (0, 2), {1: 128}), scale=0.05)
  out = qwix_amd.ragged_dot(xq, wq, _sizes((10, 20, 30, 68)))
  _check_exact(out, O.ragged_dot(oxq, owq, (10, 20, 30, 68)))
  bad, _ = _quantized((128, 256), O.BF16, 7, _how('int8', (0,), {1: 64}))
  with pytest.raises(ValueError, match='same tile size'):
    qwix_amd.ragged_dot(bad, wq, _sizes((10, 20, 30, 68)))


def test_ragged_dot_weights_stored_k_contiguous():
  """A weight kept as (G, N, K) storage and handed over as its (G, K, N) view is used in place."""
  import qwix_amd
  from qwix_amd.core.qarray import QArray
  xq, oxq = _quantized((256, 256), O.BF16, 17, _how('int8', (0,)))
  wq, owq = _quantized((3, 256, 192), O.BF16, 18, _how('int8', (0, 2)), scale=0.05)
  stored = wq.qvalue.permute(0, 2, 1).contiguous()
  view = QArray(stored.permute(0, 2, 1), wq.scale, None, wq.qtype)
  out = qwix_amd.ragged_dot(xq, view, _sizes((100, 56, 100)))
  _check_exact(out, O.ragged_dot(oxq, owq, (100, 56, 100)))


def test_ragged_dot_raw_int8_gives_int32():
  import qwix_amd
  rng = util.rng(3)
  a = rng.integers(-128, 128, (260, 128)).astype(np.int8)
  b = rng.integers(-128, 128, (3, 128, 136)).astype(np.int8)
  sizes = (130, 0, 100)
  out = qwix_amd.ragged_dot(torch.from_numpy(a).to(util.DEV), torch.from_numpy(b).to(util.DEV), _sizes(sizes))
  assert out.dtype == torch.int32
  assert np.array_equal(out.cpu().numpy(), O.ragged_dot(a, b, sizes))


def test_ragged_dot_out_of_range_sizes_are_clamped():
  """Negative sizes count as empty groups and a group that would pass the last row is cut off there
  (the kernel takes group_sizes from device memory and must stay inside the operands whatever it holds)."""
  import qwix_amd
  xq, oxq = _quantized((200, 128), O.BF16, 27, _how('int8', (0,)))
  wq, owq = _quantized((4, 128, 64), O.BF16, 28, _how('int8', (0, 2)), scale=0.05)
  out = qwix_amd.ragged_dot(xq, wq, _sizes((50, -3, 400, 10)))
  _check_exact(out, O.ragged_dot(oxq, owq, (50, 0, 150, 0)))


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('shape,sizes,rcw', [((128, 256, 4, 64), (128, 100, 0, 28), (2,)),
                                             ((520, 512, 6, 384), (100, 3, 0, 257, 60, 50), (0, 2)),
                                             ((4096, 256, 4, 3072), (1000, 1100, 900, 1000), (0, 2)),
                                             ((48, 256, 8, 200), (5, 0, 9, 1, 20, 3, 2, 4), (0, 2))])   # decode sizes
def test_ragged_dot_fp8(shape, sizes, rcw, dtype):
  import qwix_amd
  M, K, G, N = shape
  xq, oxq = _quantized((M, K), dtype, 300 + M, _how(O.E4M3, (0,)))
  wq, owq = _quantized((G, K, N), dtype, 400 + N, _how(O.E4M3, rcw), scale=0.05)
  out = qwix_amd.ragged_dot(xq, wq, _sizes(sizes))
  want = O.ragged_dot(oxq, owq, sizes).v
  got = util.f32np(out)
  tol = 1e-2 if dtype == O.BF16 else 1e-3
  np.testing.assert_allclose(got, want, rtol=tol, atol=tol * np.abs(want).max())
  assert np.all(got[min(sum(sizes), M):] == 0)


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('shape,sizes,rtiled', [((200, 256, 4, 136), (50, 0, 130, 20), None),
                                                ((300, 512, 3, 264), (100, 100, 60), {1: 128}),
                                                ((64, 1024, 6, 128), (1, 0, 30, 3, 0, 9), {1: 256})])
def test_ragged_dot_int4_expert_weights(shape, sizes, rtiled, dtype):
  """int8 activations x int4 expert weights (per channel and sub-channel along K): the sub-channel MFMA GEMM of
  dot_general, group by group.  Its f32 sum of the scaled partials is ordered differently from the oracle's, so
  the comparison is the one of the dense sub-channel tests (rtol 1e-2 for bf16 results, 1e-3 for f32)."""
  import qwix_amd
  M, K, G, N = shape
  xq, oxq = _quantized((M, K), dtype, 61, _how('int8', (0,)))
  wq, owq = _quantized((G, K, N), dtype, 62, _how('int4', (0, 2), rtiled), scale=0.05)
  out = qwix_amd.ragged_dot(xq, wq, _sizes(sizes))
  torch.cuda.synchronize()
  want = O.ragged_dot(oxq, owq, sizes).v
  got = util.f32np(out)
  assert out.dtype == util.TORCH_DT[dtype] and tuple(got.shape) == (M, N)
  # The reference rounds every K tile's scaled partial to the result dtype before summing them; the default
  # kernel keeps them in f32 (as for dot_general): with bf16 results that is up to half a bf16 step of the
  # largest partial per tile, on top of the 1e-2 bar.
  tol = 1e-2 if dtype == O.BF16 else 1e-3
  ntiles = K // (rtiled or {1: K})[1]
  atol = tol * np.abs(want).mean() + (ntiles * 2.0 ** -8 * np.abs(want).max() if dtype == O.BF16 else 0.0)
  np.testing.assert_allclose(got, want, rtol=tol, atol=atol)
  assert np.all(got[min(sum(sizes), M):] == 0)


@pytest.mark.parametrize('wq_type,tiled', [('int4', {1: 128}), ('int8', None), ('float8_e4m3fn', None)])
@pytest.mark.parametrize('sizes', [(3, 0, 20, 1), (300, 40, 0, 172)])
def test_ragged_dot_weight_only_experts(sizes, wq_type, tiled):
  """bf16 activations x quantized expert weights (the dequantize-first path, ragged_dot.py:229-241), group by group
  on this library's weight-only kernels: a few rows per expert (fused dequantize + bf16 MFMA) and hundreds
  (dequantize, then the bf16 MFMA GEMM)."""
  import qwix_amd
  M, K, G, N = 512, 512, 4, 192
  x_np, x_t = util.make((M, K), O.BF16, seed=71)
  wq, owq = _quantized((G, K, N), O.BF16, 72, _how(wq_type, (0, 2), tiled), scale=0.05)
  out = qwix_amd.ragged_dot(x_t, wq, _sizes(sizes))
  torch.cuda.synchronize()
  want = O.ragged_dot(O.FArr(x_np, O.BF16), owq, sizes).v
  got = util.f32np(out)
  assert out.dtype == torch.bfloat16
  np.testing.assert_allclose(got, want, rtol=1e-2, atol=1e-2 * np.abs(want).max())   # as for the fp8 experts above
  assert np.all(got[min(sum(sizes), M):] == 0)


def test_ragged_dot_dequantize_first_path():
  """A raw float lhs or a zero point sends the call to the dequantize-first path (ragged_dot.py:278-292)."""
  import qwix_amd
  from qwix_amd.core import qarray
  x_np, x_t = util.make((128, 256), O.F32, seed=31)
  wq, owq = _quantized((4, 256, 64), O.F32, 32, _how('int8', (0, 2)), scale=0.05)
  sizes = (50, 50, 28, 0)
  out = qwix_amd.ragged_dot(x_t, wq, _sizes(sizes))
  want = O.ragged_dot(O.FArr(x_np, O.F32), owq, sizes).v
  np.testing.assert_allclose(util.f32np(out), want, rtol=1e-4, atol=1e-4 * np.abs(want).max())
  xz = qarray.quantize(x_t, qarray.HowToQuantize(qtype='int8', calibration_method='minmax'))
  oxz = O.quantize(O.FArr(x_np, O.F32), O.HowToQuantize(qtype='int8', calibration_method='minmax'))
  out = qwix_amd.ragged_dot(xz, wq, _sizes(sizes))
  want = O.ragged_dot(oxz, owq, sizes).v
  np.testing.assert_allclose(util.f32np(out), want, rtol=1e-4, atol=1e-4 * np.abs(want).max())


def test_ragged_dot_errors():
  import qwix_amd
  from qwix_amd.core import ragged_dot as rd
  xq, _ = _quantized((128, 256), O.BF16, 41, _how('int8', (0,)))
  wq, _ = _quantized((4, 256, 64), O.BF16, 42, _how('int8', (0, 2)), scale=0.05)
  with pytest.raises(ValueError, match='one entry per group'):
    qwix_amd.ragged_dot(xq, wq, _sizes((64, 64)))
  with pytest.raises(NotImplementedError, match='group_offset'):
    qwix_amd.ragged_dot(xq, wq, _sizes((64, 64, 0, 0)), group_offset=_sizes((0,)))
  dn = rd.RaggedDotDimensionNumbers((((0,), (1,)), ((), ())), (1,), (0,))   # contracts 128 rows with K = 256
  with pytest.raises(ValueError, match='differ'):
    qwix_amd.ragged_dot_general(xq, wq, _sizes((64, 64, 0, 0)), dn)
  dn = rd.RaggedDotDimensionNumbers((((1,), (1,)), ((), ())), (0,), ())     # no group axis: another ragged mode
  with pytest.raises(NotImplementedError, match='one group axis'):
    qwix_amd.ragged_dot_general(xq, wq, _sizes((64, 64, 0, 0)), dn)


def _rdn(dn, ragged, group):
  from qwix_amd.core.ragged_dot import RaggedDotDimensionNumbers
  return RaggedDotDimensionNumbers(dot_dimension_numbers=dn, lhs_ragged_dimensions=(ragged,), rhs_group_dimensions=(group,))


GENERAL_CASES = [
    # name, lhs shape, rhs shape, dot dimension numbers, ragged axis, group axis, sizes, lhs how, rhs how
    ("the reference's non-basic case: a batch axis, K in tiles of 64, no free axis on the rhs", (8, 620, 256), (8, 4, 256),
     (((2,), (2,)), ((0,), (0,))), 1, 1, (60, 120, 190, 250), dict(tiled_axes={2: 64}), dict(tiled_axes={2: 64})),
    ('weights stored (G, N, K)', (200, 128), (3, 72, 128), (((1,), (2,)), ((), ())), 0, 0, (60, 0, 100),
     dict(channelwise_axes=[0]), dict(channelwise_axes=[0, 1])),
    ('rows last on the lhs, group axis in the middle of the rhs', (128, 300), (128, 5, 40), (((0,), (0,)), ((), ())), 1, 1,
     (10, 0, 130, 1, 70), dict(channelwise_axes=[1]), dict(channelwise_axes=[1, 2])),
    ('two contracting axes', (96, 4, 64), (3, 4, 64, 24), (((1, 2), (1, 2)), ((), ())), 0, 0, (30, 50, 16),
     dict(channelwise_axes=[0]), dict(channelwise_axes=[0, 3])),
    ('batch axis and K in tiles of 128', (2, 150, 256), (2, 4, 256, 136), (((2,), (2,)), ((0,), (0,))), 1, 1, (40, 0, 100, 10),
     dict(channelwise_axes=[0, 1], tiled_axes={2: 128}), dict(channelwise_axes=[0, 1, 3], tiled_axes={2: 128})),
]


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('name,lshape,rshape,dn,ragged,group,sizes,lhow,rhow', GENERAL_CASES)
def test_ragged_dot_general_dimension_numbers(name, lshape, rshape, dn, ragged, group, sizes, lhow, rhow, dtype):
  """Dimension numbers other than ragged_dot's (ragged_dot.py:123-226 passes any to lax.ragged_dot_general): the ragged
  axis as the only free axis of the lhs, with batch axes, several contracting axes and any axis order.  int8: exact
  sums and an elementwise epilogue, so bit for bit wherever a single K tile is scaled; f32 sums of tile partials at
  1e-5."""
  import qwix_amd
  from qwix_amd.core import qarray
  print('case ragged general', name, dtype, flush=True)
  x_np, x_t = util.make(lshape, dtype, seed=len(name))
  w_np, w_t = util.make(rshape, dtype, seed=len(name) + 1, scale=0.05)
  xq, oxq = qarray.quantize(x_t, qarray.HowToQuantize(qtype='int8', **lhow)), O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(qtype='int8', **lhow))
  wq, owq = qarray.quantize(w_t, qarray.HowToQuantize(qtype='int8', **rhow)), O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(qtype='int8', **rhow))
  util.assert_qarray_equal(xq, oxq, 'lhs')
  util.assert_qarray_equal(wq, owq, 'rhs')
  out = qwix_amd.ragged_dot_general(xq, wq, _sizes(sizes), _rdn(dn, ragged, group))
  want = O.ragged_dot_general(oxq, owq, sizes, dn, ragged, group)
  assert out.dtype == util.TORCH_DT[want.dtype]
  tiled = 'tiled_axes' in lhow or 'tiled_axes' in rhow
  if tiled and dtype == O.F32:
    np.testing.assert_allclose(util.f32np(out), want.v, rtol=0, atol=1e-5 * float(np.abs(want.v).max()))
  elif tiled:
    # bf16 partials: the reference rounds each three times before the f32 sum; the default mode keeps them in f32
    np.testing.assert_allclose(util.f32np(out), want.v, rtol=0, atol=2e-2 * float(np.abs(want.v).max()))
  else:
    _check_exact(out, want)


def test_ragged_dot_general_weight_only_and_errors():
  import qwix_amd
  from qwix_amd.core import qarray
  x_np, x_t = util.make((200, 128), O.BF16, seed=3)
  w_np, w_t = util.make((3, 72, 128), O.BF16, seed=4, scale=0.05)
  how = dict(qtype='int8', channelwise_axes=[0, 1])
  wq, owq = qarray.quantize(w_t, qarray.HowToQuantize(**how)), O.quantize(O.FArr(w_np, O.BF16), O.HowToQuantize(**how))
  dn = (((1,), (2,)), ((), ()))
  out = qwix_amd.ragged_dot_general(x_t, wq, _sizes((60, 0, 100)), _rdn(dn, 0, 0))     # float lhs: dequantize first
  want = O.ragged_dot_general(O.FArr(x_np, O.BF16), owq, (60, 0, 100), dn, 0, 0)
  np.testing.assert_allclose(util.f32np(out), want.v, rtol=1e-2, atol=1e-2 * float(np.abs(want.v).max()))
  assert np.all(util.f32np(out)[160:] == 0)
  with pytest.raises(NotImplementedError, match='ragged contracting or batch axis'):
    qwix_amd.ragged_dot_general(x_t, wq, _sizes((60, 0, 100)), _rdn(dn, 1, 0))
  x3 = torch.zeros(4, 200, 128, dtype=torch.bfloat16, device=util.DEV)
  with pytest.raises(NotImplementedError, match='only free axis'):
    qwix_amd.ragged_dot_general(x3, wq, _sizes((60, 0, 100)), _rdn((((2,), (2,)), ((), ())), 1, 0))
