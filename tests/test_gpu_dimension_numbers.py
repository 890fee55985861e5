"""GPU parity: general dimension numbers (batch axes, several contracting axes, contracting axes that are
not trailing, permuted einsum outputs) through dot_general / einsum vs the CPU oracle.

int8 x int8 per-channel contractions are exact integers followed by an elementwise epilogue, so every
case here is compared bit for bit."""
import numpy as np
import pytest
import torch

from oracle import qwix_oracle as O
from tests import util

pytestmark = pytest.mark.gpu


def _quantize_both(einsum_str, lshape, rshape, dtype, seed, qtype='int8'):
  from qwix_amd.core import einsum as es
  from qwix_amd.core import qarray
  x_np, x_t = util.make(lshape, dtype, seed=seed)
  w_np, w_t = util.make(rshape, dtype, seed=seed + 1, scale=0.05)
  nd = (len(lshape), len(rshape))
  hl = es.get_how_to_quantize(einsum_str=einsum_str, ndims=nd, for_lhs=True, tile_size=None, qtype=qtype)
  hr = es.get_how_to_quantize(einsum_str=einsum_str, ndims=nd, for_lhs=False, tile_size=None, qtype=qtype)
  ohl = O.einsum_get_how_to_quantize(einsum_str=einsum_str, ndims=nd, for_lhs=True, tile_size=None, qtype=qtype)
  ohr = O.einsum_get_how_to_quantize(einsum_str=einsum_str, ndims=nd, for_lhs=False, tile_size=None, qtype=qtype)
  assert list(hl.channelwise_axes) == list(ohl.channelwise_axes) and list(hr.channelwise_axes) == list(ohr.channelwise_axes)
  xq, wq = qarray.quantize(x_t, hl), qarray.quantize(w_t, hr)
  oxq, owq = O.quantize(O.FArr(x_np, dtype), ohl), O.quantize(O.FArr(w_np, dtype), ohr)
  util.assert_qarray_equal(xq, oxq, 'lhs')
  util.assert_qarray_equal(wq, owq, 'rhs')
  return xq, wq, oxq, owq


CASES = [
    ('btd,dnh->btnh', (2, 16, 64), (64, 4, 32)),       # attention projection: two free axes on the weight
    ('btnh,nhd->btd', (2, 16, 4, 32), (4, 32, 48)),    # output projection: two contracting axes
    ('bqd,bkd->bqk', (3, 40, 64), (3, 24, 64)),        # one batch axis, activation x activation
    ('bhqd,bhkd->bhqk', (2, 3, 20, 64), (2, 3, 12, 64)),  # two batch axes
    ('td,dn->nt', (50, 128), (128, 70)),               # permuted output
    ('dt,dn->tn', (128, 50), (128, 70)),               # contracting axis of the lhs is not the last one
    ('bdq,bkd->bkq', (2, 64, 10), (2, 12, 64)),        # batch + leading contraction + permuted output
    ('bqd,bkd->bqk', (4, 200, 128), (4, 136, 128)),    # K a multiple of 128: the direct-to-LDS batched kernel, ragged tile edges
    ('bhqd,bhkd->bhqk', (2, 2, 130, 256), (2, 2, 260, 256)),
]


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('einsum_str,lshape,rshape', CASES)
def test_einsum_general_dimension_numbers_bit_exact(einsum_str, lshape, rshape, dtype):
  from qwix_amd.core import einsum as es
  print('case einsum', einsum_str, lshape, rshape, dtype, flush=True)
  xq, wq, oxq, owq = _quantize_both(einsum_str, lshape, rshape, dtype, seed=sum(lshape))
  out = es.einsum(einsum_str, xq, wq)
  torch.cuda.synchronize()
  want = O.einsum(einsum_str, oxq, owq)
  assert tuple(out.shape) == tuple(want.v.shape)
  got = util.f32np(out)
  bad = np.flatnonzero(got.ravel() != want.v.ravel())
  assert bad.size == 0, f'{bad.size} outputs differ: {got.ravel()[bad[:5]]} vs {want.v.ravel()[bad[:5]]}'


def test_batch_axes_take_one_launch(monkeypatch):
  """Quantized operands with batch axes go through the batched kernel, not through one launch per element,
  and both routes give the same bits (int8) / the same values to the fp8 tolerance."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  dn = (((2,), (2,)), ((0,), (0,)))
  for qtype in ('int8', O.E4M3):
    x_np, x_t = util.make((3, 70, 128), O.BF16, seed=31)
    w_np, w_t = util.make((3, 50, 128), O.BF16, seed=32)
    xq = qarray.quantize(x_t, qarray.HowToQuantize(qtype=qtype, channelwise_axes=[0, 1]))
    wq = qarray.quantize(w_t, qarray.HowToQuantize(qtype=qtype, channelwise_axes=[0, 1]))
    looped = dg._over_batch(dg._fast_dot_general, xq, wq, dn)
    with monkeypatch.context() as m:
      m.setattr(dg, '_over_batch', lambda *a, **k: (_ for _ in ()).throw(AssertionError('looped over the batch')))
      out = dg.dot_general(xq, wq, dn)
    assert tuple(out.shape) == (3, 70, 50) and out.dtype == torch.bfloat16
    if qtype == 'int8':
      assert torch.equal(out, looped)
      oxq = O.quantize(O.FArr(x_np, O.BF16), O.HowToQuantize(qtype=qtype, channelwise_axes=[0, 1]))
      owq = O.quantize(O.FArr(w_np, O.BF16), O.HowToQuantize(qtype=qtype, channelwise_axes=[0, 1]))
      assert np.array_equal(util.f32np(out), O.dot_general(oxq, owq, dn).v)
    else:
      np.testing.assert_allclose(util.f32np(out), util.f32np(looped), rtol=1e-2, atol=1e-2 * float(looped.abs().max()))


def test_batched_dot_general_on_the_dequantize_path():
  """A float activation against a batched quantized operand takes the dequantize-first path."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  x_np, x_t = util.make((2, 10, 64), O.F32, seed=11)
  w_np, w_t = util.make((2, 64, 24), O.F32, seed=12, scale=0.05)
  how = dict(qtype='int8', channelwise_axes=[0, 2])
  wq = qarray.quantize(w_t, qarray.HowToQuantize(**how))
  owq = O.quantize(O.FArr(w_np, O.F32), O.HowToQuantize(**how))
  dn = (((2,), (1,)), ((0,), (0,)))
  out = dg.dot_general(x_t, wq, dn)
  want = O.dot_general(O.FArr(x_np, O.F32), owq, dn)
  assert tuple(out.shape) == (2, 10, 24)
  np.testing.assert_allclose(util.f32np(out), want.v, rtol=1e-5, atol=1e-6)


def test_batch_shape_mismatch_is_an_error():
  from qwix_amd.core import dot_general as dg
  a = torch.zeros(2, 4, 16, device=util.DEV)
  b = torch.zeros(3, 16, 4, device=util.DEV)
  with pytest.raises(ValueError, match='batch dimensions differ'):
    dg.dot_general(a, b, (((2,), (1,)), ((0,), (0,))))


def test_three_operand_einsum_contracts_pairwise():
  """activation x quantized weight x float matrix: the first contraction takes the quantized path."""
  from qwix_amd.core import einsum as es
  from qwix_amd.core import qarray
  x_np, x_t = util.make((24, 64), O.F32, seed=21)
  w_np, w_t = util.make((64, 32), O.F32, seed=22, scale=0.05)
  p_np, p_t = util.make((32, 8), O.F32, seed=23)
  xq = qarray.quantize(x_t, qarray.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  wq = qarray.quantize(w_t, qarray.HowToQuantize(qtype='int8', channelwise_axes=[1]))
  out = es.einsum('td,dn,nk->tk', xq, wq, p_t)
  oxq = O.quantize(O.FArr(x_np, O.F32), O.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  owq = O.quantize(O.FArr(w_np, O.F32), O.HowToQuantize(qtype='int8', channelwise_axes=[1]))
  first = O.einsum('td,dn->tn', oxq, owq)
  want = first.v.astype(np.float64) @ p_np.astype(np.float64)
  assert tuple(out.shape) == (24, 8)
  np.testing.assert_allclose(util.f32np(out), want, rtol=1e-4, atol=1e-5)


def test_empty_operands_launch_nothing():
  """Zero-size operands behave like lax.dot_general's: an empty result, zeros for an empty contraction, and
  the reduction over an empty axis is refused as jnp.max refuses it."""
  from qwix_amd.core import dot_general as dg, einsum, qarray, ragged_dot
  dev = util.DEV
  how_a = qarray.HowToQuantize(qtype='int8', channelwise_axes=[0])
  how_w = qarray.HowToQuantize(qtype='int8', channelwise_axes=[1])
  x0 = torch.empty(0, 128, device=dev, dtype=torch.bfloat16)
  w = torch.randn(128, 64, device=dev, dtype=torch.bfloat16)
  wq = qarray.quantize(w, how_w)
  for qtype in ('int8', 'int4', 'float8_e4m3fn'):
    q0 = qarray.quantize(x0, qarray.HowToQuantize(qtype=qtype, channelwise_axes=[0]))
    assert tuple(q0.shape) == (0, 128) and tuple(q0.scale.shape) == (0, 1) and q0.scale.dtype == torch.bfloat16
    qarray.validate_qarray(q0)
    assert tuple(qarray.dequantize(q0).shape) == (0, 128)
  with pytest.raises(ValueError, match='zero-size array'):
    qarray.quantize(torch.empty(128, 0, device=dev, dtype=torch.bfloat16), how_a)
  with pytest.raises(ValueError, match='zero-size array'):
    qarray.calibrate(torch.empty(0, 128, device=dev, dtype=torch.bfloat16), how_w)
  assert tuple(qarray.calibrate(x0, how_a)['absmax'].shape) == (0, 1)
  dn = (((1,), (0,)), ((), ()))
  q0 = qarray.quantize(x0, how_a)
  out = dg.dot_general(q0, wq, dn)
  assert tuple(out.shape) == (0, 64) and out.dtype == torch.bfloat16
  out = dg.dot_general(x0, wq, dn, preferred_element_type=torch.float32)
  assert tuple(out.shape) == (0, 64) and out.dtype == torch.float32
  assert tuple(einsum.einsum('mk,kn->mn', x0, wq).shape) == (0, 64)
  # an empty contraction: zeros
  a = qarray.QArray(torch.empty(4, 0, dtype=torch.int8, device=dev), torch.ones(4, 1, device=dev), None, 'int8')
  b = qarray.QArray(torch.empty(0, 8, dtype=torch.int8, device=dev), torch.ones(1, 8, device=dev), None, 'int8')
  out = dg.dot_general(a, b, dn)
  assert tuple(out.shape) == (4, 8) and torch.count_nonzero(out).item() == 0
  with pytest.raises(TypeError):
    dg.dot_general(q0, qarray.quantize(torch.randn(64, 64, device=dev, dtype=torch.bfloat16), how_w), dn)
  wg = qarray.quantize(torch.randn(2, 128, 64, device=dev, dtype=torch.bfloat16),
                       qarray.HowToQuantize(qtype='int8', channelwise_axes=[0, 2]))
  out = ragged_dot.ragged_dot(q0, wg, torch.zeros(2, dtype=torch.int32, device=dev))
  assert tuple(out.shape) == (0, 64)


def test_reference_output_dtype_table_by_execution():
  """dot_general_test.py:28-146 builds 10 x 10 operands of ones with per-tensor scales and checks the result
  dtype of the slow path, the fast path, the dispatcher and einsum under every preferred_element_type.  Here
  the four are run, not only shape-evaluated: K = 10 is not a multiple of the kernels' 16-byte pieces, the
  int4 left operand is widened, and every output element must be exactly 10."""
  from qwix_amd.core import dot_general as dg, einsum, qarray
  dev = util.DEV

  def mk(spec):
    if not isinstance(spec, tuple):
      return torch.ones(10, 10, dtype=spec, device=dev)
    qd, sd = spec
    if qd == 'int4':
      qv = qarray.Int4Tensor(torch.full((10, 5), 0x11, dtype=torch.uint8, device=dev), (10, 10), 1)
    elif qd == 'int8':
      qv = torch.ones(10, 10, dtype=torch.int8, device=dev)
    else:
      qv = torch.ones(10, 10, device=dev).to(torch.float8_e4m3fn)
    return qarray.QArray(qv, torch.ones(1, 1, dtype=sd, device=dev), None, qd)

  bf16, f32 = torch.bfloat16, torch.float32
  cases = [(bf16, f32, f32), (bf16, ('int8', bf16), bf16), (bf16, ('int8', f32), f32),
           (('int4', bf16), ('int8', f32), f32), (('float8_e4m3fn', bf16), ('float8_e4m3fn', f32), f32)]
  dn = (((1,), (0,)), ((), ()))
  for l, r, expected in cases:
    lhs, rhs = mk(l), mk(r)
    for pet in (None, bf16, f32):
      want = pet or expected
      outs = [dg._slow_dot_general(lhs, rhs, dn, preferred_element_type=pet),
              dg._fast_dot_general(lhs, rhs, dn, preferred_element_type=pet),
              dg.dot_general(lhs, rhs, dn, preferred_element_type=pet),
              einsum.einsum('ab,bc->ac', lhs, rhs, preferred_element_type=pet)]
      for o in outs:
        assert o.dtype == want, (l, r, pet, o.dtype)
        assert tuple(o.shape) == (10, 10) and torch.all(o.float() == 10).item(), (l, r, pet)


@pytest.mark.parametrize('einsum_str,explicit,lshape,rshape', [
    ('a b c, b c d -> a d', 'abc,bcd->ad', (10, 256, 16), (256, 16, 128)),       # einsum_test.py:176-182
    ('...ab,...bc->...ac', 'xab,xbc->xac', (10, 256, 16), (10, 16, 128)),        # :183-190
    ('...ab,bc->...ac', 'xab,bc->xac', (10, 256, 16), (16, 128)),                # :191-198
    ('abc,bcd->acd', 'abc,bcd->acd', (10, 256, 16), (256, 16, 128)),             # :199-207
])
def test_reference_einsum_strings_bit_exact(einsum_str, explicit, lshape, rshape):
  """The einsum strings of the reference's own einsum test (spaces, ellipses, a shared kept axis), int8 per
  channel: bit-exact against the oracle run on the equivalent explicit string."""
  from qwix_amd.core import einsum as es
  xq, wq, oxq, owq = _quantize_both(explicit, lshape, rshape, O.BF16, seed=91)
  out = es.einsum(einsum_str, xq, wq)
  want = O.einsum(explicit, oxq, owq)
  assert tuple(out.shape) == tuple(want.v.shape)
  assert np.array_equal(util.f32np(out), want.v)


def test_einsum_asymmetric_subchannel_lhs():
  """einsum_test.py:208-217: 'abc,bcd->acd' with a minmax lhs and tiles of a quarter of the contracted axis
  (64 < 128: the dequantize-first path, over slices of the shared kept axis)."""
  from qwix_amd.core import einsum as es, qarray
  x_np, x_t = util.make((10, 256, 16), O.BF16, seed=92)
  x_np = O.round_to_bf16(x_np + np.float32(1.0))
  x_t = torch.from_numpy(x_np).to(torch.bfloat16).to(util.DEV)
  w_np, w_t = util.make((256, 16, 128), O.BF16, seed=93)
  nd = (3, 3)
  hl = es.get_how_to_quantize(einsum_str='abc,bcd->acd', ndims=nd, for_lhs=True, tile_size=1 / 4, qtype='int8',
                              calibration_method='minmax')
  hr = es.get_how_to_quantize(einsum_str='abc,bcd->acd', ndims=nd, for_lhs=False, tile_size=1 / 4, qtype='int8')
  out = es.einsum('abc,bcd->acd', qarray.quantize(x_t, hl), qarray.quantize(w_t, hr))
  ref = np.einsum('abc,bcd->acd', x_np.astype(np.float64), w_np.astype(np.float64))
  assert tuple(out.shape) == (10, 16, 128) and out.dtype == torch.bfloat16
  assert np.abs(util.f32np(out) - ref).mean() / np.abs(ref).mean() < 0.012


@pytest.mark.parametrize('einsum_str,lshape,rshape,expected', [
    ('BTNH,BSNH->BTNS', (1, 2, 4, 8), (1, 3, 1, 8), (1, 2, 4, 3)),   # einsum_test.py:332-339: size-1 broadcast
    ('BTNH,BSNH->BTNS', (1, 2, 4, 8), (1, 3, 8, 8), (1, 2, 8, 3)),   # :340-347: 4 heads against 8
    ('BTNH,BSNH->BTNS', (1, 2, 8, 8), (1, 3, 4, 8), (1, 2, 8, 3)),   # :348-355
    ('bth,thk->btk', (2, 3, 4), (3, 4, 5), (2, 3, 5)),               # :356-362
])
def test_einsum_generic_broadcasting(einsum_str, lshape, rshape, expected):
  """Operands whose shared axes differ by a whole factor are repeated tile-wise first (einsum_info.py:197-241)."""
  from qwix_amd.core import einsum as es, qarray
  _, lhs = util.make(lshape, O.F32, seed=94)
  _, rhs = util.make(rshape, O.F32, seed=95)
  out = es.einsum(einsum_str, lhs, rhs)
  assert tuple(out.shape) == expected
  subs = einsum_str.split('->')[0].split(',')
  size = {}
  for sub, shp in zip(subs, (lshape, rshape)):
    for ch, d in zip(sub, shp):
      size[ch] = max(size.get(ch, 1), d)
  grow = lambda t, sub: qarray.broadcast_to(t, tuple(size[c] for c in sub))
  want = torch.einsum(einsum_str, grow(lhs, subs[0]), grow(rhs, subs[1]))
  assert torch.allclose(out, want, rtol=1e-5, atol=1e-5)
  # quantized operands broadcast the same way
  ql = qarray.quantize(lhs, qarray.HowToQuantize(qtype='int8', channelwise_axes=list(range(len(lshape) - 1))))
  qo = es.einsum(einsum_str, ql, rhs)
  assert tuple(qo.shape) == expected
  assert ((qo - want).abs().mean() / want.abs().mean()).item() < 0.02


def test_einsum_mixed_operands_scalar_and_incompatible_shapes():
  """einsum_test.py:363-383 (a quantized lhs with a float rhs, a scalar rhs) and :443-448."""
  from qwix_amd.core import einsum as es, qarray
  _, lhs = util.make((128, 128), O.F32, seed=96)
  _, rhs = util.make((128, 32), O.F32, seed=97)
  ql = qarray.quantize(lhs, qarray.HowToQuantize(qtype='int8'))
  out = es.einsum('ij,jk->ik', ql, rhs)
  want = lhs @ rhs
  assert tuple(out.shape) == (128, 32) and ((out - want).abs().mean() / want.abs().mean()).item() < 0.02
  out = es.einsum('ij,->ij', ql, torch.tensor(2.0, device=util.DEV))
  assert tuple(out.shape) == (128, 128) and ((out - 2 * lhs).abs().mean() / (2 * lhs).abs().mean()).item() < 0.02
  with pytest.raises(ValueError, match='Cannot broadcast'):
    es.einsum('BTNH,BSNH->BTNS', torch.ones(1, 2, 3, 8, device=util.DEV), torch.ones(1, 3, 4, 8, device=util.DEV))


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('group', [None, 128])
def test_int4_weights_with_a_batch_axis(group, dtype):
  """Batched contraction 'bmk,bkn->bmn' against int4 weights (one weight matrix per batch element, with and without
  sub-channel scales): the packed bytes are sliced per element, each element runs the 2-D kernels; int8 activations
  give the oracle's int32 sums and outputs bit for bit, bf16 activations (weight-only) meet the 1e-2 bar."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  B, M, K, N = 3, 24, 256, 72
  x_np, x_t = util.make((B, M, K), dtype, seed=61)
  w_np, w_t = util.make((B, K, N), dtype, seed=62, scale=0.05)
  rkw = dict(qtype='int4', channelwise_axes=[0, 2])
  if group:
    rkw['tiled_axes'] = {1: group}
  lkw = dict(qtype='int8', channelwise_axes=[0, 1])
  wq = qarray.quantize(w_t, qarray.HowToQuantize(**rkw))
  owq = O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(**rkw))
  util.assert_qarray_equal(wq, owq, 'int4 weights')
  xq = qarray.quantize(x_t, qarray.HowToQuantize(**lkw))
  oxq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(**lkw))
  dn = (((2,), (1,)), ((0,), (0,)))
  out = dg._fast_dot_general(xq, wq, dn, exact=True)   # the mode whose roundings are the reference's, step by step
  torch.cuda.synchronize()
  want = O.dot_general(oxq, owq, dn)
  assert tuple(out.shape) == (B, M, N)
  assert np.array_equal(util.f32np(out), want.v)
  # weight-only: a float activation against the batched int4 weight
  out2 = dg.dot_general(x_t, wq, dn)
  want2 = O.dot_general(O.FArr(x_np, dtype), owq, dn)
  np.testing.assert_allclose(util.f32np(out2), want2.v, rtol=1e-2, atol=1e-2 * float(np.abs(want2.v).mean()))


def _pair(lshape, rshape, lhow, rhow, dtype, seed):
  from qwix_amd.core import qarray
  x_np, x_t = util.make(lshape, dtype, seed=seed)
  w_np, w_t = util.make(rshape, dtype, seed=seed + 1, scale=0.05)
  xq, wq = qarray.quantize(x_t, qarray.HowToQuantize(**lhow)), qarray.quantize(w_t, qarray.HowToQuantize(**rhow))
  oxq, owq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(**lhow)), O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(**rhow))
  util.assert_qarray_equal(xq, oxq, 'lhs')
  util.assert_qarray_equal(wq, owq, 'rhs')
  return xq, wq, oxq, owq


# lhs (T, N, H) x rhs (N, H, D), contracting (N, H): the output projection of attention
TILED_DN = (((1, 2), (0, 1)), ((), ()))
TILED_CASES = [
    # both contracting axes tiled on both sides (2 x 2 tile combinations)
    ('both axes, both sides', (24, 256, 256), (256, 256, 40), {1: 128, 2: 128}, {0: 128, 1: 128}),
    # last axis tiled on the weight only, heads untiled: groups that are not contiguous in the flattened K
    ('last axis, weight only', (24, 4, 256), (4, 256, 40), {}, {1: 128}),
    # first contracting axis tiled only
    ('first axis only', (24, 256, 8), (256, 8, 40), {1: 128}, {0: 128}),
    # activation tiled, weight per channel
    ('lhs only', (10, 2, 384), (2, 384, 24), {2: 128}, {}),
]


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('name,lshape,rshape,ltiles,rtiles', TILED_CASES)
def test_tiled_scales_over_several_contracting_axes_bit_exact(name, lshape, rshape, ltiles, rtiles, dtype):
  """dot_general.py:93-122, 186-226, 255-260: every tiled contracting axis becomes a tile axis of the product, the
  partials are scaled tile by tile and summed.  int8 x int8: exact partials, the oracle's roundings, the oracle's
  order of the sum over tiles: equal bits."""
  from qwix_amd.core import dot_general as dg
  print('case tiled multi-axis', name, dtype, flush=True)
  xq, wq, oxq, owq = _pair(lshape, rshape, dict(qtype='int8', channelwise_axes=[0], tiled_axes=ltiles),
                           dict(qtype='int8', channelwise_axes=[2], tiled_axes=rtiles), dtype, seed=sum(lshape))
  assert dg._use_fast_path(xq, wq, TILED_DN)
  for pet, opet in ((None, None), (torch.float32, O.F32)):
    out = dg.dot_general(xq, wq, TILED_DN, preferred_element_type=pet)
    torch.cuda.synchronize()
    want = O.dot_general(oxq, owq, TILED_DN, opet)
    assert tuple(out.shape) == tuple(want.v.shape) and out.dtype == util.TORCH_DT[want.dtype]
    got = util.f32np(out)
    bad = np.flatnonzero(got.ravel() != want.v.ravel())
    assert bad.size == 0, f'{bad.size} outputs differ: {got.ravel()[bad[:5]]} vs {want.v.ravel()[bad[:5]]}'


def test_tiled_zero_points_over_several_contracting_axes_bit_exact():
  """An asymmetric activation tiled along the last of two contracting axes: the zero point is split with the tiles
  (dot_general.py:196-203) and every tile's partial corrected before it is scaled."""
  from qwix_amd.core import dot_general as dg
  xq, wq, oxq, owq = _pair((12, 3, 256), (3, 256, 20),
                           dict(qtype='int8', channelwise_axes=[0], tiled_axes={2: 128}, calibration_method='minmax'),
                           dict(qtype='int8', channelwise_axes=[2], tiled_axes={1: 128}), O.BF16, seed=77)
  assert xq.zero_point is not None
  out = dg.dot_general(xq, wq, TILED_DN)
  torch.cuda.synchronize()
  want = O.dot_general(oxq, owq, TILED_DN)
  assert np.array_equal(util.f32np(out), want.v)


@pytest.mark.parametrize('tile', [128, 192])
def test_tiled_scales_that_the_sub_channel_kernel_does_not_take(tile):
  """One contracting axis, tiles of 192 (not a multiple of the kernel's 128-wide slabs): int8 bit-exact; e4m3
  operands with sub-channel scales (no sub-channel fp8 kernel): the fp8 tolerance."""
  from qwix_amd.core import dot_general as dg
  dn = (((1,), (0,)), ((), ()))
  K = 3 * tile
  for qtype in ('int8', O.E4M3):
    if qtype == 'int8' and tile == 128:
      continue  # the sub-channel kernel's own case
    print('case tile-by-tile', tile, qtype, flush=True)
    xq, wq, oxq, owq = _pair((40, K), (K, 72), dict(qtype=qtype, channelwise_axes=[0], tiled_axes={1: tile}),
                             dict(qtype=qtype, channelwise_axes=[1], tiled_axes={0: tile}), O.BF16, seed=tile)
    out = dg.dot_general(xq, wq, dn, preferred_element_type=torch.float32)
    torch.cuda.synchronize()
    want = O.dot_general(oxq, owq, dn, O.F32).v
    got = util.f32np(out)
    if qtype == 'int8':
      assert np.array_equal(got, want)
    else:
      assert np.allclose(got, want, rtol=1e-2, atol=1e-2 * np.abs(want).mean()), np.abs(got - want).max()


def test_int4_weights_tiled_under_two_contracting_axes():
  """int4 weights (N, H, D) packed along D, tiled along H: tiles are cut out of the packed bytes."""
  from qwix_amd.core import dot_general as dg
  xq, wq, oxq, owq = _pair((16, 2, 256), (2, 256, 48), dict(qtype='int8', channelwise_axes=[0]),
                           dict(qtype='int4', channelwise_axes=[2], tiled_axes={1: 128}), O.BF16, seed=91)
  out = dg._fast_dot_general(xq, wq, TILED_DN, exact=True)
  torch.cuda.synchronize()
  want = O.dot_general(oxq, owq, TILED_DN)
  assert np.array_equal(util.f32np(out), want.v)


@pytest.mark.parametrize('sdt', [O.BF16, O.F32])
@pytest.mark.parametrize('ltile,rtile', [(128, 128), (None, 128), (256, None), (128, 256)])
def test_e4m3_operands_with_sub_channel_scales(ltile, rtile, sdt):
  """e4m3 x e4m3 with scales tiled along the contracting axis: one launch of the sub-channel kernel (f32 partial per
  group on the fp8 matrix-core instruction, the oracle's roundings per group, f32 sum over groups).  The order in
  which the hardware adds inside a group is not the oracle's: the fp8 tolerance."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  dn = (((1,), (0,)), ((), ()))
  M, K, N = 200, 1024, 136
  if ltile and rtile and ltile != rtile:
    with pytest.raises(ValueError):
      xq, wq, _, _ = _pair((M, K), (K, N), dict(qtype=O.E4M3, channelwise_axes=[0], tiled_axes={1: ltile}),
                           dict(qtype=O.E4M3, channelwise_axes=[1], tiled_axes={0: rtile}), O.BF16, seed=5)
      dg.dot_general(xq, wq, dn)
    return
  print('case e4m3 sub-channel', ltile, rtile, sdt, flush=True)
  x_np, x_t = util.make((M, K), O.BF16, seed=41)
  w_np, w_t = util.make((K, N), O.BF16, seed=42, scale=0.05)
  lkw = dict(qtype=O.E4M3, channelwise_axes=[0], tiled_axes={1: ltile} if ltile else {})
  rkw = dict(qtype=O.E4M3, channelwise_axes=[1], tiled_axes={0: rtile} if rtile else {})
  tsdt = util.TORCH_DT[sdt]
  xq = qarray.quantize_api(x_t, scale_dtype=tsdt, **lkw)
  wq = qarray.quantize_api(w_t, scale_dtype=tsdt, **rkw)
  oxq = O.quantize_api(O.FArr(x_np, O.BF16), scale_dtype=sdt, **lkw)
  owq = O.quantize_api(O.FArr(w_np, O.BF16), scale_dtype=sdt, **rkw)
  util.assert_qarray_equal(xq, oxq, 'lhs')
  util.assert_qarray_equal(wq, owq, 'rhs')
  for pet, opet in ((None, None), (torch.float32, O.F32), (torch.bfloat16, O.BF16)):
    out = dg.dot_general(xq, wq, dn, preferred_element_type=pet)
    torch.cuda.synchronize()
    want = O.dot_general(oxq, owq, dn, opet)
    assert out.dtype == util.TORCH_DT[want.dtype] and tuple(out.shape) == (M, N)
    got = util.f32np(out)
    mag = np.abs(want.v).mean()
    # The default kernel keeps every scaled partial in f32 where the reference rounds it to the scale dtype three
    # times per group (more accurate than the reference, inside its rounding envelope): the mean error is held to
    # about a bf16 step (2^-8), single elements to a few steps.
    assert np.abs(got - want.v).mean() < 5e-3 * mag, np.abs(got - want.v).mean() / mag
    assert np.allclose(got, want.v, rtol=2e-2, atol=2e-2 * mag), np.abs(got - want.v).max()
    # with the reference's roundings per group: only the order of the f32 additions inside a group is left
    ex = dg._fast_dot_general(xq, wq, dn, preferred_element_type=pet, exact=True)
    torch.cuda.synchronize()
    assert np.allclose(util.f32np(ex), want.v, rtol=1e-2, atol=1e-2 * mag), np.abs(util.f32np(ex) - want.v).max()
  # and the same numbers as the tile-by-tile route on the untiled kernels, up to the order of the f32 additions
  tiled = [(1, 0, ltile or rtile)]
  ref = dg._tile_by_tile(xq, wq, dn, tiled, torch.float32, False)
  out = dg.dot_general(xq, wq, dn, preferred_element_type=torch.float32)
  torch.cuda.synchronize()
  assert torch.allclose(out, ref, rtol=1e-4, atol=1e-4 * ref.abs().mean().item())


@pytest.mark.parametrize('act_calibration', ['absmax', 'minmax'])
@pytest.mark.parametrize('M,K,N,dtype', [
    (64, 2048, 264, O.BF16), (513, 256, 264, O.BF16), (128, 1152, 128, O.F32), (8, 768, 72, O.BF16),
    (256, 64, 1024, O.BF16), (17, 192, 1024, O.BF16), (3, 144, 64, O.F32),  # K the sub-channel kernel does not take
])
def test_int4_weights_with_per_channel_scales_bit_exact(M, K, N, dtype, act_calibration):
  """int8 x int4 with one scale per row / column is the untiled contraction of dot_general.py:205-226,255-261:
  exact integers, then (T(acc) * sx) * sy with a rounding per step, whatever kernel multiplies."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  print('case int4 per-channel', M, K, N, dtype, act_calibration, flush=True)
  x_np, x_t = util.make((M, K), dtype, seed=M + K)
  if act_calibration == 'minmax':
    x_np = O.rnd(x_np + 0.7, dtype)
    x_t = util.to_gpu(x_np, dtype)
  w_np, w_t = util.make((K, N), dtype, seed=N + K, scale=0.05)
  ha = dict(qtype='int8', channelwise_axes=[0], calibration_method=act_calibration)
  hw = dict(qtype='int4', channelwise_axes=[1])
  xq, wq = qarray.quantize(x_t, qarray.HowToQuantize(**ha)), qarray.quantize(w_t, qarray.HowToQuantize(**hw))
  oxq, owq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(**ha)), O.quantize(O.FArr(w_np, dtype), O.HowToQuantize(**hw))
  util.assert_qarray_equal(xq, oxq, 'lhs')
  util.assert_qarray_equal(wq, owq, 'rhs')
  dn = (((1,), (0,)), ((), ()))
  got = util.f32np(dg.dot_general(xq, wq, dn))
  want = O.dot_general(oxq, owq, dn).v
  bad = np.flatnonzero(got.ravel() != want.ravel())
  assert bad.size == 0, f'{bad.size} of {got.size} outputs differ: {got.ravel()[bad[:4]]} vs {want.ravel()[bad[:4]]}'


def test_f32_result_of_the_dequantize_first_path_is_not_rounded_to_bf16():
  """Tiles finer than 128 send both operands through dequantize + float dot (dot_general.py:407-491, 264-275); with
  preferred_element_type f32 the bf16 x bf16 products are summed and delivered in f32.  Compared at 1e-5 of the
  largest output (the order of the f32 additions is free); a result rounded to bf16 on the way is off by 2e-3."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  x_np, x_t = util.make((33, 128), O.BF16, seed=34)
  w_np, w_t = util.make((128, 16), O.BF16, seed=35, scale=0.05)
  ha = dict(qtype='int8', channelwise_axes=[0], tiled_axes={1: 32})
  hw = dict(qtype='int8', channelwise_axes=[1], tiled_axes={0: 32})
  xq, wq = qarray.quantize(x_t, qarray.HowToQuantize(**ha)), qarray.quantize(w_t, qarray.HowToQuantize(**hw))
  oxq, owq = O.quantize(O.FArr(x_np, O.BF16), O.HowToQuantize(**ha)), O.quantize(O.FArr(w_np, O.BF16), O.HowToQuantize(**hw))
  dn = (((1,), (0,)), ((), ()))
  assert not O.use_fast_path(oxq, owq, dn)
  out = dg.dot_general(xq, wq, dn, preferred_element_type=torch.float32)
  want = O.dot_general(oxq, owq, dn, preferred_element_type=O.F32)
  assert out.dtype == torch.float32 and want.dtype == O.F32
  np.testing.assert_allclose(util.f32np(out), want.v, rtol=0, atol=1e-5 * float(np.abs(want.v).max()))
