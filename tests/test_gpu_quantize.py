"""GPU parity: HIP quantize / calibrate / dequantize kernels vs the CPU oracle, bit-exact."""
import numpy as np
import pytest
import torch

from oracle import qwix_oracle as O
from tests import util

pytestmark = pytest.mark.gpu

QTYPES = ['int8', 'int4', 'float8_e4m3fn']


def _check(x_np, x_t, dtype, how_kwargs, layout=None, what=''):

  from qwix_amd.core import qarray
  print('case', what, x_np.shape, dtype, how_kwargs, layout, flush=True)
  qa = qarray.quantize(x_t, qarray.HowToQuantize(**how_kwargs), layout=layout)
  torch.cuda.synchronize()
  want = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(**how_kwargs))
  util.assert_qarray_equal(qa, want, what)
  return qa


@pytest.mark.parametrize('qtype', QTYPES)
@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('shape', [(64, 4096), (7, 1000), (5, 130), (3, 20000), (1, 8), (300, 256), (2, 3, 512)])
def test_per_token_rows(shape, dtype, qtype):
  x_np, x_t = util.make(shape, dtype, seed=hash((shape, dtype, qtype)) % 1000)
  cw = list(range(len(shape) - 1))
  _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=cw), what='rows')


@pytest.mark.parametrize('qtype', QTYPES)
@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
def test_rows_subchannel_tiles(dtype, qtype):
  x_np, x_t = util.make((48, 1024), dtype, seed=11)
  for tile in (128, 32, 1 / 4):
    _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=[0], tiled_axes={1: tile}), what=f'rows tile {tile}')


@pytest.mark.parametrize('qtype', QTYPES)
def test_every_bf16_value_rows(qtype):
  """All finite bf16 bit patterns, grouped so that rows span very different magnitudes."""
  bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.uint16)
  xb = bits.view(torch.bfloat16)
  xb = xb[torch.isfinite(xb)]
  order = torch.argsort(xb.abs().to(torch.float32), stable=True)
  xb = xb[order]
  n = (xb.numel() // 512) * 512
  for rows_of in (512, 64):
    x = xb[:n].reshape(-1, rows_of).contiguous()
    x_np = x.to(torch.float32).numpy()
    _check(x_np, x.to(util.DEV), O.BF16, dict(qtype=qtype, channelwise_axes=[0]), what=f'all-bf16 rows of {rows_of}')
  # mixed magnitudes within a row: a strided shuffle
  x = xb[:n].reshape(512, -1).t().contiguous()
  _check(x.to(torch.float32).numpy(), x.to(util.DEV), O.BF16, dict(qtype=qtype, channelwise_axes=[0]), what='all-bf16 mixed')


@pytest.mark.parametrize('qtype', QTYPES)
@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('layout', ['natural', 'reduce_minor'])
@pytest.mark.parametrize('shape,tile', [((512, 256), None), ((512, 256), 128), ((1000, 64), None), ((384, 128), 64), ((256, 40), None)])
def test_weight_columns(shape, tile, layout, dtype, qtype):
  x_np, x_t = util.make(shape, dtype, seed=21, scale=0.02)
  kw = dict(qtype=qtype, channelwise_axes=[1])
  if tile:
    kw['tiled_axes'] = {0: tile}
  qa = _check(x_np, x_t, dtype, kw, layout=layout, what=f'cols {layout}')
  from qwix_amd.core.qarray import Int4Tensor
  data = qa.qvalue.data if isinstance(qa.qvalue, Int4Tensor) else qa.qvalue
  if layout == 'reduce_minor':
    assert data.stride(0) == 1, 'reduce-minor layout must be K-contiguous'


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
def test_weight_3d_einsum_kernel(dtype):
  """(d, n, h) weight contracting d: outer=1, reduce=d, inner=n*h."""
  x_np, x_t = util.make((256, 4, 32), dtype, seed=31, scale=0.02)
  _check(x_np, x_t, dtype, dict(qtype='int8', channelwise_axes=[1, 2]), what='dnh')
  _check(x_np, x_t, dtype, dict(qtype='int4', channelwise_axes=[1, 2], tiled_axes={0: 128}), what='dnh tiled')
  # (n, h, d) contracting n, h: reduce = n*h
  x_np, x_t = util.make((4, 64, 128), dtype, seed=32, scale=0.02)
  _check(x_np, x_t, dtype, dict(qtype='int8', channelwise_axes=[2]), what='nhd')


@pytest.mark.parametrize('qtype', ['int8', 'int4'])
@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
def test_minmax(dtype, qtype):
  x_np, x_t = util.make((40, 512), dtype, seed=41)
  x_np = x_np + np.float32(0.5) if dtype == O.F32 else O.round_to_bf16(x_np + np.float32(0.5))
  x_t = torch.from_numpy(x_np).to(util.TORCH_DT[dtype]).to(util.DEV)
  _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=[0], calibration_method='minmax'), what='minmax rows')
  _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=[1], calibration_method='minmax'), what='minmax cols')
  _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=[0], calibration_method='absmax,0.8'), what='absmax factor')
  # tall groups: the strided reduction in 256-row pieces
  x_np, x_t = util.make((600, 96), dtype, seed=42)
  x_np = x_np + np.float32(0.25) if dtype == O.F32 else O.round_to_bf16(x_np + np.float32(0.25))
  x_t = torch.from_numpy(x_np).to(util.TORCH_DT[dtype]).to(util.DEV)
  _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=[1], calibration_method='minmax'), what='minmax tall cols')
  _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=[1], tiled_axes={0: 300}), what='absmax tall cols, 2 groups')


def test_reference_exact_minmax_vector():
  """qarray_test.py:191-219 on the GPU."""
  from qwix_amd.core import qarray
  a = (np.arange(256) / 255.0).astype(np.float32)
  qa = qarray.quantize(torch.from_numpy(a).to(util.DEV), qarray.HowToQuantize(qtype='int8', calibration_method='minmax'))
  assert qa.zero_point.reshape(()).item() == -128
  assert np.array_equal(util.qvalues_np(qa), np.arange(-128, 128).astype(np.int8))
  dq = qarray.dequantize(qa)
  assert np.allclose(util.f32np(dq), a)


def test_2d_tiles_generic():
  """two_dim_scales_test.py:29-50."""
  x_np, x_t = util.make((128, 128), O.BF16, seed=51)
  qa = _check(x_np, x_t, O.BF16, dict(qtype='int8', tiled_axes={0: 8, 1: 8}), what='2d tiles')
  assert tuple(qa.scale.shape) == (16, 16)
  x_np, x_t = util.make((6, 10), O.F32, seed=52)
  _check(x_np, x_t, O.F32, dict(qtype='int8', channelwise_axes=[1]), what='ragged cols')
  _check(x_np, x_t, O.F32, dict(qtype='int4'), what='per tensor')


@pytest.mark.parametrize('qtype', QTYPES)
@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('shape,tiles', [
    ((256, 384), {0: 128, 1: 128}),          # block-scaled weight, 16 loads per thread for f32
    ((96, 160), {0: 32, 1: 32}),
    ((64, 80), {0: 8, 1: 16}),               # several blocks per wavefront
    ((64, 64), {0: 16, 1: 8}),               # one 16-byte vector per block row (bf16)
    ((192, 96), {0: 96, 1: 48}),             # block row pieces that are not a power of two
    ((3, 128, 256), {1: 64, 2: 128}),        # a stack of matrices (experts)
    ((64, 3, 128), {0: 32, 2: 64}),          # a kept axis between the two tiled ones
    ((512, 128), {0: 256, 1: 128}),          # the largest block the single-pass kernel holds (bf16)
    ((40, 24), {0: 8, 1: 12}),               # row pieces shorter than a 16-byte vector: the scalar kernels
])
def test_2d_blocks(shape, tiles, dtype, qtype):
  x_np, x_t = util.make(shape, dtype, seed=61, scale=0.05)
  # different magnitudes per block, so that a scale written to the wrong block shows
  ramp = np.linspace(0.25, 4.0, int(np.prod(shape)), dtype=np.float32).reshape(shape)
  x_np = x_np * ramp if dtype == O.F32 else O.round_to_bf16(x_np * ramp)
  x_t = torch.from_numpy(x_np).to(util.TORCH_DT[dtype]).to(util.DEV)
  cw = [a for a in range(len(shape)) if a not in tiles]
  _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=cw, tiled_axes=tiles), what='2d blocks')
  if qtype != 'float8_e4m3fn':
    x_np = x_np + np.float32(0.03) if dtype == O.F32 else O.round_to_bf16(x_np + np.float32(0.03))
    x_t = torch.from_numpy(x_np).to(util.TORCH_DT[dtype]).to(util.DEV)
    _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=cw, tiled_axes=tiles, calibration_method='minmax'),
           what='2d blocks minmax')


@pytest.mark.parametrize('qtype', QTYPES)
@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
def test_fixed_calibration(dtype, qtype):
  """'fixed,a[,b]': a constant per-tensor range, whatever axes are named channelwise."""
  x_np, x_t = util.make((48, 256), dtype, seed=71, scale=2.0)
  _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=[0], calibration_method='fixed,3'), what='fixed symmetric')
  _check(x_np, x_t, dtype, dict(qtype=qtype, calibration_method='fixed,-2.5,2.5'), what='fixed symmetric pair')
  if qtype != 'float8_e4m3fn':
    _check(x_np, x_t, dtype, dict(qtype=qtype, channelwise_axes=[1], calibration_method='fixed,-1,3'), what='fixed asymmetric')
  from qwix_amd.core import qarray
  with pytest.raises(ValueError):
    qarray.quantize(x_t, qarray.HowToQuantize(qtype=qtype, calibration_method='fixed,1,2'))
  with pytest.raises(ValueError, match='scale factor'):
    qarray.quantize(x_t, qarray.HowToQuantize(qtype=qtype, calibration_method='rms'))


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('shape,kw', [
    ((64, 512), dict(channelwise_axes=[0], tiled_axes={1: 1 / 8})),   # qarray_test.py:92-100 ('rms,7', tiles of 1/8)
    ((40, 256), dict(channelwise_axes=[0])),
    ((256, 48), dict(channelwise_axes=[1])),                           # reduction along the strided axis
    ((64, 64), dict(tiled_axes={0: 16, 1: 32})),                       # two reduced axis groups
])
def test_rms_calibration(shape, kw, dtype):
  """'rms,7': scale = D(D(sqrt(D(mean(D(x^2))))) * 7) / qmax.  The mean is an f32 sum whose order neither XLA nor
  this kernel pins: the calibration must match the oracle to one unit in the last place of the array dtype, and
  where it matches exactly the quantized values must too (parity unpinned beyond that, as the oracle says)."""
  from qwix_amd.core import qarray
  x_np, x_t = util.make(shape, dtype, seed=75)
  how = dict(qtype='int8', calibration_method='rms,7', **kw)
  cal = qarray.calibrate(x_t, qarray.HowToQuantize(**how))
  want = O.calibrate(O.FArr(x_np, dtype), O.HowToQuantize(**how))
  assert set(cal) == {'absmax'} and tuple(cal['absmax'].shape) == want['absmax'].v.shape
  got = util.f32np(cal['absmax'])
  ulp = 2.0 ** -7 if dtype == O.BF16 else 2.0 ** -22
  assert np.all(np.abs(got - want['absmax'].v) <= ulp * np.abs(want['absmax'].v))
  if dtype == O.BF16:  # f32 shows the summation order directly; bf16 hides it behind its rounding almost always
    assert np.mean(got == want['absmax'].v) > 0.9
  # closed form on a constant array: rms of all-c is |c|
  c = torch.full(shape, -0.75, dtype=util.TORCH_DT[dtype], device=util.DEV)
  assert torch.all(qarray.calibrate(c, qarray.HowToQuantize(**how))['absmax'] == 0.75 * 7).item()
  if 'tiled_axes' in kw and len(kw['tiled_axes']) == 2:
    return  # the static-scale kernel takes one reduced axis group
  qa = qarray.quantize(x_t, qarray.HowToQuantize(**how))
  oq = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(**how))
  if np.array_equal(util.f32np(qa.scale), oq.scale.v):
    util.assert_qarray_equal(qa, oq, 'rms')
  else:
    same = util.f32np(qa.scale) == oq.scale.v
    for ax, (d, sd) in enumerate(zip(shape, same.shape)):
      same = np.repeat(same, d // sd, axis=ax)
    assert np.array_equal(util.qvalues_np(qa)[same], oq.qvalue[same])


def test_zero_rows_and_reference_convert_vectors():
  from qwix_amd.core import qarray
  x = torch.zeros(4, 256, dtype=torch.bfloat16, device=util.DEV)
  x[1] = 3.0
  qa = qarray.quantize(x, qarray.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  assert util.f32np(qa.scale)[:, 0].tolist() == [1.0, float(torch.tensor(3.0 / 127.5).to(torch.bfloat16)), 1.0, 1.0]
  # numerics_test.py:34-56 through the static-scale kernel with scale 1
  v = torch.tensor([[1.2, 3.5, -127.5, 129, -1300, float('inf'), float('-inf'), 0.5]], dtype=torch.float32, device=util.DEV)
  one = torch.ones(1, 1, device=util.DEV)
  q8 = qarray.quantize_with_scale_zero_point(v, 'int8', one, None)
  assert util.qvalues_np(q8)[0].tolist() == [1, 4, -128, 127, -128, 127, -128, 0]
  q4 = qarray.quantize_with_scale_zero_point(v, 'int4', one, None)
  assert util.qvalues_np(q4)[0].tolist() == [1, 4, -8, 7, -8, 7, -8, 0]
  f8 = qarray.quantize_with_scale_zero_point(torch.tensor([[10.0, 500.0, -1000.0, 0.0]], device=util.DEV), 'float8_e4m3fn', one, None)
  assert O.e4m3_to_f32(util.qvalues_np(f8))[0].tolist() == [10.0, 448.0, -448.0, 0.0]


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
def test_calibrate_scale_static_pipeline(dtype):
  """calibrate -> compute_scale_zero_point -> quantize_with_scale_zero_point == quantize."""
  from qwix_amd.core import qarray
  for shape, kw in [((32, 512), dict(channelwise_axes=[0])), ((256, 64), dict(channelwise_axes=[1])),
                    ((256, 64), dict(channelwise_axes=[1], tiled_axes={0: 128}))]:
    for cal in ('absmax', 'minmax'):
      x_np, x_t = util.make(shape, dtype, seed=61)
      how = qarray.HowToQuantize(qtype='int8', calibration_method=cal, **kw)
      c = qarray.calibrate(x_t, how)
      oc = O.calibrate(O.FArr(x_np, dtype), O.HowToQuantize(qtype='int8', calibration_method=cal, **kw))
      for k in oc:
        assert np.array_equal(util.f32np(c[k]), oc[k].v), (shape, kw, cal, k)
      s, zp = qarray.compute_scale_zero_point(c, 'int8')
      qa = qarray.quantize_with_scale_zero_point(x_t, 'int8', s, zp)
      want = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(qtype='int8', calibration_method=cal, **kw))
      util.assert_qarray_equal(qa, want, f'pipeline {shape} {kw} {cal}')


@pytest.mark.parametrize('qtype', QTYPES)
@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
def test_dequantize(dtype, qtype):
  from qwix_amd.core import qarray
  cases = [((32, 512), dict(channelwise_axes=[0]), None), ((256, 64), dict(channelwise_axes=[1], tiled_axes={0: 128}), 'natural'),
           ((256, 64), dict(channelwise_axes=[1], tiled_axes={0: 128}), 'reduce_minor'),
           # shapes that miss the vector paths (odd widths) and shapes with ragged 64 x 64 tiles
           ((10, 130), dict(channelwise_axes=[0]), None), ((96, 36), dict(channelwise_axes=[1]), 'natural'),
           ((96, 36), dict(channelwise_axes=[1]), 'reduce_minor'), ((160, 208), dict(channelwise_axes=[1]), 'reduce_minor'),
           ((1024, 400), dict(channelwise_axes=[1], tiled_axes={0: 256}), 'reduce_minor'),
           ((3, 128, 80), dict(channelwise_axes=[0, 2]), 'reduce_minor'), ((64, 4096), dict(channelwise_axes=[0], tiled_axes={1: 128}), None),
           ((512, 96), dict(), None)]
  for shape, kw, layout in cases:
    x_np, x_t = util.make(shape, dtype, seed=71)
    qa = qarray.quantize(x_t, qarray.HowToQuantize(qtype=qtype, **kw), layout=layout)
    dq = qarray.dequantize(qa)
    want = O.dequantize(O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(qtype=qtype, **kw)))
    assert dq.dtype == util.TORCH_DT[dtype]
    assert np.array_equal(util.f32np(dq), want.v), (shape, kw, layout)
  if qtype == 'int8':  # zero points on each path
    for shape, kw, layout in cases[:3] + cases[6:8]:
      x_np, x_t = util.make(shape, dtype, seed=72, dist='uniform')
      qa = qarray.quantize(x_t, qarray.HowToQuantize(qtype=qtype, calibration_method='minmax', **kw), layout=layout)
      want = O.dequantize(O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(qtype=qtype, calibration_method='minmax', **kw)))
      assert np.array_equal(util.f32np(qarray.dequantize(qa)), want.v), ('minmax', shape, kw, layout)


def test_errors_match_reference_behaviour():
  from qwix_amd.core import qarray
  x = torch.zeros(4, 10, device=util.DEV)
  with pytest.raises(ValueError, match='cannot be tiled'):
    qarray.quantize(x, qarray.HowToQuantize(qtype='int8', tiled_axes={1: 4}))
  with pytest.raises(ValueError, match='both channelwise and tiled'):
    qarray.quantize(x, qarray.HowToQuantize(qtype='int8', channelwise_axes=[1], tiled_axes={1: 5}))
  with pytest.raises(ValueError, match='Refuse to quantize'):
    qarray.quantize(x.to(torch.int32), qarray.HowToQuantize(qtype='int8'))
  with pytest.raises(ValueError, match="doesn't support asymmetric"):
    qarray.quantize(x, qarray.HowToQuantize(qtype='float8_e4m3fn', calibration_method='minmax'))


@pytest.mark.parametrize('qtype', QTYPES)
@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('shape,kw', [
    ((512, 1024), dict()),                                   # one scale for the whole array (524288 elements)
    ((3, 40000), dict(channelwise_axes=[0])),                # rows longer than a workgroup keeps in registers
    ((2, 6, 20480), dict(channelwise_axes=[0])),             # 122880 contiguous elements per scale
    ((4, 98304), dict(channelwise_axes=[0], tiled_axes={1: 49152})),
])
def test_long_contiguous_groups(shape, kw, dtype, qtype):
  """Scale groups of more than 16384 contiguous elements are calibrated in pieces and merged."""
  x_np, x_t = util.make(shape, dtype, seed=len(shape) * 7 + shape[-1] % 13)
  _check(x_np, x_t, dtype, dict(qtype=qtype, **kw), what='long rows')
  if qtype == 'int8':
    _check(x_np, x_t, dtype, dict(qtype=qtype, calibration_method='minmax', **kw), what='long rows minmax')


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
def test_long_contiguous_groups_calibrate_and_static(dtype):
  from qwix_amd.core import qarray
  x_np, x_t = util.make((300, 2048), dtype, seed=99)
  for cal in ('absmax', 'minmax'):
    how = qarray.HowToQuantize(qtype='int8', calibration_method=cal)
    ohow = O.HowToQuantize(qtype='int8', calibration_method=cal)
    c = qarray.calibrate(x_t, how)
    oc = O.calibrate(O.FArr(x_np, dtype), ohow)
    for k in oc:
      assert tuple(c[k].shape) == (1, 1) and np.array_equal(util.f32np(c[k]), oc[k].v), (cal, k)
    s, zp = qarray.compute_scale_zero_point(c, 'int8')
    qa = qarray.quantize_with_scale_zero_point(x_t, 'int8', s, zp)   # static range: the scale is given
    util.assert_qarray_equal(qa, O.quantize(O.FArr(x_np, dtype), ohow), f'static per-tensor {cal}')


@pytest.mark.parametrize('qtype', ['int8', 'int4', 'float8_e4m3fn'])
def test_bf16_division_for_every_pair_of_significands(qtype):
  """The kernels divide bf16 by bf16 as x * rcp(s).  Every scale significand (128 of them, two exponents) against
  every finite bf16 value: each (significand of x, significand of s) pair occurs at every exponent difference, in
  particular where the quotient lies in [64, 128) and a bf16 step is 0.5, so that a quotient rounded to the wrong
  bf16 neighbour changes the int8 that comes out.  Given scales (the static-range kernel) and the oracle's true
  division."""
  from qwix_amd.core import qarray
  bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.uint16)
  xb = bits.view(torch.bfloat16)
  xb = xb[torch.isfinite(xb)]
  n = (xb.numel() // 64) * 64
  row = xb[:n].to(torch.float32).numpy()
  for e in (-2, 9):
    sig = (np.arange(128, 256, dtype=np.float32) / 128.0) * np.float32(2.0 ** e)
    x_np = np.broadcast_to(row, (128, n)).copy()
    scale_np = sig.reshape(128, 1)
    assert np.array_equal(O.round_to_bf16(scale_np), scale_np)
    x_t = util.to_gpu(x_np, O.BF16)
    qa = qarray.quantize_with_scale_zero_point(x_t, qtype, util.to_gpu(scale_np, O.BF16), None)
    want = O.quantize_with_scale_zero_point(O.FArr(x_np, O.BF16), qtype, O.FArr(scale_np, O.BF16), None)
    util.assert_qarray_equal(qa, want, f'all significand pairs, scale exponent {e}')


@pytest.mark.parametrize('qtype', ['int8', 'float8_e4m3fn'])
def test_static_scale_with_overflowing_quotients(qtype):
  """A given scale need not come from the data: quotients that overflow or are infinite must still follow
  true division (saturate), on rows that mix them with ordinary values and on rows that hold none."""
  from qwix_amd.core import qarray
  x_np = util.make_np((6, 512), O.BF16, seed=5)
  x_np[0, :8] = [3e38, -3e38, 1e30, -1e30, np.inf, -np.inf, 0.0, 1.0]
  x_np[3, 100] = 2e35
  x_np = O.round_to_bf16(x_np)
  x_t = util.to_gpu(x_np, O.BF16)
  for s in (2.0 ** -120, 2.0 ** -20, 1.0):
    scale_np = np.full((6, 1), s, np.float32)
    qa = qarray.quantize_with_scale_zero_point(x_t, qtype, util.to_gpu(scale_np, O.BF16), None)
    want = O.quantize_with_scale_zero_point(O.FArr(x_np, O.BF16), qtype, O.FArr(scale_np, O.BF16), None)
    util.assert_qarray_equal(qa, want, f'static scale {s}')


def test_array_methods_commute_with_dequantize():
  """qarray_test.py:244-283: dequantize(q.reshape(...)) == dequantize(q).reshape(...), and the same for a slice."""
  from qwix_amd.core import qarray
  x_np, x_t = util.make((2, 2, 6), O.F32, seed=73)
  q = qarray.quantize(x_t, qarray.HowToQuantize(qtype='int8', channelwise_axes=[0], tiled_axes={2: 2}))
  assert tuple(q.scale.shape) == (2, 1, 3)
  full = qarray.dequantize(q)
  assert torch.equal(qarray.dequantize(q.reshape(4, 1, 3, 2)), full.reshape(4, 1, 3, 2))
  assert torch.equal(qarray.dequantize(q[..., 1]), full[..., 1])
  assert torch.equal(qarray.dequantize(q[1]), full[1])
  assert torch.equal(qarray.dequantize(q.transpose(1, 2, 0)), full.permute(1, 2, 0))


@pytest.mark.parametrize('qtype', ['int8', 'int4'])
@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('shape,kw', [((64, 512), dict(channelwise_axes=[0])), ((256, 96), dict(channelwise_axes=[1])),
                                      ((128, 256), dict(channelwise_axes=[1], tiled_axes={0: 64})),
                                      ((6, 40, 64), dict(channelwise_axes=[0, 1], calibration_method='minmax')),
                                      ((32, 128), dict(calibration_method='fixed,-3,3'))])
def test_stochastic_rounding_with_caller_noise(shape, kw, dtype, qtype):
  """`noise_fn` (numerics.py:191-195): the noise is added in f32 before the rounding.  The same noise array through the
  HIP kernel and through the oracle: qvalues, scales and zero points bit for bit; float qtypes ignore the noise."""
  from qwix_amd.core import qarray
  x_np, x_t = util.make(shape, dtype, seed=sum(shape))
  noise_np = util.rng(17).uniform(-0.5, 0.5, shape).astype(np.float32)
  noise_t = torch.from_numpy(noise_np).to(util.DEV)
  calls = []
  def noise_fn(s):
    calls.append(tuple(s))
    return noise_t
  how = qarray.HowToQuantize(qtype=qtype, noise_fn=noise_fn, **kw)
  got = qarray.quantize(x_t, how)
  torch.cuda.synchronize()
  assert calls == [shape]
  want = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(qtype=qtype, **kw), noise_np)
  util.assert_qarray_equal(got, want, f'noise {qtype}')
  plain = O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(qtype=qtype, **kw))
  assert (want.qvalue != plain.qvalue).mean() > 0.1        # the noise did move roundings
  if 'calibration_method' not in kw:
    f8 = qarray.quantize(x_t, qarray.HowToQuantize(qtype='float8_e4m3fn', noise_fn=noise_fn, **kw))
    util.assert_qarray_equal(f8, O.quantize(O.FArr(x_np, dtype), O.HowToQuantize(qtype='float8_e4m3fn', **kw)), 'f8 ignores noise')


@pytest.mark.parametrize('qtype,calibration', [('int8', 'absmax'), ('int4', 'minmax'), (O.E4M3, 'absmax')])
def test_three_separate_groups_of_reduced_axes(qtype, calibration):
  """Blocks on the first two axes and the whole last axis under one scale, a kept axis between them: more groups
  of reduced axes than the kernels take in place; the elements of a scale are gathered into rows first."""
  from qwix_amd.core import qarray
  shape, how = (48, 16, 40, 2), dict(qtype=qtype, channelwise_axes=[2], tiled_axes={0: 2, 1: 8}, calibration_method=calibration)
  x_np, x_t = util.make(shape, O.BF16, seed=77)
  q = qarray.quantize(x_t, qarray.HowToQuantize(**how))
  oq = O.quantize(O.FArr(x_np, O.BF16), O.HowToQuantize(**how))
  assert tuple(q.scale.shape) == (24, 2, 40, 1)
  util.assert_qarray_equal(q, oq, 'regrouped')
  assert np.array_equal(util.f32np(qarray.dequantize(q)), O.dequantize(oq).v)


def test_int4_with_a_scale_per_element_and_unit_reduced_axes():
  """Groups of one element (every axis channelwise) and reduced axes of size 1 next to real ones."""
  from qwix_amd.core import qarray
  for shape, how in [((64, 16), dict(qtype='int4', channelwise_axes=[0, 1])),
                     ((16, 256, 1, 24), dict(qtype='int4', channelwise_axes=[0, 3], tiled_axes={2: 1}, calibration_method='minmax'))]:
    x_np, x_t = util.make(shape, O.BF16, seed=5)
    q = qarray.quantize(x_t, qarray.HowToQuantize(**how))
    oq = O.quantize(O.FArr(x_np, O.BF16), O.HowToQuantize(**how))
    util.assert_qarray_equal(q, oq, str(shape))
    assert np.array_equal(util.f32np(qarray.dequantize(q)), O.dequantize(oq).v)


@pytest.mark.parametrize('shape,sshape,qtype,asym', [
    ((64, 2, 128), (4, 2, 1), 'int4', True),       # two groups of reduced axes around a kept one
    ((8, 64), (2, 4), 'int8', False),              # 2-D blocks
    ((16, 2), (4, 2), 'int8', False),              # a kept inner axis shorter than a 16-byte piece
    ((256, 128, 8), (2, 2, 4), O.E4M3, False),     # three groups of reduced axes
])
def test_static_scales_of_any_tiling(shape, sshape, qtype, asym):
  """quantize_with_scale_zero_point (qarray.py:594-635) broadcasts a scale of any tiling; so does calibrate."""
  from qwix_amd.core import qarray
  x_np, x_t = util.make(shape, O.BF16, seed=sum(shape))
  s_np = O.round_to_bf16(np.abs(util.make_np(sshape, O.BF16, seed=9)) * 0.02 + 0.005)
  z_np = util.rng(4).integers(-20, 20, sshape).astype(np.int8) if asym else None
  z_t = None if z_np is None else torch.from_numpy(z_np).to(util.DEV)
  q = qarray.quantize_with_scale_zero_point(x_t, qtype, util.to_gpu(s_np, O.BF16), z_t)
  oq = O.quantize_with_scale_zero_point(O.FArr(x_np, O.BF16), qtype, O.FArr(s_np, O.BF16), z_np)
  util.assert_qarray_equal(q, oq, 'static')
  assert np.array_equal(util.f32np(qarray.dequantize(q)), O.dequantize(oq).v)
  how = dict(qtype=qtype, channelwise_axes=[a for a in range(len(shape)) if sshape[a] == shape[a]],
             tiled_axes={a: shape[a] // sshape[a] for a in range(len(shape)) if 1 < sshape[a] < shape[a]},
             calibration_method='minmax' if asym else 'absmax')
  got, want = qarray.calibrate(x_t, qarray.HowToQuantize(**how)), O.calibrate(O.FArr(x_np, O.BF16), O.HowToQuantize(**how))
  for k in want:
    assert np.array_equal(util.f32np(got[k]), want[k].v), k


@pytest.mark.parametrize('shape,how', [
    ((2, 1024, 3), dict(channelwise_axes=[0, 2], tiled_axes={1: 128})),
    ((16, 5), dict(channelwise_axes=[1])),
    ((6, 4, 7), dict(channelwise_axes=[0], calibration_method='minmax')),
])
def test_int4_with_an_odd_last_axis(shape, how):
  """Packed int4 pairs need an axis of even length; when the last axis is odd another one carries them."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  x_np, x_t = util.make(shape, O.BF16, seed=sum(shape))
  q = qarray.quantize(x_t, qarray.HowToQuantize(qtype='int4', **how))
  oq = O.quantize(O.FArr(x_np, O.BF16), O.HowToQuantize(qtype='int4', **how))
  assert q.qvalue.packed_axis != len(shape) - 1
  util.assert_qarray_equal(q, oq, 'int4')
  assert np.array_equal(util.f32np(qarray.dequantize(q)), O.dequantize(oq).v)
  if len(shape) == 2:  # and it multiplies: contracted over the first axis against an int8 activation
    a_np, a_t = util.make((8, shape[0]), O.BF16, seed=3)
    aq = qarray.quantize(a_t, qarray.HowToQuantize(qtype='int8', channelwise_axes=[0]))
    oaq = O.quantize(O.FArr(a_np, O.BF16), O.HowToQuantize(qtype='int8', channelwise_axes=[0]))
    dn = (((1,), (0,)), ((), ()))
    assert np.array_equal(util.f32np(dg.dot_general(aq, q, dn)), O.dot_general(oaq, oq, dn).v)
