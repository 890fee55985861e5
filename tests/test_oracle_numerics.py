"""Pins the CPU oracle's numerics (no GPU needed).

Sources of truth, none of which is the oracle's own formula retyped:
  * the reference's known-answer vectors (tests/golden/known_answers.json),
  * torch-CPU's bf16 / float8_e4m3fn / rounding arithmetic (an independent
    implementation that is present offline), swept over all 2^16 bf16 patterns,
  * brute-force Python loops on tiny shapes,
  * closed forms.
"""
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import qwix_oracle as O

GOLD = json.load(
    open(os.path.join(os.path.dirname(__file__), 'golden', 'known_answers.json'))
)


def all_bf16() -> torch.Tensor:
  bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.uint16)
  return bits.view(torch.bfloat16)


def t2f(t: torch.Tensor) -> np.ndarray:
  return t.to(torch.float32).numpy()


# ---------------------------------------------------------------- dtype emulation


def test_round_to_bf16_matches_torch_everywhere():
  rng = np.random.default_rng(0)
  bits = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
  # add hand-picked ties and edge patterns
  edge = np.array(
      [0x3F808000, 0x3F818000, 0x3F80FFFF, 0x7F7FFFFF, 0x7F800000, 0xFF800000,
       0x00000001, 0x80000001, 0x00008000, 0x00018000, 0x7FC00001, 0x3F807FFF],
      np.uint32,
  )
  bits = np.concatenate([bits, edge])
  x = bits.view(np.float32)
  want = torch.from_numpy(x.copy()).to(torch.bfloat16).to(torch.float32).numpy()
  got = O.round_to_bf16(x)
  assert np.array_equal(np.isnan(want), np.isnan(got))
  m = ~np.isnan(want)
  assert np.array_equal(want[m].view(np.uint32), got[m].view(np.uint32))


def test_e4m3_decode_table_matches_torch():
  bits = torch.arange(256, dtype=torch.int32).to(torch.uint8)
  want = bits.view(torch.float8_e4m3fn).to(torch.float32).numpy()
  got = O.e4m3_to_f32(bits.numpy())
  assert np.array_equal(np.isnan(want), np.isnan(got))
  assert np.array_equal(want[~np.isnan(want)], got[~np.isnan(got)])


def test_e4m3_encode_matches_torch_on_all_bf16_and_random_f32():
  xs = [t2f(all_bf16())]
  rng = np.random.default_rng(1)
  xs.append((rng.standard_normal(500_000) * 100).astype(np.float32))
  xs.append((rng.standard_normal(500_000) * 0.01).astype(np.float32))
  # exact ties between neighbouring e4m3 values, and subnormal ties
  vals = O.E4M3_TABLE[:0x7F].astype(np.float64)
  ties = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)
  xs.append(np.concatenate([ties, -ties]))
  for x in xs:
    x = x[np.abs(x) <= 448.0]  # the path always clips first
    want = torch.from_numpy(x.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = O.f32_to_e4m3_bits(x)
    assert np.array_equal(want, got)


# ---------------------------------------------------------------- numerics.py


@pytest.mark.parametrize('case', GOLD['convert_to'])
def test_convert_to_reference_vectors(case):
  x = np.array([float(v) for v in case['x']], np.float32)
  got = O.convert_to(x, case['qtype'])
  assert got.tolist() == case['expect'], case['src']


def test_convert_to_e4m3_reference_vector():
  case = GOLD['convert_to_e4m3'][0]
  got = O.e4m3_to_f32(O.convert_to(np.array(case['x'], np.float32), 'float8_e4m3fn'))
  assert got.tolist() == case['expect_value']


def test_bounds_reference_values():
  for k, v in GOLD['symmetric_bound'].items():
    assert O.get_symmetric_bound(k) == v
  for k, v in GOLD['asymmetric_bound'].items():
    assert list(O.get_asymmetric_bound(k)) == v
  with pytest.raises(ValueError, match="doesn't support asymmetric"):
    O.get_asymmetric_bound('float8_e4m3fn')


def test_convert_to_half_to_even_and_saturation_closed_form():
  x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, -128.5, 1e30, np.nan], np.float32)
  assert O.convert_to(x, 'int8').tolist() == [0, 2, 2, 0, -2, -2, 126, 127, -128, 127, 0]
  x4 = np.array([6.5, 7.5, -8.5, 7.49, -7.5], np.float32)
  assert O.convert_to(x4, 'int4').tolist() == [6, 7, -8, 7, -8]


# ------------------------------------------- quantize on all bf16 values vs torch


@pytest.mark.parametrize('qtype,qmax,lo,hi', [('int8', 127.5, -128, 127), ('int4', 7.5, -8, 7)])
@pytest.mark.parametrize('absmax', [1.0, 0.0337, 3.14159, 1000.0, 2.0**-70, 65280.0])
def test_int_quantize_all_bf16_vs_torch(qtype, qmax, lo, hi, absmax):
  """scale = bf16(absmax/qmax); q = sat(rint(bf16(x/scale))) for every finite bf16 x."""
  xb = all_bf16()
  am = torch.tensor(absmax, dtype=torch.bfloat16)
  xb = xb[torch.isfinite(xb) & (xb.abs() <= am)]
  # torch-CPU bf16 ops compute in f32 and round to bf16 per op.
  scale_t = am / torch.tensor(qmax, dtype=torch.bfloat16)
  if float(scale_t) < 2.0**-63:
    scale_t = torch.ones_like(scale_t)
  q_t = torch.clamp(torch.round(xb / scale_t), lo, hi).to(torch.int8).numpy()

  x = O.FArr(np.concatenate([t2f(xb), [float(am)]]).astype(np.float32), O.BF16)
  qa = O.quantize(x, O.HowToQuantize(qtype=qtype))
  assert float(qa.scale.v.reshape(())) == float(scale_t)
  assert np.array_equal(qa.qvalue[:-1], q_t)


@pytest.mark.parametrize('absmax', [1.0, 0.0337, 57.0, 448.0, 30000.0])
def test_e4m3_quantize_all_bf16_vs_torch(absmax):
  xb = all_bf16()
  am = torch.tensor(absmax, dtype=torch.bfloat16)
  xb = xb[torch.isfinite(xb) & (xb.abs() <= am)]
  scale_t = am / torch.tensor(448.0, dtype=torch.bfloat16)
  q_t = torch.clamp(xb / scale_t, -448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
  x = O.FArr(np.concatenate([t2f(xb), [float(am)]]).astype(np.float32), O.BF16)
  qa = O.quantize(x, O.HowToQuantize(qtype='float8_e4m3fn'))
  assert float(qa.scale.v.reshape(())) == float(scale_t)
  assert np.array_equal(qa.qvalue[:-1], q_t)


def test_f32_quantize_vs_torch_f32():
  rng = np.random.default_rng(3)
  x = rng.standard_normal((64, 300)).astype(np.float32)
  xt = torch.from_numpy(x)
  s = xt.abs().amax(dim=1, keepdim=True) / 127.5
  q = torch.clamp(torch.round(xt / s), -128, 127).to(torch.int8).numpy()
  qa = O.quantize(O.FArr(x), O.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  assert np.array_equal(qa.scale.v, s.numpy())
  assert np.array_equal(qa.qvalue, q)


def test_zero_rows_get_scale_one():
  x = np.zeros((3, 8), np.float32)
  x[1] = 2.0
  for d in (O.F32, O.BF16):
    qa = O.quantize(O.FArr(x, d), O.HowToQuantize(qtype='int8', channelwise_axes=[0]))
    assert qa.scale.v[:, 0].tolist()[0] == 1.0 and qa.scale.v[2, 0] == 1.0
    assert not qa.qvalue[0].any() and not qa.qvalue[2].any()


# ------------------------------------------- reference vector: exact minmax int8


@pytest.mark.parametrize('with_error', [False, True])
def test_exact_minmax_quantization_reference_vector(with_error):
  """qarray_test.py:191-219."""
  a = (np.arange(256) / 255.0).astype(np.float32)
  if with_error:
    a = a + np.random.default_rng(42).uniform(-1e-7, 1e-7, a.shape).astype(np.float32)
  qa = O.quantize(O.FArr(a), O.HowToQuantize(qtype='int8', calibration_method='minmax'))
  assert qa.zero_point.reshape(()).item() == -128
  assert np.array_equal(qa.qvalue, np.arange(-128, 128).astype(np.int8))
  dq = O.dequantize(qa).v
  assert np.allclose(dq, a, atol=1e-6 if with_error else 1e-8, rtol=1e-5)


# ------------------------------------------- tiled calibrate: brute force loops


def _brute_quantize(x, cw, tiled, qtype, dtype):
  """Per-element Python loops: find the tile of each element, absmax it."""
  qmax = {'int8': 127.5, 'int4': 7.5}[qtype]
  lo, hi = {'int8': (-128, 127), 'int4': (-8, 7)}[qtype]
  tile = []
  for ax, d in enumerate(x.shape):
    tile.append(1 if ax in cw else tiled.get(ax, d))
  sshape = tuple(d // t for d, t in zip(x.shape, tile))
  am = np.zeros(sshape, np.float32)
  for idx in np.ndindex(*x.shape):
    s = tuple(i // t for i, t in zip(idx, tile))
    am[s] = max(am[s], abs(float(x[idx])))
  rt = (lambda v: float(torch.tensor(v, dtype=torch.float32).to(torch.bfloat16))) if dtype == O.BF16 else (lambda v: float(np.float32(v)))
  scale = np.zeros(sshape, np.float32)
  for s in np.ndindex(*sshape):
    v = rt(np.float32(am[s]) / np.float32(qmax))
    scale[s] = 1.0 if v < 2.0**-63 else v
  q = np.zeros(x.shape, np.int8)
  for idx in np.ndindex(*x.shape):
    s = tuple(i // t for i, t in zip(idx, tile))
    v = rt(np.float32(x[idx]) / np.float32(scale[s]))
    r = round(v)  # Python round is half-to-even
    q[idx] = min(max(r, lo), hi)
  return q, scale


@pytest.mark.parametrize('dtype', [O.F32, O.BF16])
@pytest.mark.parametrize(
    'shape,cw,tiled',
    [
        ((4, 12), [0], {}),
        ((12, 5), [1], {0: 4}),
        ((8, 8), [], {0: 4, 1: 2}),
        ((2, 2, 6), [0], {2: 2}),
        ((6, 4), [], {}),
        ((3, 8, 4), [0, 2], {1: 4}),
    ],
)
def test_tiled_quantize_vs_bruteforce(shape, cw, tiled, dtype):
  rng = np.random.default_rng(hash((shape, dtype)) % 2**32)
  x = rng.standard_normal(shape).astype(np.float32) * 3
  if dtype == O.BF16:
    x = O.round_to_bf16(x)
  for qtype in ('int8', 'int4'):
    qa = O.quantize(O.FArr(x, dtype), O.HowToQuantize(qtype=qtype, channelwise_axes=cw, tiled_axes=tiled))
    q, scale = _brute_quantize(x, cw, tiled, qtype, dtype)
    assert qa.scale.shape == scale.shape
    assert np.array_equal(qa.scale.v, scale)
    assert np.array_equal(qa.qvalue, q)


def test_float_tile_size_means_one_over_count():
  x = np.arange(48, dtype=np.float32).reshape(4, 12)
  how = O.HowToQuantize(qtype='int8', channelwise_axes=[0], tiled_axes={1: 1 / 3})
  assert O.get_scale_shape(x.shape, how) == (4, 3)
  with pytest.raises(ValueError, match='cannot be tiled'):
    O.get_scale_shape((4, 10), O.HowToQuantize(qtype='int8', tiled_axes={1: 4}))
  with pytest.raises(ValueError, match='both channelwise and tiled'):
    O.get_scale_shape((4, 8), O.HowToQuantize(qtype='int8', channelwise_axes=[1], tiled_axes={1: 4}))


@pytest.mark.parametrize('case', GOLD['scale_shapes'])
def test_scale_shapes_reference(case):
  how = O.HowToQuantize(
      qtype='int8',
      channelwise_axes=case['channelwise_axes'],
      tiled_axes={int(k): v for k, v in case['tiled_axes'].items()},
  )
  assert list(O.get_scale_shape(case['shape'], how)) == case['expect'], case['src']


def test_get_tiled_axes_reference():
  c = GOLD['get_tiled_axes']
  qa = O.QArray(np.ones(c['qvalue_shape'], np.int8), O.FArr(np.ones(c['scale_shape'], np.float32)))
  assert O.get_tiled_axes(qa) == {int(k): v for k, v in c['expect'].items()}


def test_minmax_bf16_vs_torch():
  rng = np.random.default_rng(5)
  x = O.round_to_bf16(rng.standard_normal((16, 64)).astype(np.float32) + 0.3)
  xt = torch.from_numpy(x).to(torch.bfloat16)
  mn = torch.clamp(xt.amin(dim=1, keepdim=True), max=0)
  mx = torch.clamp(xt.amax(dim=1, keepdim=True), min=0)
  scale = (mx - mn) / torch.tensor(255.0, dtype=torch.bfloat16)
  zp_f = torch.tensor(-128.0, dtype=torch.bfloat16) - mn / scale
  zp = torch.clamp(torch.round(zp_f), -128, 127)
  q = torch.clamp(torch.round(xt / scale + zp.to(torch.bfloat16)), -128, 127).to(torch.int8)
  qa = O.quantize(O.FArr(x, O.BF16), O.HowToQuantize(qtype='int8', channelwise_axes=[0], calibration_method='minmax'))
  assert np.array_equal(qa.scale.v, t2f(scale))
  assert np.array_equal(qa.zero_point, zp.to(torch.int8).numpy())
  assert np.array_equal(qa.qvalue, q.numpy())


def test_quantize_api_scale_dtype_cast_happens_after():
  rng = np.random.default_rng(6)
  x = O.round_to_bf16(rng.standard_normal((256, 8)).astype(np.float32) * 0.02)
  qa = O.quantize_api(O.FArr(x, O.BF16), 'int4', channelwise_axes=[1], tiled_axes={0: 128}, scale_dtype=O.F32)
  assert qa.scale.dtype == O.F32 and qa.scale.shape == (2, 8)
  assert np.array_equal(O.round_to_bf16(qa.scale.v), qa.scale.v)  # bf16-representable
  qb = O.quantize_api(O.FArr(x, O.BF16), 'int4', channelwise_axes=[1], tiled_axes={0: 128})
  assert np.array_equal(qa.qvalue, qb.qvalue)


def test_dequantize_closed_form():
  q = np.array([[-8, 7, 3, 0]], np.int8)
  s = O.FArr(np.array([[0.5, 0.25]], np.float32), O.BF16)
  dq = O.dequantize(O.QArray(q, s, None, 'int4'))
  assert dq.dtype == O.BF16 and dq.v.tolist() == [[-4.0, 3.5, 0.75, 0.0]]
  zp = np.array([[1, -1]], np.int8)
  dq = O.dequantize(O.QArray(q, s, zp, 'int4'))
  assert dq.v.tolist() == [[-4.5, 3.0, 1.0, 0.25]]


def test_fixed_calibration_closed_form():
  """qarray.py:518-532: 'fixed,a' is a per-tensor absmax of a, 'fixed,a,b' a per-tensor (min, max); with
  a = 127.5 the int8 scale is exactly 1 and quantize reduces to convert_to (numerics_test.py:34-50)."""
  x = O.FArr(np.array([[1.2, 3.5, -127.5, 129.0, -1300.0]], np.float32), O.F32)
  how = O.HowToQuantize(qtype='int8', channelwise_axes=[0], calibration_method='fixed,127.5')
  cal = O.calibrate(x, how)
  assert set(cal) == {'absmax'} and cal['absmax'].v.shape == (1, 1) and cal['absmax'].v.item() == 127.5
  q = O.quantize(x, how)
  assert q.scale.v.shape == (1, 1) and q.scale.v.item() == 1.0
  assert q.qvalue.tolist() == [[1, 4, -128, 127, -128]]
  # asymmetric: range [-1, 3] on int8 -> scale = 4/255, zero point = rint(-128 + 1/scale) = -64
  how = O.HowToQuantize(qtype='int8', calibration_method='fixed,-1,3')
  q = O.quantize(O.FArr(np.array([[-1.0, 0.0, 3.0, 10.0]], np.float32), O.F32), how)
  s = np.float32(4.0) / np.float32(255.0)
  assert q.scale.v.item() == s
  assert q.zero_point.item() == int(np.rint(np.float32(-128.0) - np.float32(-1.0) / s))
  assert q.qvalue.tolist() == [[-128, int(q.zero_point.item()), 127, 127]]
  for bad in ('fixed', 'fixed,1,2', 'fixed,-1,-0.5', 'fixed,0,0'):
    with pytest.raises(ValueError):
      O.calibrate(x, O.HowToQuantize(qtype='int8', calibration_method=bad))


def test_rms_calibration_closed_forms():
  """qarray.py:511-515: rms of a constant array is |c|, of (+a, -a, +a, ...) is a; the factor multiplies it."""
  x = O.FArr(np.full((4, 64), -0.75, np.float32), O.BF16)
  how = O.HowToQuantize(qtype='int8', channelwise_axes=[0], calibration_method='rms,7')
  cal = O.calibrate(x, how)
  assert set(cal) == {'absmax'} and cal['absmax'].v.shape == (4, 1) and np.all(cal['absmax'].v == 0.75 * 7)
  alt = np.tile(np.array([2.0, -2.0], np.float32), (3, 16))
  cal = O.calibrate(O.FArr(alt, O.F32), O.HowToQuantize(qtype='int8', channelwise_axes=[0], tiled_axes={1: 8},
                                                         calibration_method='rms,0.5'))
  assert cal['absmax'].v.shape == (3, 4) and np.all(cal['absmax'].v == 1.0)
  with pytest.raises(ValueError, match='scale factor'):
    O.calibrate(x, O.HowToQuantize(qtype='int8', calibration_method='rms'))


def test_stochastic_rounding_noise_is_added_in_float32():
  """numerics.py:191-195: the noise meets the scaled value in float32, not in the array dtype.  The reference's own
  example: bf16(41) - 0.4 rounds to 41 (40.6), where bf16 arithmetic would give round(40.5) = 40.  Brute force on a
  small grid: the rounding is floor(v + noise + 0.5) away from ties for every value and noise."""
  x = O.FArr(np.array([[41.0, -41.0, 3.0, 0.0]], np.float32), O.BF16)
  one = O.FArr(np.ones((1, 1), np.float32), O.BF16)
  noise = np.array([[-0.4, 0.4, 0.49, -0.49]], np.float32)
  q = O.quantize_with_scale_zero_point(x, 'int8', one, None, noise)
  assert q.qvalue.tolist() == [[41, -41, 3, 0]]
  assert O.round_to_bf16(np.float32(41.0) - np.float32(0.4)) == 40.5   # what the bf16 sum would have been
  # zero noise is the plain rounding; float qtypes ignore the noise
  g = np.random.Generator(np.random.PCG64(5))
  v = O.round_to_bf16((g.standard_normal((8, 64)) * 40).astype(np.float32))
  for qtype in ('int8', 'int4'):
    assert np.array_equal(O.convert_to(v, qtype, np.zeros_like(v)), O.convert_to(v, qtype))
  assert np.array_equal(O.convert_to(v, 'float8_e4m3fn', np.full_like(v, 0.3)), O.convert_to(v, 'float8_e4m3fn'))
  # brute force, element by element, in Python floats restricted to float32 steps
  nz = g.uniform(-0.5, 0.5, v.shape).astype(np.float32)
  got = O.convert_to(v, 'int8', nz)
  for a, b, c in zip(v.ravel(), nz.ravel(), got.ravel()):
    s = float(np.float32(a) + np.float32(b))
    lo = np.floor(s)
    want = lo if s - lo < 0.5 else lo + 1 if s - lo > 0.5 else (lo if lo % 2 == 0 else lo + 1)
    assert c == int(min(max(want, -128), 127))
  # saturation and the zero point still apply: the zero point is added in the array dtype, before the noise
  xs = O.FArr(np.array([[300.0, -300.0, 10.0]], np.float32), O.F32)
  qz = O.quantize_with_scale_zero_point(xs, 'int8', O.FArr(np.ones((1, 1), np.float32), O.F32),
                                        np.array([[5]], np.int8), np.array([[0.3, -0.3, 0.4]], np.float32))
  assert qz.qvalue.tolist() == [[127, -128, 15]]
