"""CPU oracle: a NumPy restatement of Qwix's quantize + quantized dot_general path.

THIS FILE IS TEST INFRASTRUCTURE.  It exists only to check the HIP kernels.
Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may
import it; nothing under qwix_amd/ does.

What it restates (file:line refer to the google/qwix v0.1.8 source tree):

  numerics    qwix/_src/core/numerics.py:64-196      bounds, convert_to
  qarray      qwix/_src/core/qarray.py:332-349       get_scale_shape
              qwix/_src/core/qarray.py:390-444       split_axis, generic broadcast
              qwix/_src/core/qarray.py:470-534       calibrate (absmax / minmax / rms / fixed)
              qwix/_src/core/qarray.py:537-584       compute_scale_zero_point
              qwix/_src/core/qarray.py:594-644       quantize_with_scale_zero_point, quantize
              qwix/_src/core/qarray.py:647-708       quantize_api, dequantize
              qwix/_src/core/qarray.py:781-821       get_accumulator_and_result_type
  dot_general qwix/_src/core/dot_general.py:28-76    get_how_to_quantize
              qwix/_src/core/dot_general.py:135-275  _fast_dot_general, _slow_dot_general
              qwix/_src/core/dot_general.py:407-491  dispatcher
  ragged_dot  qwix/_src/core/ragged_dot.py:123-353   quantized / dequantize-first ragged dot
  einsum      qwix/_src/core/einsum.py:27-103        get_how_to_quantize, binary einsum
              qwix/_src/core/einsum_info.py:26-174   EinsumInfo
  hadamard    qwix/contrib/hadamard_rot.py:35-190    Sylvester matrix, sign flips, rotate

The arithmetic of the reference lives in JAX/XLA (not part of that tree, and not
installed where this oracle was written), so the restatement encodes *eager,
op-by-op* XLA:CPU semantics: every elementwise op on a bf16 array is computed in
f32 and rounded to bf16 (round-to-nearest-even) before the next op; float ->
int casts saturate; int32 -> bf16 goes through f32.

How each function is pinned (tests/test_oracle_*.py):
  * convert_to, bounds ............. the reference's known-answer vectors
    (tests/_src/core/numerics_test.py:34-88,133-143) + an exhaustive sweep of all
    2^16 bf16 bit patterns against torch-CPU's independent casts.
  * calibrate / scale / quantize ... reference vector qarray_test.py:191-219
    (arange(256)/255, minmax) + closed forms + brute-force Python loops on tiny
    tiled shapes + torch-CPU bf16 arithmetic as an independent implementation.
  * calibrate 'fixed' .............. closed forms (scale exactly 1 reproduces the convert_to vectors).
  * calibrate 'rms' ................ PARITY UNPINNED in its last bit: jnp.mean of the rounded squares is an
    f32 sum in XLA's own order; pinned only by closed forms (constant arrays) and to one ulp.
  * integer dot ..................... exact integer arithmetic (any order agrees);
    checked against np.int64 matmul.
  * _fast == _slow == dequant-dot ... invariant of two_dim_scales_test.py:57-93.
  * dtype rule, tiling heuristics, EinsumInfo ... the reference's tables
    (dot_general_test.py:28-146,175-197; einsum_info_test.py).
  * ragged dot ...................... reduces, group by group, to the pinned dot_general on
    row slices; brute-force loops on tiny inputs; empty groups, rows of no group, groups
    reaching past the last row (the group_sizes of ragged_dot_test.py:36-80).
  * hadamard ........................ H H^T = n I, (xH)(H^T w / n) = x w
    (hadamard_rot_test.py:24-41,92-147), popcount closed form.

PARITY UNPINNED (nothing available offline fixes these; stated tolerance instead):
  * the accumulation order / internal precision of XLA:CPU's bf16 and fp8
    `dot_general` (fp8 GEMM accumulator; the dense x @ H of hadamard_rot) -- the
    oracle accumulates exactly (f64) and rounds once via f32;
  * NaN -> integer casts (the oracle gives 0);
  * whether `jit` elides the bf16 round trips (the oracle is the eager contract);
  * jax.random-derived inputs and sign vectors: sign vectors are *inputs* here.
"""

from __future__ import annotations

import dataclasses
import math
import re
from typing import Mapping, Sequence

import numpy as np

F32 = 'f32'
BF16 = 'bf16'
INT8 = 'int8'
INT4 = 'int4'
E4M3 = 'float8_e4m3fn'
INT32 = 'int32'

_FLOAT_DTYPES = (BF16, F32)
_INT_QTYPES = (INT8, INT4)


# ----------------------------------------------------------------------------
# dtype emulation
# ----------------------------------------------------------------------------


def round_to_bf16(x) -> np.ndarray:
  """RNE f32 -> bf16, returned as f32 holding bf16-representable values."""
  shape = np.shape(x)  # ascontiguousarray turns a 0-d array into one of shape (1,)
  x = np.ascontiguousarray(x, dtype=np.float32)
  u = x.view(np.uint32).astype(np.uint64)
  bias = ((u >> 16) & 1) + 0x7FFF
  r = ((u + bias) & 0xFFFF0000).astype(np.uint32)
  r = np.where(np.isnan(x), np.uint32(0x7FC00000), r).astype(np.uint32)
  return r.view(np.float32).reshape(shape)


def rnd(x, dtype: str) -> np.ndarray:
  """Round an f32-computed result into `dtype` (kept in an f32 container)."""
  if dtype == F32:
    return np.asarray(x, dtype=np.float32)
  if dtype == BF16:
    return round_to_bf16(x)
  raise ValueError(f'unsupported float dtype {dtype}')


def promote(a: str, b: str) -> str:
  """jnp.result_type restricted to {int32, bf16, f32}."""
  if a == b:
    return a
  if F32 in (a, b):
    return F32
  if BF16 in (a, b):
    return BF16
  raise ValueError(f'cannot promote {a} {b}')


@dataclasses.dataclass
class FArr:
  """A float array of dtype bf16 or f32; `v` always holds f32 storage."""

  v: np.ndarray
  dtype: str = F32

  def __post_init__(self):
    self.v = np.asarray(self.v, dtype=np.float32)
    if self.dtype == BF16:
      assert np.array_equal(
          round_to_bf16(self.v), self.v, equal_nan=True
      ), 'values are not bf16-representable'

  shape = property(lambda self: self.v.shape)
  ndim = property(lambda self: self.v.ndim)

  def astype(self, dtype: str) -> 'FArr':
    return FArr(rnd(self.v, dtype), dtype)

  def reshape(self, *shape) -> 'FArr':
    return FArr(self.v.reshape(*shape), self.dtype)


# --- float8_e4m3fn (OCP): 1-4-3, bias 7, no inf, NaN = S.1111.111, max 448 ---


def _e4m3_table() -> np.ndarray:
  t = np.zeros(256, np.float32)
  for b in range(256):
    s = -1.0 if b & 0x80 else 1.0
    e = (b >> 3) & 0xF
    m = b & 7
    if e == 0xF and m == 7:
      t[b] = np.nan
    elif e == 0:
      t[b] = s * (m / 8.0) * 2.0**-6
    else:
      t[b] = s * (1 + m / 8.0) * 2.0 ** (e - 7)
  return t


E4M3_TABLE = _e4m3_table()


def e4m3_to_f32(bits) -> np.ndarray:
  return E4M3_TABLE[np.asarray(bits, dtype=np.uint8)]


def f32_to_e4m3_bits(x) -> np.ndarray:
  """RNE f32 -> e4m3fn bit patterns.  |x| > 448 after rounding -> NaN (0x7f)."""
  x = np.asarray(x, dtype=np.float32)
  a = np.abs(x).astype(np.float64)
  sign = np.signbit(x).astype(np.uint8) << 7
  out = np.zeros(x.shape, np.uint8)
  # Exponent of the quantisation step: normal numbers have 3 mantissa bits,
  # subnormals share the step 2^-9.
  with np.errstate(divide='ignore', invalid='ignore'):
    e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
  e = np.maximum(e, -6.0)
  step = 2.0 ** (e - 3)
  q = np.rint(a / step) * step  # np.rint is half-to-even; a/step is exact.
  # Encode q (exactly representable, maybe one binade up after rounding).
  with np.errstate(divide='ignore', invalid='ignore'):
    e2 = np.floor(np.log2(np.where(q > 0, q, 1.0)))
  is_sub = q < 2.0**-6
  exp_field = np.where(is_sub, 0, e2 + 7).astype(np.int64)
  man = np.where(is_sub, q / 2.0**-9, (q / 2.0**e2 - 1.0) * 8.0)
  man = np.rint(man).astype(np.int64)
  code = (exp_field << 3) | man
  code = np.where(q > 448.0, 0x7F, code)
  out = (code.astype(np.uint8) & 0x7F) | sign
  out = np.where(np.isnan(x), np.uint8(0x7F) | sign, out)
  return out.astype(np.uint8)


# ----------------------------------------------------------------------------
# numerics.py
# ----------------------------------------------------------------------------


def canonical_qtype(qtype) -> str:
  s = str(qtype)
  s = s.replace('torch.', '').replace('jnp.', '')
  if s in ('int8', 'int4'):
    return s
  if s in ('float8_e4m3fn', 'e4m3', 'fp8', 'float8_e4m3'):
    return E4M3
  raise ValueError(f'qtype {qtype} is outside the restated path')


def get_asymmetric_bound(qtype) -> tuple[float, float]:
  """numerics.py:64-92."""
  q = canonical_qtype(qtype)
  if q == INT8:
    return (-128.0, 127.0)
  if q == INT4:
    return (-8.0, 7.0)
  raise ValueError(f"{qtype} doesn't support asymmetric quantization.")


def get_symmetric_bound(qtype) -> float:
  """numerics.py:95-136: iinfo.max + 0.5 for ints, finfo.max for floats."""
  q = canonical_qtype(qtype)
  return {INT8: 127.5, INT4: 7.5, E4M3: 448.0}[q]


def convert_to(x: np.ndarray, qtype, noise: np.ndarray | None = None) -> np.ndarray:
  """numerics.py:139-196 for int8 / int4 / e4m3.  `noise` (what the reference's noise_fn(x.shape) returned): added in
  float32 before the rounding to an integer type (numerics.py:191-195); float types ignore it, as the reference does.

  ints: round-half-even then a saturating cast (XLA convert semantics:
  out-of-range and +-inf clamp to the bounds; NaN -> 0, unpinned).
  e4m3: clip to +-448 in the input dtype, then RNE cast.
  Returns int8 values (int8/int4) or uint8 bit patterns (e4m3).
  """
  q = canonical_qtype(qtype)
  x = np.asarray(x, dtype=np.float32)
  if q == E4M3:
    # jnp.clip propagates NaN.
    c = np.where(np.isnan(x), x, np.clip(x, -448.0, 448.0))
    return f32_to_e4m3_bits(c)
  qmin, qmax = get_asymmetric_bound(q)
  if noise is not None:
    x = (x + np.asarray(noise, dtype=np.float32)).astype(np.float32)
  r = np.rint(x)
  r = np.where(np.isnan(r), 0.0, np.clip(r, qmin, qmax))
  return r.astype(np.int8)


# ----------------------------------------------------------------------------
# qarray.py
# ----------------------------------------------------------------------------


@dataclasses.dataclass(frozen=True)
class HowToQuantize:
  """qarray.py:280-325."""

  qtype: str
  channelwise_axes: Sequence[int] = ()
  tiled_axes: Mapping[int, int | float] = dataclasses.field(default_factory=dict)
  calibration_method: str = 'absmax'


@dataclasses.dataclass
class QArray:
  """qarray.py:31-99.  qvalue: int8 ndarray (int8/int4) or uint8 bits (e4m3)."""

  qvalue: np.ndarray
  scale: FArr
  zero_point: np.ndarray | None = None
  qtype: str = INT8

  shape = property(lambda self: self.qvalue.shape)
  ndim = property(lambda self: self.qvalue.ndim)
  dtype = property(lambda self: self.scale.dtype)


def _tile_size(dim: int, tile) -> int:
  if isinstance(tile, float):
    tile = round(dim * tile)
  return tile


def get_scale_shape(array_shape, how: HowToQuantize) -> tuple[int, ...]:
  """qarray.py:332-349."""
  if set(how.channelwise_axes) & set(how.tiled_axes.keys()):
    raise ValueError('The same axis cannot be both channelwise and tiled.')
  out = []
  for axis, dim in enumerate(array_shape):
    if axis in how.channelwise_axes:
      out.append(dim)
    elif axis in how.tiled_axes:
      t = _tile_size(dim, how.tiled_axes[axis])
      if t <= 0 or dim % t != 0:
        raise ValueError(f'{array_shape} cannot be tiled as {how.tiled_axes}.')
      out.append(dim // t)
    else:
      out.append(1)
  return tuple(out)


def split_axis(v: np.ndarray, tiled_axes: Mapping[int, int | float]) -> np.ndarray:
  """qarray.py:390-406."""
  new_shape = []
  for axis, dim in enumerate(v.shape):
    if axis in tiled_axes:
      t = _tile_size(dim, tiled_axes[axis])
      if dim % t != 0:
        raise ValueError(f'{v.shape} cannot be tiled as {tiled_axes}.')
      new_shape += [dim // t, t]
    else:
      new_shape.append(dim)
  return v.reshape(new_shape)


def get_tiled_axes(array: QArray) -> dict[int, int]:
  """qarray.py:409-422."""
  return {
      i: j // k
      for i, (j, k) in enumerate(zip(array.qvalue.shape, array.scale.shape))
      if j != k and k != 1
  }


def generic_broadcast(op, x: np.ndarray, y: np.ndarray) -> np.ndarray:
  """qarray.py:425-444."""
  assert x.ndim == y.ndim
  xs, ys, os_ = [], [], []
  for a, b in zip(x.shape, y.shape):
    os_.append(max(a, b))
    if a == b or a == 1 or b == 1:
      xs.append(a)
      ys.append(b)
    elif a % b == 0:
      xs += [b, a // b]
      ys += [b, 1]
    elif b % a == 0:
      xs += [a, 1]
      ys += [a, b // a]
    else:
      raise ValueError(f'Cannot broadcast between {x.shape} {y.shape}')
  return op(x.reshape(xs), y.reshape(ys)).reshape(os_)


def calibrate(array: FArr, how: HowToQuantize) -> dict[str, FArr]:
  """qarray.py:470-534: the absmax, minmax, rms and fixed methods."""
  reduce_axes = []
  off = 0
  for axis in range(array.ndim):
    if axis in how.channelwise_axes:
      continue
    if axis in how.tiled_axes:
      off += 1
    reduce_axes.append(axis + off)
  shape = get_scale_shape(array.shape, how)
  v = split_axis(array.v, how.tiled_axes)
  method, *args = how.calibration_method.lower().split(',')
  args = [float(a) for a in args]
  ax = tuple(reduce_axes)
  d = array.dtype
  if method == 'minmax':
    mn = np.minimum(np.min(v, axis=ax, keepdims=True), np.float32(0))
    mx = np.maximum(np.max(v, axis=ax, keepdims=True), np.float32(0))
    if args:
      f = rnd(np.float32(args[0]), d)  # weak Python scalar adopts the array dtype
      mn = rnd(mn * f, d)
      mx = rnd(mx * f, d)
    return {'min': FArr(mn.reshape(shape), d), 'max': FArr(mx.reshape(shape), d)}
  if method == 'absmax':
    am = np.max(np.abs(v), axis=ax, keepdims=True)
    if args:
      am = rnd(am * rnd(np.float32(args[0]), d), d)
    return {'absmax': FArr(am.reshape(shape), d)}
  if method == 'rms':  # qarray.py:511-515.  Parity unpinned in its last bit: jnp.mean sums in f32 in XLA's own order
    if not args:
      raise ValueError('A scale factor is required for RMS calibration.')
    sq = rnd(v * v, d)
    n = np.float32(np.prod([v.shape[a] for a in ax]))
    mean = rnd(np.sum(sq, axis=ax, keepdims=True, dtype=np.float32) / n, d)
    rms = rnd(np.sqrt(mean), d)
    return {'absmax': FArr(rnd(rms * rnd(np.float32(args[0]), d), d).reshape(shape), d)}
  if method == 'fixed':  # qarray.py:518-532: a constant, per-tensor range
    if len(args) not in (1, 2):
      raise ValueError('A fixed range is required for fixed calibration.')
    if len(args) == 1:
      args = (-args[0], args[0])
    if args[0] > 0 or args[1] < 0 or args[0] >= args[1]:
      raise ValueError('The range must contain 0 and be non-empty.')
    ones = tuple(1 for _ in shape)
    if args[0] + args[1] == 0:
      return {'absmax': FArr(np.full(ones, rnd(np.float32(args[1]), d), np.float32), d)}
    return {'min': FArr(np.full(ones, rnd(np.float32(args[0]), d), np.float32), d),
            'max': FArr(np.full(ones, rnd(np.float32(args[1]), d), np.float32), d)}
  raise ValueError(f'Unsupported calibration: {how.calibration_method}')


_TINY_SQRT = np.float32(2.0**-63)  # sqrt(finfo.tiny) for both f32 and bf16


def compute_scale_zero_point(calibration: Mapping[str, FArr], qtype):
  """qarray.py:537-584 (symmetric and asymmetric branches)."""
  if 'min' in calibration and 'max' in calibration:
    mn, mx = calibration['min'], calibration['max']
    d = mn.dtype
    qmin, qmax = get_asymmetric_bound(qtype)
    with np.errstate(all='ignore'):
      rng = rnd(mx.v - mn.v, d)
      scale = rnd(rng / np.float32(qmax - qmin), d)
      scale = np.where(scale < _TINY_SQRT, np.float32(1), scale).astype(np.float32)
      zp = rnd(np.float32(qmin) - rnd(mn.v / scale, d), d)
    return FArr(scale, d), convert_to(zp, qtype)
  if 'absmax' in calibration:
    am = calibration['absmax']
    d = am.dtype
    with np.errstate(all='ignore'):
      scale = rnd(am.v / np.float32(get_symmetric_bound(qtype)), d)
      scale = np.where(scale < _TINY_SQRT, np.float32(1), scale).astype(np.float32)
    return FArr(scale, d), None
  raise ValueError(f'Unsupported calibration: {calibration}')


def quantize_with_scale_zero_point(
    array: FArr, qtype, scale: FArr, zero_point: np.ndarray | None, noise: np.ndarray | None = None
) -> QArray:
  """qarray.py:594-635 (true division, no reciprocal); `noise` as in convert_to."""
  if array.dtype not in _FLOAT_DTYPES:
    raise ValueError(f'Refuse to quantize: {array.dtype}')
  if zero_point is not None and zero_point.shape != scale.shape:
    raise ValueError(
        f'Expect zero_point shape {scale.shape} but got {zero_point.shape}'
    )
  d = array.dtype
  scale = scale.astype(d)
  with np.errstate(all='ignore'):
    q = rnd(generic_broadcast(np.divide, array.v, scale.v), d)
    if zero_point is not None:
      zpf = rnd(zero_point.astype(np.float32), d)
      q = rnd(generic_broadcast(np.add, q, zpf), d)
  return QArray(convert_to(q, qtype, noise), scale, zero_point, canonical_qtype(qtype))


def quantize(array: FArr, how: HowToQuantize, noise: np.ndarray | None = None) -> QArray:
  """qarray.py:638-644."""
  cal = calibrate(array, how)
  scale, zp = compute_scale_zero_point(cal, how.qtype)
  return quantize_with_scale_zero_point(array, how.qtype, scale, zp, noise)


def quantize_api(
    array: FArr,
    qtype,
    *,
    channelwise_axes=(),
    tiled_axes=None,
    calibration_method='absmax',
    scale_dtype=None,
) -> QArray:
  """qarray.py:647-689: scale cast happens after quantizing."""
  qa = quantize(
      array,
      HowToQuantize(
          qtype=qtype,
          channelwise_axes=channelwise_axes,
          tiled_axes=tiled_axes or {},
          calibration_method=calibration_method,
      ),
  )
  if scale_dtype is not None:
    qa = dataclasses.replace(qa, scale=qa.scale.astype(scale_dtype))
  return qa


def qvalue_as_f32(qa: QArray) -> np.ndarray:
  if qa.qtype == E4M3:
    return e4m3_to_f32(qa.qvalue)
  return qa.qvalue.astype(np.float32)


def dequantize(qa: QArray) -> FArr:
  """qarray.py:692-708: (qvalue.astype(S) - zp.astype(S)) * scale, S = scale dtype."""
  s = qa.scale.dtype
  q = rnd(qvalue_as_f32(qa), s)
  if qa.zero_point is not None:
    zp = rnd(qa.zero_point.astype(np.float32), s)
    q = rnd(generic_broadcast(np.subtract, q, zp), s)
  return FArr(rnd(generic_broadcast(np.multiply, q, qa.scale.v), s), s)


def _qvalue_dtype_name(x) -> str:
  if isinstance(x, QArray):
    return x.qtype
  if isinstance(x, FArr):
    return x.dtype
  return str(x.dtype)  # raw integer ndarray


def _dequant_dtype_name(x) -> str:
  if isinstance(x, QArray):
    return x.scale.dtype
  if isinstance(x, FArr):
    return x.dtype
  return str(x.dtype)


def get_accumulator_and_result_type(*args, preferred_element_type=None):
  """qarray.py:781-821."""
  qd = [_qvalue_dtype_name(a) for a in args]
  dd = [_dequant_dtype_name(a) for a in args]
  result = preferred_element_type
  if result is None:
    for i, t in enumerate(dd):
      # itemsize <= 1: 'int' in the dtype name -> int32, anything else -> bf16.
      if t in (INT8, INT4, 'uint8'):
        dd[i] = INT32
      elif t in (E4M3, 'bool'):
        dd[i] = BF16
    result = dd[0]
    for t in dd[1:]:
      if result == INT32:
        result = t
      elif t != INT32:
        result = promote(result, t)
  acc = result
  if all('int' in t for t in qd):
    acc = INT32
  return acc, result


# ----------------------------------------------------------------------------
# dot_general.py
# ----------------------------------------------------------------------------


def dg_get_how_to_quantize(
    *, dimension_numbers, ndims, for_lhs: bool, tile_size, **kwargs
) -> HowToQuantize:
  """dot_general.py:28-76."""
  if for_lhs:
    ndim, ca = ndims[0], dimension_numbers[0][0]
  else:
    ndim, ca = ndims[1], dimension_numbers[0][1]
  if isinstance(tile_size, Mapping):
    tiled = dict(tile_size)
  else:
    tiled = {ca[-1]: tile_size} if tile_size else {}
  cw = sorted(set(range(ndim)) - set(ca) - set(tiled.keys()))
  return HowToQuantize(channelwise_axes=cw, tiled_axes=tiled, **kwargs)


def _dot_general_f64(lhs, rhs, dimension_numbers) -> np.ndarray:
  """lax.dot_general in float64; output dims = batch, lhs free, rhs free."""
  (lca, rca), (lba, rba) = dimension_numbers
  lra = [a for a in range(lhs.ndim) if a not in lca and a not in lba]
  rra = [a for a in range(rhs.ndim) if a not in rca and a not in rba]
  l = np.transpose(lhs, list(lba) + lra + list(lca)).astype(np.float64)
  r = np.transpose(rhs, list(rba) + list(rca) + rra).astype(np.float64)
  bshape = l.shape[: len(lba)]
  lfree = l.shape[len(lba) : len(lba) + len(lra)]
  kshape = l.shape[len(lba) + len(lra) :]
  rfree = r.shape[len(rba) + len(rca) :]
  b = int(np.prod(bshape, dtype=np.int64))
  k = int(np.prod(kshape, dtype=np.int64))
  l2 = l.reshape(b, -1, k)
  r2 = r.reshape(b, k, -1)
  out = np.matmul(l2, r2)
  return out.reshape(tuple(bshape) + tuple(lfree) + tuple(rfree))


def _transpose_array(a: np.ndarray, transpose) -> np.ndarray:
  """qarray.py:352-387 (value semantics only)."""
  if any(l > 1 for ax, l in enumerate(a.shape) if ax not in transpose):
    raise ValueError(f'Cannot transpose {a.shape} as {transpose}.')
  used = [ax for ax in transpose if ax is not None]
  rest = [ax for ax in range(a.ndim) if ax not in used]
  t = np.transpose(a, used + rest).reshape([a.shape[ax] for ax in used])
  idx = tuple(slice(None) if ax is not None else None for ax in transpose)
  return t[idx]


def _apply_tiling(ca, ba, tiled):
  """dot_general.py:93-122."""
  new_ca = [a + sum(t <= a for t in tiled) for a in ca]
  new_ba = [a + sum(t < a for t in tiled) for a in ba]
  new_ba += [a + sum(t < a for t in tiled) for a in ca if a in tiled]
  return tuple(new_ca), tuple(new_ba), tuple(range(len(ba), len(new_ba)))


def _scale_transposes(dimension_numbers, ndims):
  """dot_general.py:79-90."""
  (lca, rca), (lba, rba) = dimension_numbers
  lra = sorted(set(range(ndims[0])) - set(lca) - set(lba))
  rra = sorted(set(range(ndims[1])) - set(rca) - set(rba))
  return (
      list(lba) + list(lra) + [None] * len(rra),
      list(rba) + [None] * len(lra) + list(rra),
  )


def _operand_fields(x):
  if isinstance(x, QArray):
    v = qvalue_as_f32(x) if x.qtype == E4M3 else x.qvalue
    return v, x.scale, x.zero_point, get_tiled_axes(x)
  if isinstance(x, FArr):
    return x.v, None, None, {}
  return np.asarray(x), None, None, {}


def fast_dot_general(
    lhs, rhs, dimension_numbers, preferred_element_type=None, return_acc=False
):
  """dot_general.py:135-261.

  Integer x integer products accumulate exactly (int32).  Otherwise the dot is
  accumulated in f64 and rounded once into the accumulator dtype (the reference
  leaves the order to XLA: unpinned, compared by tolerance).
  If return_acc, also returns the raw accumulator of the (tiled) dot.
  """
  lv, ls, lzp, lt = _operand_fields(lhs)
  rv, rs, rzp, rt = _operand_fields(rhs)
  if lzp is not None and rzp is not None:
    raise ValueError('Only one operand can be asymmetric.')
  (lca, rca), (lba, rba) = dimension_numbers
  ltc, rtc = {}, {}
  for l, r in zip(lca, rca):
    a, b = lt.get(l), rt.get(r)
    if a and b and a != b:
      raise ValueError('Contracting axes must be tiled with the same tile size.')
    if a or b:
      ltc[l] = a or b
      rtc[r] = a or b
  lv = split_axis(lv, ltc)
  rv = split_axis(rv, rtc)
  if lzp is not None:
    lzp = split_axis(lzp, {a: 1 for a in ltc})
  if rzp is not None:
    rzp = split_axis(rzp, {a: 1 for a in rtc})
  lca, lba, sum_axes = _apply_tiling(lca, lba, ltc)
  rca, rba, _ = _apply_tiling(rca, rba, rtc)
  dn = ((lca, rca), (lba, rba))
  ltr, rtr = _scale_transposes(dn, (lv.ndim, rv.ndim))
  if ls is not None:
    ls = FArr(
        _transpose_array(split_axis(ls.v, {a: 1 for a in ltc}), ltr), ls.dtype
    )
  if rs is not None:
    rs = FArr(
        _transpose_array(split_axis(rs.v, {a: 1 for a in rtc}), rtr), rs.dtype
    )
  acc_t, res_t = get_accumulator_and_result_type(
      lhs, rhs, preferred_element_type=preferred_element_type
  )

  def dot(a, b):
    d = _dot_general_f64(a, b, dn)
    if acc_t == INT32:
      assert np.all(np.abs(d) < 2**31)
      return d.astype(np.int64).astype(np.int32)
    return rnd(d.astype(np.float32), acc_t)

  res = dot(lv, rv)
  cur_t = acc_t

  def bcast(zp, shape, axes):
    tgt = list(zp.shape)
    for a in axes:
      tgt[a] = shape[a]
    return np.broadcast_to(zp, tgt)

  if lzp is not None:
    corr = dot(bcast(lzp, lv.shape, lca + lba), rv)
    res = generic_broadcast(np.subtract, res, corr)
    if cur_t != INT32:
      res = rnd(res, cur_t)
  if rzp is not None:
    corr = dot(lv, bcast(rzp, rv.shape, rca + rba))
    res = generic_broadcast(np.subtract, res, corr)
    if cur_t != INT32:
      res = rnd(res, cur_t)
  acc = res
  for s in (ls, rs):
    if s is None:
      continue
    if cur_t == INT32:
      # int32 -> float convert goes through f32 (then to bf16 if needed).
      res = rnd(res.astype(np.float32), s.dtype)
      cur_t = s.dtype
    else:
      nt = promote(cur_t, s.dtype)
      res = rnd(res, nt)
      cur_t = nt
    res = rnd(generic_broadcast(np.multiply, res, s.v), cur_t)
  if sum_axes:
    if cur_t == INT32:
      res = res.sum(axis=sum_axes)
    else:
      # jnp.sum upcasts bf16 to f32, reduces, casts back.  Sequential order
      # over the tile axis (XLA's order is unpinned).
      out = None
      moved = np.moveaxis(res, sum_axes, tuple(range(len(sum_axes))))
      flat = moved.reshape(-1, *moved.shape[len(sum_axes) :]).astype(np.float32)
      out = np.zeros(flat.shape[1:], np.float32)
      for g in range(flat.shape[0]):
        out = out + flat[g]
      res = rnd(out, cur_t)
  if res_t == INT32:
    out = res.astype(np.int32)
  else:
    out = FArr(rnd(np.asarray(res, np.float32), res_t), res_t)
  if return_acc:
    return out, acc
  return out


def slow_dot_general(lhs, rhs, dimension_numbers, preferred_element_type=None):
  """dot_general.py:264-275: dequantize, then a float dot (f64 accumulate here)."""
  if isinstance(lhs, QArray):
    lhs = dequantize(lhs)
  if isinstance(rhs, QArray):
    rhs = dequantize(rhs)
  res_t = preferred_element_type or promote(lhs.dtype, rhs.dtype)
  d = _dot_general_f64(lhs.v, rhs.v, dimension_numbers)
  return FArr(rnd(d.astype(np.float32), res_t), res_t)


MIN_TILE_SIZE_TO_DEQUANT_ON_OUTPUT = 128  # dot_general.py:404


def use_fast_path(lhs, rhs, dimension_numbers) -> bool:
  """dot_general.py:439-472."""
  for operand, ca in zip((lhs, rhs), dimension_numbers[0]):
    if not isinstance(operand, QArray):
      if isinstance(operand, FArr):
        return False
      continue
    for axis in ca:
      if operand.scale.shape[axis] > 1:
        t = operand.qvalue.shape[axis] // operand.scale.shape[axis]
        if t < MIN_TILE_SIZE_TO_DEQUANT_ON_OUTPUT:
          return False
  return True


def dot_general(lhs, rhs, dimension_numbers, preferred_element_type=None):
  """dot_general.py:407-491."""
  if use_fast_path(lhs, rhs, dimension_numbers):
    return fast_dot_general(lhs, rhs, dimension_numbers, preferred_element_type)
  return slow_dot_general(lhs, rhs, dimension_numbers, preferred_element_type)


# ----------------------------------------------------------------------------
# ragged_dot.py (the dimension numbers of qwix.ragged_dot: lhs (M,K), rhs (G,K,N))
# ----------------------------------------------------------------------------


def _ragged_dot_f64(lhs: np.ndarray, rhs: np.ndarray, group_sizes) -> np.ndarray:
  """lax.ragged_dot as a masked sum: out = sum_g mask_g(lhs) @ rhs[g], mask_g = rows
  [start_g, start_g + size_g).  Rows covered by no group come out as zeros; groups
  reaching past the last row are cut off by the mask."""
  m = lhs.shape[0]
  out = np.zeros((m, rhs.shape[2]), np.float64)
  rows = np.arange(m)
  start = 0
  for g, size in enumerate(group_sizes):
    mask = (rows >= start) & (rows < start + int(size))
    out += np.where(mask[:, None], lhs.astype(np.float64), 0.0) @ rhs[g].astype(np.float64)
    start += int(size)
  return out


def fast_ragged_dot(lhs, rhs, group_sizes, preferred_element_type=None):
  """ragged_dot.py:123-226 for _BASIC_RAGGED_DOT_DIMENSION_NUMBERS (:24-29).

  Tiled contracting axes become a leading batch axis t of the ragged dot (:169-180); the
  lhs scale is applied first, then the rhs scale -- expanded over the rows by a ragged dot
  of ones with the scale when it has a group axis (:32-57,205-217; 1 * s is exact, rows of
  no group get 0) -- and the tile axis is summed last (:222-224)."""
  lv, ls, lzp, lt = _operand_fields(lhs)
  rv, rs, rzp, rt = _operand_fields(rhs)
  assert lzp is None and rzp is None, 'zero points take the slow path (ragged_dot.py:278-283)'
  a, b = lt.get(1), rt.get(1)
  if a and b and a != b:
    raise ValueError('Contracting axes must be tiled with the same tile size.')
  tile = a or b or lv.shape[1]
  m, k = lv.shape
  g, _, n = rv.shape
  nt = k // tile
  acc_t, res_t = get_accumulator_and_result_type(
      lhs, rhs, preferred_element_type=preferred_element_type
  )
  parts = []
  for t in range(nt):
    d = _ragged_dot_f64(
        lv[:, t * tile : (t + 1) * tile], rv[:, t * tile : (t + 1) * tile, :], group_sizes
    )
    if acc_t == INT32:
      assert np.all(np.abs(d) < 2**31)
      parts.append(d.astype(np.int64).astype(np.int32))
    else:
      parts.append(rnd(d.astype(np.float32), acc_t))
  res = np.stack(parts)  # (nt, m, n)
  cur_t = acc_t
  scales = []
  if ls is not None:
    # (M|1, nt|1) -> (nt|1, M|1, 1)
    scales.append(FArr(ls.v.T[:, :, None], ls.dtype))
  if rs is not None:
    # (G|1, nt|1, N|tiles) -> rows pick their group's vector
    sv = rs.v
    if sv.shape[2] not in (1, n):
      sv = np.repeat(sv, n // sv.shape[2], axis=2)
    if sv.shape[0] > 1:
      ones = np.ones((m, 1), np.float32)
      sv = np.stack([
          _ragged_dot_f64(ones, sv[:, t : t + 1, :], group_sizes).astype(np.float32)
          for t in range(sv.shape[1])
      ])
    else:
      sv = np.transpose(sv, (1, 0, 2))  # (nt|1, 1, N|1)
    scales.append(FArr(sv, rs.dtype))
  for s in scales:
    if cur_t == INT32:
      res = rnd(res.astype(np.float32), s.dtype)
      cur_t = s.dtype
    else:
      cur_t = promote(cur_t, s.dtype)
      res = rnd(res, cur_t)
    res = rnd(res * s.v, cur_t)
  if a or b:
    if cur_t == INT32:
      res = res.sum(axis=0)
    else:
      out = np.zeros(res.shape[1:], np.float32)
      for t in range(nt):
        out = out + res[t].astype(np.float32)
      res = rnd(out, cur_t)
  else:
    res = res[0]
  if res_t == INT32:
    return res.astype(np.int32)
  return FArr(rnd(np.asarray(res, np.float32), res_t), res_t)


def slow_ragged_dot(lhs, rhs, group_sizes, preferred_element_type=None):
  """ragged_dot.py:229-241: dequantize, then a float ragged dot (f64 accumulate here)."""
  if isinstance(lhs, QArray):
    lhs = dequantize(lhs)
  if isinstance(rhs, QArray):
    rhs = dequantize(rhs)
  res_t = preferred_element_type or promote(lhs.dtype, rhs.dtype)
  d = _ragged_dot_f64(lhs.v, rhs.v, group_sizes)
  return FArr(rnd(d.astype(np.float32), res_t), res_t)


def ragged_dot(lhs, rhs, group_sizes, preferred_element_type=None):
  """ragged_dot.py:244-353: the quantized path unless an operand has a zero point or is a
  raw float array (:278-292)."""
  fast = True
  for operand in (lhs, rhs):
    if isinstance(operand, QArray):
      if operand.zero_point is not None:
        fast = False
    elif isinstance(operand, FArr):
      fast = False
  fn = fast_ragged_dot if fast else slow_ragged_dot
  return fn(lhs, rhs, group_sizes, preferred_element_type)


def _take(x, axis: int, index):
  """x[..., index, ...] along `axis` for an array, FArr or QArray (index: a slice keeps the axis, an int
  drops it); scales and zero points with one entry along the axis are kept whole."""
  def cut(a, n):
    if a is None:
      return None
    if a.shape[axis] == 1:
      idx = slice(None) if isinstance(index, slice) else 0
    else:
      assert a.shape[axis] == n, 'scales tiled along a ragged / group axis are not restated'
      idx = index
    return a[(slice(None),) * axis + (idx,)]

  n = x.shape[axis]
  if isinstance(x, QArray):
    zp = cut(x.zero_point, n)
    return QArray(cut(x.qvalue, n), FArr(cut(x.scale.v, n), x.scale.dtype), zp, x.qtype)
  if isinstance(x, FArr):
    return FArr(cut(x.v, n), x.dtype)
  return cut(x, n)


def ragged_dot_general(lhs, rhs, group_sizes, dot_dimension_numbers, lhs_ragged_dimension: int,
                       rhs_group_dimension: int, preferred_element_type=None):
  """ragged_dot.py:123-313 for dimension numbers whose ragged axis is the only free axis of the lhs (batch
  axes, several contracting axes, any axis order; the reference's own non-basic case is
  tests/_src/core/ragged_dot_test.py:255-275).

  The reference scales the group-wise accumulator of lax.ragged_dot_general by the lhs scale and then by the
  rhs scale that a ragged dot of ones has expanded over the rows (:32-57, 196-220), and sums the tile axes
  last (:222-224).  Row by row that is the arithmetic of dot_general on the row's group: restated here as one
  dot_general per group on slices (rows of the group along the ragged axis, the group's slice of the rhs with
  the group axis dropped), written to those rows of a zero result of shape (batch, ragged, rhs free).  For the
  dimension numbers of ragged_dot it equals fast_ragged_dot / slow_ragged_dot bit for bit (tests)."""
  (lca, rca), (lba, rba) = dot_dimension_numbers
  r, g_ax = lhs_ragged_dimension, rhs_group_dimension
  lfree = [a for a in range(len(lhs.shape)) if a not in lca and a not in lba]
  assert lfree == [r], 'the ragged axis has to be the only free axis of the lhs'
  drop = lambda a: a - (a > g_ax)
  dn = ((tuple(lca), tuple(drop(a) for a in rca)), (tuple(lba), tuple(drop(a) for a in rba)))
  fast = True
  for operand in (lhs, rhs):
    if isinstance(operand, QArray):
      if operand.zero_point is not None:
        fast = False
    elif isinstance(operand, FArr):
      fast = False
  fn = fast_dot_general if fast else slow_dot_general
  m = lhs.shape[r]
  out, out_t = None, None
  start = 0
  parts = []
  for g, size in enumerate(group_sizes):
    stop = min(start + max(int(size), 0), m)
    if stop > start:
      part = fn(_take(lhs, r, slice(start, stop)), _take(rhs, g_ax, g), dn, preferred_element_type)
      parts.append((start, stop, part))
    start = stop
  _, res_t = get_accumulator_and_result_type(lhs, rhs, preferred_element_type=preferred_element_type)
  if not fast:
    lt = lhs.scale.dtype if isinstance(lhs, QArray) else lhs.dtype
    rt = rhs.scale.dtype if isinstance(rhs, QArray) else rhs.dtype
    res_t = preferred_element_type or promote(lt, rt)
  rfree = [d for a, d in enumerate(rhs.shape) if a != g_ax and a not in rca and a not in rba]
  shape = tuple(lhs.shape[a] for a in lba) + (m,) + tuple(rfree)
  out = np.zeros(shape, np.int32 if res_t == INT32 else np.float32)
  for start, stop, part in parts:
    v = part if isinstance(part, np.ndarray) else part.v
    out[(slice(None),) * len(lba) + (slice(start, stop),)] = v
  return out if res_t == INT32 else FArr(out, res_t)


# ----------------------------------------------------------------------------
# einsum_info.py / einsum.py (binary einsum)
# ----------------------------------------------------------------------------


@dataclasses.dataclass
class EinsumInfo:
  """einsum_info.py:26-174."""

  lhs: str
  rhs: str
  out: str

  @classmethod
  def parse(cls, einsum_str: str) -> 'EinsumInfo':
    s = einsum_str.replace(' ', '')
    if not re.match(r'^[a-zA-Z]*,[a-zA-Z]*->[a-zA-Z]*$', s):
      raise NotImplementedError(f'Unsupported einsum string: "{einsum_str}".')
    ins, out = s.split('->')
    lhs, rhs = ins.split(',')
    for name, subs in zip(['lhs', 'rhs', 'out'], [lhs, rhs, out]):
      if len(set(subs)) != len(subs):
        raise NotImplementedError(f'Repeated indices in {name} ("{subs}")')
    return cls(lhs, rhs, out)

  @property
  def batch_chars(self):
    return sorted(set(self.lhs) & set(self.rhs) & set(self.out))

  @property
  def contract_chars(self):
    return sorted(set(self.lhs) & set(self.rhs) - set(self.out))

  @property
  def dimension_numbers(self):
    lm = {c: i for i, c in enumerate(self.lhs)}
    rm = {c: i for i, c in enumerate(self.rhs)}
    return (
        (
            tuple(lm[c] for c in self.contract_chars),
            tuple(rm[c] for c in self.contract_chars),
        ),
        (
            tuple(lm[c] for c in self.batch_chars),
            tuple(rm[c] for c in self.batch_chars),
        ),
    )

  @property
  def output_perm(self):
    lrem = [c for c in self.lhs if c in self.out and c not in self.batch_chars]
    rrem = [c for c in self.rhs if c in self.out and c not in self.batch_chars]
    cur = self.batch_chars + lrem + rrem
    pos = {c: i for i, c in enumerate(cur)}
    perm = tuple(pos[c] for c in self.out)
    return None if perm == tuple(range(len(perm))) else perm


def einsum_get_how_to_quantize(
    *, einsum_str, ndims, for_lhs, tile_size, **kwargs
) -> HowToQuantize:
  """einsum.py:27-81 (explicit subscripts only; `ndims` unused without ellipsis)."""
  del ndims
  info = EinsumInfo.parse(einsum_str)
  subs = info.lhs if for_lhs else info.rhs
  cw, tiled, last = [], {}, None
  for axis, ch in enumerate(subs):
    if ch not in info.contract_chars:
      cw.append(axis)
    else:
      last = axis
  if isinstance(tile_size, Mapping):
    tiled = dict(tile_size)
    cw = [a for a in cw if a not in tiled]
  elif tile_size and last is not None:
    tiled[last] = tile_size
  return HowToQuantize(channelwise_axes=cw, tiled_axes=tiled, **kwargs)


def einsum(einsum_str, lhs, rhs, preferred_element_type=None):
  """einsum.py:84-103 for a binary einsum."""
  _, res_t = get_accumulator_and_result_type(
      lhs, rhs, preferred_element_type=preferred_element_type
  )
  info = EinsumInfo.parse(einsum_str)
  out = dot_general(lhs, rhs, info.dimension_numbers, res_t)
  if info.output_perm is not None:
    if isinstance(out, FArr):
      out = FArr(np.transpose(out.v, info.output_perm), out.dtype)
    else:
      out = np.transpose(out, info.output_perm)
  return out


# ----------------------------------------------------------------------------
# contrib/hadamard_rot.py
# ----------------------------------------------------------------------------


def hadamard_matrix(power: int) -> np.ndarray:
  """hadamard_rot.py:35-42: Sylvester construction, natural order (+-1, f32)."""
  if power < 0:
    raise ValueError('Power must be non-negative.')
  h = np.ones((1, 1), np.float32)
  for _ in range(power):
    h = np.block([[h, h], [h, -h]])
  return h


def hadamard_rotate_inputs(
    act: FArr,
    weight: FArr,
    row_signs: np.ndarray | None,
    col_signs: np.ndarray | None,
    *,
    lhs_reduction_dim: int,
    rhs_reduction_dim: int,
) -> tuple[FArr, FArr]:
  """hadamard_rot.py:99-190 with the sign vectors given as inputs.

  had = H * row_signs[:, None] * col_signs[None, :]   (bf16, entries +-1)
  act'    = einsum(act, had) over lhs_reduction_dim     (unnormalised)
  weight' = einsum(had, weight) over rhs_reduction_dim, then / n
  Products with +-1 are exact; the sum is taken exactly (f64), rounded to f32 and
  then to the einsum's result dtype.  The einsum result dtype is the promotion
  of the operand dtype with bf16 (= the operand dtype for bf16/f32 operands).
  """
  n = act.shape[lhs_reduction_dim]
  if n != weight.shape[rhs_reduction_dim]:
    raise ValueError('Expected reduction dimension sizes to be the same')
  power = int(math.log2(n))
  if 2**power != n:
    raise ValueError('Expected reduction dimension size to be a power of 2')
  had = hadamard_matrix(power).astype(np.float64)
  if row_signs is not None:
    had = had * np.asarray(row_signs, np.float64)[:, None]
  if col_signs is not None:
    had = had * np.asarray(col_signs, np.float64)[None, :]
  a = np.moveaxis(act.v.astype(np.float64), lhs_reduction_dim, -1) @ had
  a = np.moveaxis(a, -1, lhs_reduction_dim)
  at = promote(act.dtype, BF16)
  act_r = FArr(rnd(a.astype(np.float32), at), at)
  w = np.moveaxis(weight.v.astype(np.float64), rhs_reduction_dim, 0)
  w = np.tensordot(had.T, w, axes=([1], [0]))
  w = np.moveaxis(w, 0, rhs_reduction_dim)
  wt = promote(weight.dtype, BF16)
  w = rnd(w.astype(np.float32), wt)
  w = rnd(w / np.float32(n), wt)
  return act_r, FArr(w, wt)
