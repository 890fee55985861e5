"""QArray and the quantize / dequantize operators, backed by the HIP kernels.

Host-side mirror of qwix/_src/core/qarray.py: same names, argument meaning and errors
(`QArray` :31-99, `HowToQuantize` :280-325, `get_scale_shape` :332-349, `calibrate` :470-534,
`compute_scale_zero_point` :537-584, `quantize_with_scale_zero_point` :594-635, `quantize`
:638-644, `quantize_api` :647-689, `dequantize` :692-708, `get_accumulator_and_result_type`
:781-821).  Arrays are torch tensors living in HBM; torch only provides memory and streams,
all arithmetic is done by libqwix_hip.so.

Differences that come from the device layout, not from the numerics:
  * int4 values are stored packed, two per byte, in an `Int4Tensor` (logical shape preserved);
  * when the reduced axis of a weight is strided (per-channel / sub-channel (K, N) kernels) the
    quantized values are written K-contiguous ("reduce-minor") and handed back as a strided view
    with the logical shape, because that is the operand layout the MFMA GEMM kernels read.
    `quantize(..., layout='natural')` keeps the input's own layout.
"""
from __future__ import annotations

import dataclasses
import functools
import math
from typing import Any, Callable, Collection, Mapping, Sequence

import torch

from qwix_amd import _lib
from qwix_amd.core import numerics

# ------------------------------------------------------------------------------------------
# Int4 storage
# ------------------------------------------------------------------------------------------


class Int4LayoutError(NotImplementedError):
  """Packed int4 values in a layout that a kernel cannot read in place; callers may widen them to int8 and go on."""


class Int4Tensor:
  """Packed int4 values: `data` (uint8) has the logical shape with `packed_axis` halved.

  Element 2i of the packed axis sits in the low nibble of byte i, element 2i+1 in the high nibble
  (two's complement).  `data` may be a strided view; the packed axis is the physically contiguous
  one for tensors produced by `quantize`.
  """

  dtype = 'int4'

  def __init__(self, data: torch.Tensor, shape: Sequence[int], packed_axis: int):
    shape = tuple(int(s) for s in shape)
    packed_axis = packed_axis % len(shape)
    want = tuple(s // 2 if a == packed_axis else s for a, s in enumerate(shape))
    if data.dtype != torch.uint8 or tuple(data.shape) != want or shape[packed_axis] % 2:
      raise ValueError(f'packed data {tuple(data.shape)} {data.dtype} does not match int4 shape {shape}')
    self.data, self.shape, self.packed_axis = data, shape, packed_axis

  ndim = property(lambda self: len(self.shape))
  device = property(lambda self: self.data.device)

  def unpack(self) -> torch.Tensor:
    """int8 tensor of the logical shape (host-side convenience for inspection and tests)."""
    d = self.data.movedim(self.packed_axis, -1)
    lo = ((d & 0xF).to(torch.int8) ^ 8) - 8
    hi = ((d >> 4).to(torch.int8) ^ 8) - 8
    out = torch.stack([lo, hi], dim=-1).reshape(*d.shape[:-1], d.shape[-1] * 2)
    return out.movedim(-1, self.packed_axis)

  @staticmethod
  def pack(values: torch.Tensor, packed_axis: int = -1) -> 'Int4Tensor':
    """The reverse of unpack(): int8 values in [-8, 7] to nibble pairs along `packed_axis` (a host-side convenience
    for re-laying out values that exist already; quantization itself writes packed nibbles)."""
    packed_axis = packed_axis % values.ndim
    v = values.movedim(packed_axis, -1).to(torch.uint8) & 0xF
    data = (v[..., 0::2] | (v[..., 1::2] << 4)).contiguous()
    return Int4Tensor(data.movedim(-1, packed_axis), tuple(values.shape), packed_axis)

  def permute(self, *axes) -> 'Int4Tensor':
    axes = tuple(axes[0]) if len(axes) == 1 and not isinstance(axes[0], int) else tuple(axes)
    return Int4Tensor(self.data.permute(*axes), tuple(self.shape[a] for a in axes), axes.index(self.packed_axis))

  def __repr__(self):
    return f'Int4Tensor(shape={self.shape}, packed_axis={self.packed_axis}, device={self.device})'


def _qshape(q) -> tuple[int, ...]:
  return tuple(q.shape)


# ------------------------------------------------------------------------------------------
# QArray / HowToQuantize
# ------------------------------------------------------------------------------------------


@dataclasses.dataclass
class QArray:
  """A quantized array: original ~= (qvalue - zero_point) * generic_broadcast(scale).

  qvalue.shape == original.shape; scale.ndim == original.ndim and every scale dim divides the
  array dim (sub-channel scales); zero_point is None for symmetric quantization; qtype is the
  logical type ('int8', 'int4', 'float8_e4m3fn').
  """

  qvalue: Any  # torch.Tensor (int8 / float8_e4m3fn) or Int4Tensor
  scale: torch.Tensor
  zero_point: torch.Tensor | None = None
  qtype: Any = None

  def __post_init__(self):
    if self.qtype is None:
      self.qtype = 'int4' if isinstance(self.qvalue, Int4Tensor) else str(self.qvalue.dtype).replace('torch.', '')
    self.qtype = numerics.canonical_qtype(self.qtype) if numerics.can_dequant_on_output(self.qtype) else self.qtype

  shape = property(lambda self: _qshape(self.qvalue))
  ndim = property(lambda self: len(self.shape))
  dtype = property(lambda self: self.scale.dtype)
  device = property(lambda self: self.scale.device)

  @property
  def scale_tile_shape(self) -> tuple[int, ...]:
    return tuple(o // s for o, s in zip(self.shape, self.scale.shape))

  @property
  def zero_point_tile_shape(self) -> tuple[int, ...] | None:
    if self.zero_point is None:
      return None
    return tuple(o // s for o, s in zip(self.shape, self.zero_point.shape))

  def astype(self, dtype: torch.dtype) -> 'QArray':
    """Casts the dequantized type, i.e. the scale dtype."""
    return dataclasses.replace(self, scale=self.scale.to(dtype))

  def transpose(self, *axes) -> 'QArray':
    if not axes:
      axes = tuple(reversed(range(self.ndim)))
    elif len(axes) == 1 and not isinstance(axes[0], int):
      axes = tuple(axes[0])
    zp = None if self.zero_point is None else self.zero_point.permute(*axes)
    return QArray(self.qvalue.permute(*axes), self.scale.permute(*axes), zp, self.qtype)

  def swapaxes(self, a: int, b: int) -> 'QArray':
    axes = list(range(self.ndim))
    axes[a], axes[b] = axes[b], axes[a]
    return self.transpose(*axes)

  T = property(lambda self: self.transpose())
  mT = property(lambda self: self.swapaxes(-1, -2))

  def reshape(self, *new_shape) -> 'QArray':
    return reshape(self, *new_shape)

  def __getitem__(self, idx) -> 'QArray':
    return rewriting_take(self, idx)


def _shape_groups(old: Sequence[int], new: Sequence[int]) -> list[tuple[tuple[int, ...], tuple[int, ...]]]:
  """Cuts both shapes into the shortest runs of equal size, e.g. (2, 2, 6) -> (4, 1, 3, 2) gives
  (2, 2)->(4,), ()->(1,), (6,)->(3, 2).  On a tie the old shape advances first unless its next entry is
  the larger one (qarray.py:117-146)."""
  groups, run_old, run_new = [], [], []
  size_old = size_new = 1
  i = j = 0
  while i < len(old) or j < len(new):
    if size_old < size_new:
      from_old = True
    elif size_old > size_new:
      from_old = False
    else:
      from_old = i < len(old) and (j >= len(new) or old[i] <= new[j])
    if from_old:
      if i >= len(old):
        break
      run_old.append(old[i])
      size_old *= old[i]
      i += 1
    else:
      if j >= len(new):
        break
      run_new.append(new[j])
      size_new *= new[j]
      j += 1
    if size_old == size_new:
      groups.append((tuple(run_old), tuple(run_new)))
      run_old, run_new, size_old, size_new = [], [], 1, 1
  if run_old or run_new or i < len(old) or j < len(new):
    raise ValueError(f'Cannot reshape {tuple(old)} into {tuple(new)}.')
  return groups


def reshape(array: QArray, *new_shape) -> QArray:
  """qarray.py:106-171: reshapes values, scale and zero point together, which is possible when every run of
  axes that is regrouped is either matched exactly by the scale, per-tensor in it, or channelwise on its
  first axis only (that axis must then divide the first new axis)."""
  if len(new_shape) == 1 and not isinstance(new_shape[0], int):
    new_shape = tuple(new_shape[0])
  new_shape = tuple(int(d) for d in new_shape)
  old_shape = tuple(array.shape)
  if math.prod(old_shape) != math.prod(new_shape):
    raise ValueError(f'Cannot reshape {old_shape} into {new_shape}.')
  groups = _shape_groups(old_shape, new_shape)

  def target(x_shape: tuple[int, ...]) -> list[int]:
    out, at = [], 0
    for old, new in groups:
      have = tuple(x_shape[at:at + len(old)])
      n = math.prod(have)
      if have == old:
        out.extend(new)
      elif n == 1:
        out.extend([1] * len(new))
      elif n == have[0] and new[0] % have[0] == 0:
        out.extend([have[0]] + [1] * (len(new) - 1))
      else:
        raise ValueError(f'Cannot reshape {old_shape} into {new_shape} for {tuple(x_shape)}.')
      at += len(old)
    return out

  q = array.qvalue
  if isinstance(q, Int4Tensor):
    if q.packed_axis != len(old_shape) - 1 or not q.data.is_contiguous() or not new_shape or new_shape[-1] % 2:
      raise NotImplementedError('int4 values reshape only in the natural layout and to an even last dimension')
    qv = Int4Tensor(q.data.reshape(*new_shape[:-1], new_shape[-1] // 2), new_shape, len(new_shape) - 1)
  else:
    qv = q.reshape(target(old_shape))
  zp = None if array.zero_point is None else array.zero_point.reshape(target(tuple(array.zero_point.shape)))
  return QArray(qv, array.scale.reshape(target(tuple(array.scale.shape))), zp, array.qtype)


def rewriting_take(array: QArray, idx) -> QArray:
  """array[idx] (qarray.py:174-209): integers, slices, None and one Ellipsis.  Scale and zero point follow:
  a per-tensor axis keeps its single entry, an integer on a tiled axis picks that element's tile; a partial
  slice of a tiled axis is refused."""
  idx = list(idx) if isinstance(idx, (tuple, list)) else [idx]
  named = sum(1 for it in idx if it is not None and it is not Ellipsis)
  fill = [slice(None)] * (array.ndim - named)
  if any(it is Ellipsis for it in idx):
    at = [k for k, it in enumerate(idx) if it is Ellipsis]
    if len(at) != 1:
      raise ValueError('an index can hold a single Ellipsis')
    idx[at[0]:at[0] + 1] = fill
  else:
    idx += fill
  shape = tuple(array.shape)

  def component_index(x_shape) -> tuple:
    out, k = [], 0
    for full, have in zip(shape, x_shape):
      while idx[k] is None:
        out.append(None)
        k += 1
      it = idx[k]
      whole = isinstance(it, slice) and it == slice(None)
      if full == have or whole:
        out.append(it)
      elif have == 1:
        out.append(0 if isinstance(it, int) else slice(None))
      elif isinstance(it, int):
        out.append((it % full) // (full // have))
      else:
        raise ValueError(f'Unsupported indexing {idx} for {shape}.')
      k += 1
    out.extend(idx[k:])
    return tuple(out)

  q = array.qvalue
  if isinstance(q, Int4Tensor):
    ci = component_index(shape)
    ax_items = [it for it in ci if it is not None]
    if not (isinstance(ax_items[q.packed_axis], slice) and ax_items[q.packed_axis] == slice(None)):
      raise NotImplementedError('the packed axis of int4 values can only be taken whole')
    data = q.data[ci]
    new_shape, packed, pos, src = [], None, 0, 0
    for it in ci:
      if it is None:
        new_shape.append(1)
        pos += 1
        continue
      if not isinstance(it, int):
        if src == q.packed_axis:
          packed = pos
        new_shape.append(data.shape[pos] * (2 if src == q.packed_axis else 1))
        pos += 1
      src += 1
    qv = Int4Tensor(data, new_shape, packed)
  else:
    qv = q[component_index(shape)]
  zp = None if array.zero_point is None else array.zero_point[component_index(tuple(array.zero_point.shape))]
  return QArray(qv, array.scale[component_index(tuple(array.scale.shape))], zp, array.qtype)



@dataclasses.dataclass(frozen=True, kw_only=True)
class HowToQuantize:
  """How to quantize an array (qarray.py:280-325).

  channelwise_axes get one scale per index; tiled_axes map an axis to a tile size (int) or to
  1/tile_count (float); every other axis shares one scale.  calibration_method is
  'absmax[,factor]' or 'minmax[,factor]'.
  """

  qtype: Any
  channelwise_axes: Collection[int] = ()
  tiled_axes: Mapping[int, int | float] = dataclasses.field(default_factory=dict)
  calibration_method: str = 'absmax'
  noise_fn: Callable | None = None


MaybeQArray = Any


def _resolve_tile(dim: int, tile) -> int:
  return round(dim * tile) if isinstance(tile, float) else int(tile)


def get_scale_shape(array_shape: Sequence[int], how: HowToQuantize) -> tuple[int, ...]:
  if set(how.channelwise_axes) & set(how.tiled_axes.keys()):
    raise ValueError('The same axis cannot be both channelwise and tiled.')
  out = []
  for axis, dim in enumerate(array_shape):
    if axis in how.channelwise_axes:
      out.append(dim)
    elif axis in how.tiled_axes:
      t = _resolve_tile(dim, how.tiled_axes[axis])
      if t <= 0 or dim % t != 0:
        raise ValueError(f'{tuple(array_shape)} cannot be tiled as {dict(how.tiled_axes)}.')
      out.append(dim // t)
    else:
      out.append(1)
  return tuple(out)


def get_tiled_axes(array: QArray) -> dict[int, int]:
  """Infers {axis: tile size} of the sub-channel axes from the shapes (qarray.py:409-422)."""
  return {i: j // k for i, (j, k) in enumerate(zip(array.shape, array.scale.shape)) if j != k and k != 1}


def validate_qarray(array: QArray) -> None:
  """Internal-consistency checks of qarray.py:212-247."""
  qs, ss = array.shape, tuple(array.scale.shape)
  if len(qs) != len(ss):
    raise ValueError(f'Scale {ss} should have the same rank as qvalue {qs}.')
  if not all((a % b == 0) if b else a == 0 for a, b in zip(qs, ss)):
    raise ValueError(f'Scale {ss} should be broadcastable to qvalue {qs}.')
  if not numerics.should_quantize(array.scale.dtype):
    raise ValueError(f'{array.scale.dtype} is not a valid type for scale.')
  if array.zero_point is not None:
    zs = tuple(array.zero_point.shape)
    if len(zs) != len(qs):
      raise ValueError(f'Zero point {zs} should have the same rank as qvalue {qs}.')
    if not all((a % b == 0) if b else a == 0 for a, b in zip(qs, zs)):
      raise ValueError(f'Zero point {zs} should be broadcastable to qvalue {qs}.')
    if array.zero_point.dtype != torch.int8:
      raise ValueError(f'Zero point {array.zero_point.dtype} should be int8 (the storage dtype of int8/int4).')


# ------------------------------------------------------------------------------------------
# Mapping an n-D quantization pattern to the kernels' (outer, reduce, inner, tile) view
# ------------------------------------------------------------------------------------------


@dataclasses.dataclass(frozen=True)
class _Plan:
  kind: str                      # '3d' or '5d'
  dims: tuple[int, ...]          # (outer, reduce, inner) or (d0, r1, d2, r3, d4)
  tiles: tuple[int, ...]         # (tile,) or (t1, t3)
  outer_axes: tuple[int, ...] = ()
  reduce_axes: tuple[int, ...] = ()
  inner_axes: tuple[int, ...] = ()


def _plan(shape: Sequence[int], tiles: Sequence[int]) -> _Plan:
  """tiles[a] = elements of axis a that share one scale (1 = channelwise, dim = fully reduced)."""
  return _plan_cached(tuple(int(d) for d in shape), tuple(int(t) for t in tiles))


@functools.lru_cache(maxsize=4096)
def _plan_cached(shape: tuple[int, ...], tiles: tuple[int, ...]) -> _Plan:
  blocks: list[list] = []  # ['c', size, axes] or ['r', reduce, tile, axes]
  for a, (d, t) in enumerate(zip(shape, tiles)):
    if d == 1:
      if blocks:
        blocks[-1][-1].append(a)
      else:
        blocks.append(['c', 1, [a]])
      continue
    if t == 1:
      if blocks and blocks[-1][0] == 'c':
        blocks[-1][1] *= d
        blocks[-1][-1].append(a)
      else:
        blocks.append(['c', d, [a]])
    elif t == d and blocks and blocks[-1][0] == 'r':
      blocks[-1][1] *= d
      blocks[-1][2] *= d
      blocks[-1][-1].append(a)
    else:
      blocks.append(['r', d, t, [a]])
  kinds = ''.join(b[0] for b in blocks)
  nr = kinds.count('r')
  if nr == 0:
    n = math.prod(shape)
    return _Plan('3d', (n, 1, 1), (1,), tuple(range(len(shape))), (), ())
  if nr == 1:
    i = kinds.index('r')
    if kinds[:i].count('c') > 1 or kinds[i + 1:].count('c') > 1:
      raise AssertionError(kinds)
    outer = math.prod(b[1] for b in blocks[:i])
    inner = math.prod(b[1] for b in blocks[i + 1:])
    flat = lambda bs: tuple(a for b in bs for a in b[-1])
    return _Plan('3d', (outer, blocks[i][1], inner), (blocks[i][2],), flat(blocks[:i]), tuple(blocks[i][-1]), flat(blocks[i + 1:]))
  if nr == 2 and kinds in ('rr', 'crr', 'rcr', 'rrc', 'crcr', 'crrc', 'rcrc', 'crcrc'):
    it = iter(blocks)
    dims, ts = [], []
    b = next(it, None)
    for slot in 'crcrc':
      if b is not None and b[0] == slot:
        dims.append(b[1])
        if slot == 'r':
          ts.append(b[2])
        b = next(it, None)
      else:
        dims.append(1)
        if slot == 'r':
          ts.append(1)
    return _Plan('5d', tuple(dims), tuple(ts))
  raise NotImplementedError(
      f'quantization pattern of shape {tuple(shape)} with per-axis tiles {tuple(tiles)} needs more than two '
      'separate reduced axis groups; not supported by the HIP kernels.'
  )


def _regrouped(shape, sshape):
  """Any tiling as a 2-D problem: every axis split into (tile count, tile), the counts in front.  Returns the split
  shape, the permutation that brings the counts to the front, and (rows, cols) = (scales, elements per scale)."""
  tiles = [d // s for d, s in zip(shape, sshape)]
  split = [v for st in zip(sshape, tiles) for v in st]
  n = len(shape)
  perm = [2 * a for a in range(n)] + [2 * a + 1 for a in range(n)]
  return tiles, split, perm, math.prod(sshape), math.prod(tiles)


def _ungroup(values2d: torch.Tensor, shape, sshape) -> torch.Tensor:
  tiles, _, perm, _, _ = _regrouped(shape, sshape)
  inv = [perm.index(a) for a in range(len(perm))]
  return values2d.reshape(*sshape, *tiles).permute(*inv).reshape(shape)


def _quantize_regrouped(array: torch.Tensor, how: HowToQuantize, q: str, sshape) -> 'QArray':
  """Patterns with more than two separate groups of reduced axes (say 2-D blocks and a whole axis besides): the
  elements of a scale are gathered into a row (one copy), the rows are quantized with one scale each, and the values
  return to their places (one copy).  The same maxima over the same elements: identical results."""
  shape = tuple(array.shape)
  _, split, perm, rows, cols = _regrouped(shape, sshape)
  x2 = array.reshape(split).permute(*perm).reshape(rows, cols).contiguous()
  q2 = quantize(x2, HowToQuantize(qtype=q, channelwise_axes=(0,), calibration_method=how.calibration_method),
                layout='natural')
  vals = q2.qvalue.unpack() if isinstance(q2.qvalue, Int4Tensor) else q2.qvalue
  vals = _ungroup(vals, shape, sshape).contiguous()
  if q == numerics.INT4:
    vals = Int4Tensor.pack(vals)
  zp = None if q2.zero_point is None else q2.zero_point.reshape(sshape)
  return QArray(vals, q2.scale.reshape(sshape), zp, q)


def _tiles_from_how(shape, how: HowToQuantize) -> tuple[int, ...]:
  ss = get_scale_shape(shape, how)
  return tuple(d // s for d, s in zip(shape, ss))


def _fixed_calibration(method: str, array: torch.Tensor) -> dict[str, torch.Tensor] | None:
  """'fixed,a[,b]' (qarray.py:518-532): a constant per-tensor range, nothing is read from the array.
  None for the other methods."""
  name, *args = method.lower().split(',')
  if name != 'fixed':
    return None
  args = [float(a) for a in args]
  if len(args) not in (1, 2):
    raise ValueError('A fixed range is required for fixed calibration.')
  if len(args) == 1:
    args = [-args[0], args[0]]
  if args[0] > 0 or args[1] < 0 or args[0] >= args[1]:
    raise ValueError('The range must contain 0 and be non-empty.')
  ones = (1,) * array.ndim
  full = lambda v: torch.full(ones, v, dtype=array.dtype, device=array.device)
  if args[0] + args[1] == 0:
    return {'absmax': full(args[1])}
  return {'min': full(args[0]), 'max': full(args[1])}


def _rms_calibration(method: str, array: torch.Tensor, sshape, tiles) -> dict[str, torch.Tensor] | None:
  """'rms,s' (qarray.py:511-515): an 'absmax' calibration of sqrt(mean(x^2)) * s per scale group.  None for
  the other methods."""
  name, *args = method.lower().split(',')
  if name != 'rms':
    return None
  if not args:
    raise ValueError('A scale factor is required for RMS calibration.')
  array = _check_float_input(array)
  if array.numel() == 0:
    _check_empty_reduction(sshape)
    return {'absmax': torch.empty(sshape, dtype=array.dtype, device=array.device)}
  plan = _plan(tuple(array.shape), tuple(tiles))
  dims5 = tuple(plan.dims) + (1, 1) if plan.kind == '3d' else tuple(plan.dims)
  t1, t3 = (plan.tiles[0], 1) if plan.kind == '3d' else plan.tiles
  import ctypes
  out = torch.empty(sshape, dtype=array.dtype, device=array.device)
  _lib.call('qwix_hip_calibrate_rms', array.data_ptr(), _lib.float_tag(array.dtype), (ctypes.c_int64 * 5)(*dims5), t1, t3,
            float(args[0]), out.data_ptr(), _lib.stream_of(array))
  return {'absmax': out}


def _parse_calibration(method: str) -> tuple[int, float]:
  name, *args = method.lower().split(',')
  args = [float(a) for a in args]
  if name not in ('absmax', 'minmax'):
    raise ValueError(f'Unsupported calibration: {method}')
  return (_lib.ABSMAX if name == 'absmax' else _lib.MINMAX), (args[0] if args else 0.0)


def _check_float_input(array: torch.Tensor) -> torch.Tensor:
  if not isinstance(array, torch.Tensor) or not numerics.should_quantize(array.dtype):
    raise ValueError(f'Refuse to quantize: {getattr(array, "dtype", type(array))}')
  return array if array.is_contiguous() else array.contiguous()


def _workspace(plan: _Plan, cal: int, device) -> tuple[torch.Tensor | None, int]:
  outer, reduce, inner = plan.dims
  n = _lib.load().qwix_hip_quantize_workspace_bytes(outer, reduce, inner, plan.tiles[0], cal)
  if n == 0:
    return None, 0
  return torch.empty(n, dtype=torch.uint8, device=device), n


def _reduce_minor_order(shape, plan: _Plan) -> tuple[int, ...]:
  red = tuple(plan.reduce_axes)
  return (tuple(plan.outer_axes) + tuple(plan.inner_axes) + tuple(a for a in red if shape[a] == 1) +
          tuple(a for a in red if shape[a] != 1))


def _alloc_q(shape, qtype: str, plan: _Plan, layout: int, device):
  """Allocates the qvalue buffer; returns (flat storage tensor, logical view)."""
  is4 = qtype == numerics.INT4
  if layout == _lib.LAYOUT_NATURAL or plan.kind != '3d' or plan.dims[2] == 1:
    if is4:
      if shape[-1] % 2:
        raise NotImplementedError(f'int4 needs an even last dimension, got {tuple(shape)}')
      data = torch.empty(*shape[:-1], shape[-1] // 2, dtype=torch.uint8, device=device)
      return data, Int4Tensor(data, shape, len(shape) - 1)
    data = torch.empty(tuple(shape), dtype=numerics.storage_dtype(qtype), device=device)
    return data, data
  # reduce-minor: physical order (outer axes, inner axes, reduce axes); reduce axes of size 1 lead the others
  # (the memory is the same) so that the last axis, which int4 pairs run along, is a real one.
  order = _reduce_minor_order(shape, plan)
  phys_shape = [shape[a] for a in order]
  inv = [order.index(a) for a in range(len(shape))]
  if is4:
    if phys_shape[-1] % 2:
      raise NotImplementedError(f'int4 in the reduce-minor layout needs an even last reduced axis, got {tuple(shape)}')
    phys_shape[-1] //= 2
    data = torch.empty(phys_shape, dtype=torch.uint8, device=device)
    return data, Int4Tensor(data.permute(*inv), shape, order[-1])
  data = torch.empty(phys_shape, dtype=numerics.storage_dtype(qtype), device=device)
  return data, data.permute(*inv)


def _empty_qvalue(shape, qtype: str, device):
  """A qvalue with no elements (nothing is launched for it)."""
  if qtype == numerics.INT4:
    if shape[-1] % 2:
      raise NotImplementedError(f'int4 needs an even last dimension, got {tuple(shape)}')
    data = torch.empty(*shape[:-1], shape[-1] // 2, dtype=torch.uint8, device=device)
    return Int4Tensor(data, shape, len(shape) - 1)
  return torch.empty(tuple(shape), dtype=numerics.storage_dtype(qtype), device=device)


def _check_empty_reduction(sshape) -> None:
  # jnp.max over an empty axis has no identity; an empty scale means there is nothing to reduce at all.
  if math.prod(sshape):
    raise ValueError('zero-size array to reduction operation max which has no identity')


def _default_layout(plan: _Plan, layout: str | None, shape=None, qtype: str | None = None) -> int:
  if layout is None:
    layout = 'reduce_minor' if (plan.kind == '3d' and plan.dims[2] > 1 and plan.dims[1] % 8 == 0 and plan.tiles[0] % 8 == 0) else 'natural'
    if layout == 'reduce_minor' and qtype == numerics.INT4:
      # int4 pairs run along the last reduce axis that is not of size 1: it has to be even
      real = [shape[a] for a in plan.reduce_axes if shape[a] != 1]
      if not real or real[-1] % 2:
        layout = 'natural'
  if layout not in ('natural', 'reduce_minor'):
    raise ValueError(f'unknown layout {layout!r}')
  return _lib.LAYOUT_NATURAL if layout == 'natural' else _lib.LAYOUT_REDUCE_MINOR


# ------------------------------------------------------------------------------------------
# calibrate / compute_scale_zero_point / quantize_with_scale_zero_point / quantize
# ------------------------------------------------------------------------------------------


def calibrate(array: torch.Tensor, how: HowToQuantize) -> dict[str, torch.Tensor]:
  """Returns {'absmax': ...} or {'min': ..., 'max': ...}, each shaped like the scale."""
  array = _check_float_input(array)
  shape = tuple(array.shape)
  sshape = get_scale_shape(shape, how)
  fixed = _fixed_calibration(how.calibration_method, array)
  if fixed is not None:
    return fixed
  rms = _rms_calibration(how.calibration_method, array, sshape, _tiles_from_how(shape, how) if array.numel() else ())
  if rms is not None:
    return rms
  cal, factor = _parse_calibration(how.calibration_method)
  if array.numel() == 0:
    _check_empty_reduction(sshape)
    outs = [torch.empty(sshape, dtype=array.dtype, device=array.device) for _ in range(2 if cal == _lib.MINMAX else 1)]
    return {'min': outs[0], 'max': outs[1]} if cal == _lib.MINMAX else {'absmax': outs[0]}
  try:
    plan = _plan(shape, _tiles_from_how(shape, how))
  except NotImplementedError:
    plan = None
  ev = 8 if array.dtype == torch.bfloat16 else 4
  if plan is None or plan.kind != '3d' or (plan.dims[2] > 1 and plan.dims[2] % ev):
    # more than one group of reduced axes: the elements of a scale gathered into a row, one statistic per row
    _, split, perm, rows, cols = _regrouped(shape, sshape)
    x2 = array.reshape(split).permute(*perm).reshape(rows, cols).contiguous()
    got = calibrate(x2, HowToQuantize(qtype=how.qtype, channelwise_axes=(0,), calibration_method=how.calibration_method))
    return {k: v.reshape(sshape) for k, v in got.items()}
  outs = [torch.empty(sshape, dtype=array.dtype, device=array.device) for _ in range(2 if cal == _lib.MINMAX else 1)]
  ws, nws = _workspace(plan, cal, array.device)
  _lib.call('qwix_hip_calibrate', array.data_ptr(), _lib.float_tag(array.dtype), *plan.dims, plan.tiles[0], cal,
            factor, outs[0].data_ptr(), _lib.ptr(outs[1] if len(outs) > 1 else None), _lib.ptr(ws), nws,
            _lib.stream_of(array))
  if cal == _lib.MINMAX:
    return {'min': outs[0], 'max': outs[1]}
  return {'absmax': outs[0]}


def compute_scale_zero_point(calibration: Mapping[str, torch.Tensor], qtype) -> tuple[torch.Tensor, torch.Tensor | None]:
  """scale (and zero_point for min/max calibrations) from calibration statistics."""
  if 'min' in calibration and 'max' in calibration:
    c0, c1, cal = calibration['min'].contiguous(), calibration['max'].contiguous(), _lib.MINMAX
    numerics.get_asymmetric_bound(qtype)  # raises for fp8
  elif 'absmax' in calibration:
    c0, c1, cal = calibration['absmax'].contiguous(), None, _lib.ABSMAX
  else:
    raise ValueError(f'Unsupported calibration: {calibration}')
  scale = torch.empty_like(c0)
  zp = torch.empty(c0.shape, dtype=torch.int8, device=c0.device) if cal == _lib.MINMAX else None
  _lib.call('qwix_hip_compute_scale_zero_point', c0.data_ptr(), _lib.ptr(c1), _lib.float_tag(c0.dtype), c0.numel(),
            numerics.qtype_tag(qtype), cal, scale.data_ptr(), _lib.ptr(zp), _lib.stream_of(c0))
  return scale, zp


def quantize_with_scale_zero_point(array: torch.Tensor, qtype, scale: torch.Tensor, zero_point: torch.Tensor | None,
                                   noise_fn=None, *, layout: str | None = None) -> QArray:
  """Quantizes with a given (static) scale; the scale is first cast to the array dtype.  `noise_fn(shape)` returns the
  noise of stochastic rounding (numerics.py:191-195): added in f32 before the rounding to an integer type; float
  qtypes ignore it, as the reference does."""
  array = _check_float_input(array)
  if zero_point is not None and tuple(zero_point.shape) != tuple(scale.shape):
    raise ValueError(f'Expect zero_point shape {tuple(scale.shape)} but got {tuple(zero_point.shape)}')
  shape = tuple(array.shape)
  if len(shape) != scale.ndim or any((d % s) if s else d for d, s in zip(shape, scale.shape)):
    raise ValueError(f'Cannot broadcast between {shape} {tuple(scale.shape)}')
  q = numerics.canonical_qtype(qtype)
  scale = scale.to(array.dtype).contiguous()
  if array.numel() == 0:
    return QArray(_empty_qvalue(shape, q, array.device), scale, zero_point, q)
  try:
    plan = _plan(shape, tuple(d // s for d, s in zip(shape, scale.shape)))
  except NotImplementedError:
    plan = None
  ev = 8 if array.dtype == torch.bfloat16 else 4
  if (plan is None or plan.kind != '3d' or (plan.dims[2] > 1 and plan.dims[2] % ev)
      or (q == numerics.INT4 and plan.dims[2] == 1 and plan.tiles[0] % 2)):
    # The static-scale kernels take one group of reduced axes (and whole 16-byte pieces of kept inner axes): any
    # other pattern gathers the elements of a scale into a row first and puts the values back afterwards.
    if layout not in (None, 'natural'):
      raise NotImplementedError(f'static-scale quantization of shape {shape} with scales {tuple(scale.shape)} is '
                                'delivered in the natural layout only')
    sshape = tuple(scale.shape)
    _, split, perm, rows, cols = _regrouped(shape, sshape)
    if q == numerics.INT4 and cols % 2:
      raise NotImplementedError(f'static-scale int4 quantization needs an even number of elements per scale, got {cols}')
    regroup = lambda t: t.reshape(split).permute(*perm).reshape(rows, cols).contiguous()
    noise2 = None
    if noise_fn is not None and q in (numerics.INT8, numerics.INT4):
      noise = noise_fn(shape)
      if not isinstance(noise, torch.Tensor) or tuple(noise.shape) != shape:
        raise ValueError(f'noise_fn must return a tensor of shape {shape}')
      noise2 = lambda _shape, n=regroup(noise.to(array.device)): n
    q2 = quantize_with_scale_zero_point(regroup(array), q, scale.reshape(rows, 1),
                                        None if zero_point is None else zero_point.reshape(rows, 1), noise2,
                                        layout='natural')
    vals = q2.qvalue.unpack() if isinstance(q2.qvalue, Int4Tensor) else q2.qvalue
    vals = _ungroup(vals, shape, sshape).contiguous()
    if q == numerics.INT4:
      vals = Int4Tensor.pack(vals)
    return QArray(vals, scale, zero_point, q)
  if noise_fn is not None and q in (numerics.INT8, numerics.INT4):
    noise = noise_fn(shape)
    if not isinstance(noise, torch.Tensor) or tuple(noise.shape) != shape:
      raise ValueError(f'noise_fn must return a tensor of shape {shape}')
    noise = noise.to(device=array.device, dtype=torch.float32).contiguous()
    data, view = _alloc_q(shape, q, plan, _lib.LAYOUT_NATURAL, array.device)
    zp = None if zero_point is None else zero_point.contiguous()
    _lib.call('qwix_hip_quantize_with_scale_noise', array.data_ptr(), _lib.float_tag(array.dtype), *plan.dims,
              plan.tiles[0], numerics.qtype_tag(q), scale.data_ptr(), _lib.ptr(zp), noise.data_ptr(), data.data_ptr(),
              _lib.stream_of(array))
    return QArray(view, scale, zero_point, q)
  lay = _default_layout(plan, layout, shape, q)
  data, view = _alloc_q(shape, q, plan, lay, array.device)
  zp = None if zero_point is None else zero_point.contiguous()
  _lib.call('qwix_hip_quantize_with_scale', array.data_ptr(), _lib.float_tag(array.dtype), *plan.dims, plan.tiles[0],
            numerics.qtype_tag(q), scale.data_ptr(), _lib.ptr(zp), lay, data.data_ptr(), _lib.stream_of(array))
  return QArray(view, scale, zero_point, q)


def quantize(array: torch.Tensor, how: HowToQuantize, *, layout: str | None = None) -> QArray:
  """Dynamic-range quantization: calibrate, derive scale (and zero point), quantize -- one fused pass.  With a
  `noise_fn` (stochastic rounding) the three steps run one after the other, as the reference's do (qarray.py:638-644)."""
  try:
    return _quantize(array, how, layout=layout)
  except NotImplementedError as e:
    # Packed int4 pairs run along one axis of even length; the natural layout takes the last one.  With an odd last
    # axis the array is quantized with an even axis moved to the end (one copy) and the packed values are handed back
    # as a view in the caller's axis order.
    if 'even last dimension' not in str(e) or layout is not None or how.noise_fn is not None:
      raise
    shape, nd = tuple(array.shape), array.ndim
    even = [a for a in range(nd - 1) if shape[a] % 2 == 0]
    if not even:
      raise
    a = even[-1]
    order = [d for d in range(nd) if d != a] + [a]        # new axis i is old axis order[i]
    new_of = {old: new for new, old in enumerate(order)}
    how2 = dataclasses.replace(how, channelwise_axes=tuple(new_of[c % nd] for c in how.channelwise_axes),
                               tiled_axes={new_of[k % nd]: v for k, v in how.tiled_axes.items()})
    q2 = _quantize(array.permute(*order).contiguous(), how2, layout='natural')
    inv = [new_of[d] for d in range(nd)]
    back = lambda t: None if t is None else t.permute(*inv).contiguous()
    return QArray(q2.qvalue.permute(*inv), back(q2.scale), back(q2.zero_point), q2.qtype)


def _quantize(array: torch.Tensor, how: HowToQuantize, *, layout: str | None = None) -> QArray:
  if how.noise_fn is not None and numerics.canonical_qtype(how.qtype) in (numerics.INT8, numerics.INT4) and array.numel():
    scale, zp = compute_scale_zero_point(calibrate(array, how), how.qtype)
    return quantize_with_scale_zero_point(array, how.qtype, scale, zp, how.noise_fn, layout='natural')
  if not isinstance(array, torch.Tensor) or not numerics.should_quantize(array.dtype):
    raise ValueError(f'Refuse to quantize: {getattr(array, "dtype", type(array))}')
  shape = tuple(array.shape)
  q = numerics.canonical_qtype(how.qtype)
  sshape = get_scale_shape(shape, how)
  fixed = _fixed_calibration(how.calibration_method, array)
  if fixed is not None:
    return fixed
  rms = _rms_calibration(how.calibration_method, array, sshape, _tiles_from_how(shape, how) if array.numel() else ())
  if rms is not None:
    return rms
  cal, factor = _parse_calibration(how.calibration_method)
  if array.numel() == 0:
    _check_empty_reduction(sshape)
    outs = [torch.empty(sshape, dtype=array.dtype, device=array.device) for _ in range(2 if cal == _lib.MINMAX else 1)]
    return {'min': outs[0], 'max': outs[1]} if cal == _lib.MINMAX else {'absmax': outs[0]}
  try:
    plan = _plan(shape, _tiles_from_how(shape, how))
  except NotImplementedError:
    plan = None
  ev = 8 if array.dtype == torch.bfloat16 else 4
  if plan is None or plan.kind != '3d' or (plan.dims[2] > 1 and plan.dims[2] % ev):
    # more than one group of reduced axes: the elements of a scale gathered into a row, one statistic per row
    _, split, perm, rows, cols = _regrouped(shape, sshape)
    x2 = array.reshape(split).permute(*perm).reshape(rows, cols).contiguous()
    got = calibrate(x2, HowToQuantize(qtype=how.qtype, channelwise_axes=(0,), calibration_method=how.calibration_method))
    return {k: v.reshape(sshape) for k, v in got.items()}
  outs = [torch.empty(sshape, dtype=array.dtype, device=array.device) for _ in range(2 if cal == _lib.MINMAX else 1)]
  ws, nws = _workspace(plan, cal, array.device)
  _lib.call('qwix_hip_calibrate', array.data_ptr(), _lib.float_tag(array.dtype), *plan.dims, plan.tiles[0], cal,
            factor, outs[0].data_ptr(), _lib.ptr(outs[1] if len(outs) > 1 else None), _lib.ptr(ws), nws,
            _lib.stream_of(array))
  if cal == _lib.MINMAX:
    return {'min': outs[0], 'max': outs[1]}
  return {'absmax': outs[0]}


def compute_scale_zero_point(calibration: Mapping[str, torch.Tensor], qtype) -> tuple[torch.Tensor, torch.Tensor | None]:
  """scale (and zero_point for min/max calibrations) from calibration statistics."""
  if 'min' in calibration and 'max' in calibration:
    c0, c1, cal = calibration['min'].contiguous(), calibration['max'].contiguous(), _lib.MINMAX
    numerics.get_asymmetric_bound(qtype)  # raises for fp8
  elif 'absmax' in calibration:
    c0, c1, cal = calibration['absmax'].contiguous(), None, _lib.ABSMAX
  else:
    raise ValueError(f'Unsupported calibration: {calibration}')
  scale = torch.empty_like(c0)
  zp = torch.empty(c0.shape, dtype=torch.int8, device=c0.device) if cal == _lib.MINMAX else None
  _lib.call('qwix_hip_compute_scale_zero_point', c0.data_ptr(), _lib.ptr(c1), _lib.float_tag(c0.dtype), c0.numel(),
            numerics.qtype_tag(qtype), cal, scale.data_ptr(), _lib.ptr(zp), _lib.stream_of(c0))
  return scale, zp


def quantize_with_scale_zero_point(array: torch.Tensor, qtype, scale: torch.Tensor, zero_point: torch.Tensor | None,
                                   noise_fn=None, *, layout: str | None = None) -> QArray:
  """Quantizes with a given (static) scale; the scale is first cast to the array dtype.  `noise_fn(shape)` returns the
  noise of stochastic rounding (numerics.py:191-195): added in f32 before the rounding to an integer type; float
  qtypes ignore it, as the reference does."""
  array = _check_float_input(array)
  if zero_point is not None and tuple(zero_point.shape) != tuple(scale.shape):
    raise ValueError(f'Expect zero_point shape {tuple(scale.shape)} but got {tuple(zero_point.shape)}')
  shape = tuple(array.shape)
  if len(shape) != scale.ndim or any((d % s) if s else d for d, s in zip(shape, scale.shape)):
    raise ValueError(f'Cannot broadcast between {shape} {tuple(scale.shape)}')
  q = numerics.canonical_qtype(qtype)
  scale = scale.to(array.dtype).contiguous()
  if array.numel() == 0:
    return QArray(_empty_qvalue(shape, q, array.device), scale, zero_point, q)
  try:
    plan = _plan(shape, tuple(d // s for d, s in zip(shape, scale.shape)))
  except NotImplementedError:
    plan = None
  ev = 8 if array.dtype == torch.bfloat16 else 4
  if (plan is None or plan.kind != '3d' or (plan.dims[2] > 1 and plan.dims[2] % ev)
      or (q == numerics.INT4 and plan.dims[2] == 1 and plan.tiles[0] % 2)):
    # The static-scale kernels take one group of reduced axes (and whole 16-byte pieces of kept inner axes): any
    # other pattern gathers the elements of a scale into a row first and puts the values back afterwards.
    if layout not in (None, 'natural'):
      raise NotImplementedError(f'static-scale quantization of shape {shape} with scales {tuple(scale.shape)} is '
                                'delivered in the natural layout only')
    sshape = tuple(scale.shape)
    _, split, perm, rows, cols = _regrouped(shape, sshape)
    if q == numerics.INT4 and cols % 2:
      raise NotImplementedError(f'static-scale int4 quantization needs an even number of elements per scale, got {cols}')
    regroup = lambda t: t.reshape(split).permute(*perm).reshape(rows, cols).contiguous()
    noise2 = None
    if noise_fn is not None and q in (numerics.INT8, numerics.INT4):
      noise = noise_fn(shape)
      if not isinstance(noise, torch.Tensor) or tuple(noise.shape) != shape:
        raise ValueError(f'noise_fn must return a tensor of shape {shape}')
      noise2 = lambda _shape, n=regroup(noise.to(array.device)): n
    q2 = quantize_with_scale_zero_point(regroup(array), q, scale.reshape(rows, 1),
                                        None if zero_point is None else zero_point.reshape(rows, 1), noise2,
                                        layout='natural')
    vals = q2.qvalue.unpack() if isinstance(q2.qvalue, Int4Tensor) else q2.qvalue
    vals = _ungroup(vals, shape, sshape).contiguous()
    if q == numerics.INT4:
      vals = Int4Tensor.pack(vals)
    return QArray(vals, scale, zero_point, q)
  if noise_fn is not None and q in (numerics.INT8, numerics.INT4):
    noise = noise_fn(shape)
    if not isinstance(noise, torch.Tensor) or tuple(noise.shape) != shape:
      raise ValueError(f'noise_fn must return a tensor of shape {shape}')
    noise = noise.to(device=array.device, dtype=torch.float32).contiguous()
    data, view = _alloc_q(shape, q, plan, _lib.LAYOUT_NATURAL, array.device)
    zp = None if zero_point is None else zero_point.contiguous()
    _lib.call('qwix_hip_quantize_with_scale_noise', array.data_ptr(), _lib.float_tag(array.dtype), *plan.dims,
              plan.tiles[0], numerics.qtype_tag(q), scale.data_ptr(), _lib.ptr(zp), noise.data_ptr(), data.data_ptr(),
              _lib.stream_of(array))
    return QArray(view, scale, zero_point, q)
  lay = _default_layout(plan, layout, shape, q)
  data, view = _alloc_q(shape, q, plan, lay, array.device)
  zp = None if zero_point is None else zero_point.contiguous()
  _lib.call('qwix_hip_quantize_with_scale', array.data_ptr(), _lib.float_tag(array.dtype), *plan.dims, plan.tiles[0],
            numerics.qtype_tag(q), scale.data_ptr(), _lib.ptr(zp), lay, data.data_ptr(), _lib.stream_of(array))
  return QArray(view, scale, zero_point, q)


def quantize(array: torch.Tensor, how: HowToQuantize, *, layout: str | None = None) -> QArray:
  """Dynamic-range quantization: calibrate, derive scale (and zero point), quantize -- one fused pass.  With a
  `noise_fn` (stochastic rounding) the three steps run one after the other, as the reference's do (qarray.py:638-644)."""
  if how.noise_fn is not None and numerics.canonical_qtype(how.qtype) in (numerics.INT8, numerics.INT4) and array.numel():
    scale, zp = compute_scale_zero_point(calibrate(array, how), how.qtype)
    return quantize_with_scale_zero_point(array, how.qtype, scale, zp, how.noise_fn, layout='natural')
  if not isinstance(array, torch.Tensor) or not numerics.should_quantize(array.dtype):
    raise ValueError(f'Refuse to quantize: {getattr(array, "dtype", type(array))}')
  shape = tuple(array.shape)
  q = numerics.canonical_qtype(how.qtype)
  if q == numerics.INT4 and array.ndim > 1 and shape[-1] % 2 and layout is None and math.prod(shape):
    # Packed int4 pairs run along one axis of even length; the natural layout takes the last one.  With an odd last
    # axis the array is quantized with an even axis moved to the end (one copy) and the packed values are handed back
    # as a view in the caller's axis order.
    even = [a for a in range(array.ndim - 1) if shape[a] % 2 == 0]
    if even:
      a = even[-1]
      order = [d for d in range(array.ndim) if d != a] + [a]        # new axis i is old axis order[i]
      new_of = {old: new for new, old in enumerate(order)}
      how2 = dataclasses.replace(
          how, channelwise_axes=tuple(new_of[c % array.ndim] for c in how.channelwise_axes),
          tiled_axes={new_of[k % array.ndim]: v for k, v in how.tiled_axes.items()})
      q2 = quantize(array.permute(*order).contiguous(), how2, layout='natural')
      inv = [new_of[d] for d in range(array.ndim)]
      back = lambda t: None if t is None else t.permute(*inv).contiguous()
      return QArray(q2.qvalue.permute(*inv), back(q2.scale), back(q2.zero_point), q)
  sshape = get_scale_shape(shape, how)
  fixed = _fixed_calibration(how.calibration_method, array)
  if fixed is None:  # rms: its own reduction kernel, then the static-scale kernel
    fixed = _rms_calibration(how.calibration_method, array, sshape, _tiles_from_how(shape, how) if array.numel() else ())
  if fixed is not None:  # a constant range: the static-scale kernel, with one scale for the whole array
    scale, zp = compute_scale_zero_point(fixed, q)
    return quantize_with_scale_zero_point(array, q, scale, zp, layout=layout)
  cal, factor = _parse_calibration(how.calibration_method)
  if cal == _lib.MINMAX:
    numerics.get_asymmetric_bound(q)
  if array.numel() == 0:
    _check_empty_reduction(sshape)
    zp = torch.empty(sshape, dtype=torch.int8, device=array.device) if cal == _lib.MINMAX else None
    return QArray(_empty_qvalue(shape, q, array.device), torch.empty(sshape, dtype=array.dtype, device=array.device), zp, q)
  try:
    plan = _plan(shape, tuple(d // s for d, s in zip(shape, sshape)))
  except NotImplementedError:
    if layout not in (None, 'natural'):
      raise
    return _quantize_regrouped(_check_float_input(array), how, q, sshape)
  if not array.is_contiguous() and plan.kind == '3d' and plan.dims[2] > 1 and layout in (None, 'reduce_minor'):
    # A strided view whose reduced axes are already the contiguous ones (e.g. a rotated weight kept
    # K-contiguous): quantize its physical rows and hand back views with the logical shape.
    order = plan.outer_axes + plan.inner_axes + plan.reduce_axes
    phys = array.permute(*order)
    if phys.is_contiguous():
      nr = len(plan.reduce_axes)
      phys_how = HowToQuantize(
          qtype=q, channelwise_axes=tuple(range(phys.ndim - nr)),
          tiled_axes={phys.ndim - nr: plan.tiles[0] // math.prod(shape[a] for a in plan.reduce_axes[1:])}
          if plan.tiles[0] != plan.dims[1] else {},
          calibration_method=how.calibration_method)
      pq = quantize(phys, phys_how, layout='natural')
      inv = [order.index(a) for a in range(len(shape))]
      qv = pq.qvalue.permute(*inv)
      zp = None if pq.zero_point is None else pq.zero_point.permute(*inv).contiguous()
      return QArray(qv, pq.scale.permute(*inv).contiguous(), zp, q)
  array = _check_float_input(array)
  scale = torch.empty(sshape, dtype=array.dtype, device=array.device)
  zp = torch.empty(sshape, dtype=torch.int8, device=array.device) if cal == _lib.MINMAX else None
  tag = _lib.float_tag(array.dtype)
  if plan.kind == '5d':
    data, view = _alloc_q(shape, q, plan, _lib.LAYOUT_NATURAL, array.device)
    import ctypes
    dims = (ctypes.c_int64 * 5)(*plan.dims)
    _lib.call('qwix_hip_quantize_generic', array.data_ptr(), tag, dims, plan.tiles[0], plan.tiles[1],
              numerics.qtype_tag(q), cal, factor, data.data_ptr(), scale.data_ptr(), _lib.ptr(zp),
              _lib.stream_of(array))
    return QArray(view, scale, zp, q)
  lay = _default_layout(plan, layout, shape, q)
  outer, reduce, inner = plan.dims
  if (inner > 1 and (inner % (8 if array.dtype == torch.bfloat16 else 4) != 0)) or (
      q == numerics.INT4 and inner == 1 and plan.tiles[0] % 2):
    # ragged strided reduce, or int4 groups of odd length (a nibble pair straddles two groups): the
    # complete-but-slow kernel handles it (natural layout).
    data, view = _alloc_q(shape, q, plan, _lib.LAYOUT_NATURAL, array.device)
    import ctypes
    dims = (ctypes.c_int64 * 5)(outer, reduce, inner, 1, 1)
    _lib.call('qwix_hip_quantize_generic', array.data_ptr(), tag, dims, plan.tiles[0], 1, numerics.qtype_tag(q), cal,
              factor, data.data_ptr(), scale.data_ptr(), _lib.ptr(zp), _lib.stream_of(array))
    return QArray(view, scale, zp, q)
  data, view = _alloc_q(shape, q, plan, lay, array.device)
  ws, nws = _workspace(plan, cal, array.device)
  _lib.call('qwix_hip_quantize', array.data_ptr(), tag, outer, reduce, inner, plan.tiles[0], numerics.qtype_tag(q), cal,
            factor, lay, data.data_ptr(), scale.data_ptr(), _lib.ptr(zp), _lib.ptr(ws), nws, _lib.stream_of(array))
  return QArray(view, scale, zp, q)


def quantize_api(array: torch.Tensor, qtype, *, channelwise_axes: Collection[int] = (),
                 tiled_axes: Mapping[int, int | float] | None = None, calibration_method: str = 'absmax',
                 scale_dtype: torch.dtype | None = None, layout: str | None = None) -> QArray:
  """Public `qwix.quantize`: like quantize() without building a HowToQuantize; the optional
  scale_dtype cast is applied to the already computed scale."""
  how = HowToQuantize(qtype=qtype, channelwise_axes=channelwise_axes, tiled_axes=tiled_axes or {},
                      calibration_method=calibration_method)
  qa = quantize(array, how, layout=layout)
  if scale_dtype is not None:
    qa = dataclasses.replace(qa, scale=qa.scale.to(scale_dtype))
  return qa


# ------------------------------------------------------------------------------------------
# dequantize
# ------------------------------------------------------------------------------------------


def physical_layout(qa: QArray) -> tuple[_Plan, int, torch.Tensor]:
  """Finds how a QArray's values are laid out: (plan, layout tag, storage tensor)."""
  shape = qa.shape
  plan = _plan(shape, qa.scale_tile_shape)
  is4 = isinstance(qa.qvalue, Int4Tensor)
  data = qa.qvalue.data if is4 else qa.qvalue
  if data.is_contiguous() and (not is4 or qa.qvalue.packed_axis == len(shape) - 1):
    return plan, _lib.LAYOUT_NATURAL, data
  if plan.kind == '3d':
    order = _reduce_minor_order(shape, plan)
    phys = data.permute(*order)
    if phys.is_contiguous() and (not is4 or qa.qvalue.packed_axis == order[-1]):
      return plan, _lib.LAYOUT_REDUCE_MINOR, phys
  if not is4:  # any other strided view (a slice of a batch, a transposed copy): one compaction
    return plan, _lib.LAYOUT_NATURAL, data.contiguous()
  raise Int4LayoutError(
      f'int4 values of shape {shape} with strides {tuple(data.stride())} are neither row-major nor '
      'reduce-minor; make them contiguous first.'
  )


def dequantize(array: QArray) -> torch.Tensor:
  """(qvalue - zero_point) * scale in the scale dtype; the reverse of quantize."""
  validate_qarray(array)
  if math.prod(array.shape) == 0:
    return torch.empty(array.shape, dtype=array.scale.dtype, device=array.scale.device)
  try:
    plan, lay, data = physical_layout(array)
  except Int4LayoutError:
    # packed pairs along an axis that is neither the last nor the reduced one: the same integers, one byte each
    return dequantize(QArray(array.qvalue.unpack().contiguous(), array.scale, array.zero_point, numerics.INT8))
  except NotImplementedError as e:
    if 'separate reduced axis groups' not in str(e):
      raise
    # more than two separate groups of reduced axes: gather the elements of a scale into a row, dequantize the rows,
    # put the values back (a copy each way)
    shape, sshape = tuple(array.shape), tuple(array.scale.shape)
    _, split, perm, rows, cols = _regrouped(shape, sshape)
    vals = array.qvalue.unpack() if isinstance(array.qvalue, Int4Tensor) else array.qvalue
    v2 = vals.reshape(split).permute(*perm).reshape(rows, cols).contiguous()
    q2 = QArray(v2, array.scale.reshape(rows, 1), None if array.zero_point is None else array.zero_point.reshape(rows, 1),
                numerics.INT8 if array.qtype == numerics.INT4 else array.qtype)
    return _ungroup(dequantize(q2), shape, sshape).contiguous()
  out = torch.empty(array.shape, dtype=array.scale.dtype, device=array.scale.device)
  scale = array.scale.contiguous()
  zp = None if array.zero_point is None else array.zero_point.contiguous()
  if plan.kind != '3d':  # two reduced axis groups (block scales); physical_layout only passes the natural layout
    import ctypes
    dims = (ctypes.c_int64 * 5)(*plan.dims)
    _lib.call('qwix_hip_dequantize_generic', data.data_ptr(), numerics.qtype_tag(array.qtype), dims, plan.tiles[0],
              plan.tiles[1], scale.data_ptr(), _lib.ptr(zp), _lib.float_tag(scale.dtype), out.data_ptr(),
              _lib.stream_of(scale))
    return out
  _lib.call('qwix_hip_dequantize', data.data_ptr(), numerics.qtype_tag(array.qtype), lay, *plan.dims, plan.tiles[0],
            scale.data_ptr(), _lib.ptr(zp), _lib.float_tag(scale.dtype), out.data_ptr(), _lib.stream_of(scale))
  return out


# ------------------------------------------------------------------------------------------
# generic broadcast
# ------------------------------------------------------------------------------------------


def _broadcast_tensor(x: torch.Tensor, shape: tuple[int, ...]) -> torch.Tensor:
  """An axis of size s grows to a multiple t * s by repeating each element t times (size 1: plain
  broadcast) -- call_with_generic_broadcast of qarray.py:425-444 against an array of the target shape."""
  if x.ndim < len(shape):
    x = x.reshape((1,) * (len(shape) - x.ndim) + tuple(x.shape))
  if x.ndim != len(shape):
    raise ValueError(f'Cannot broadcast between {tuple(x.shape)} {shape}')
  for axis, (have, want) in enumerate(zip(x.shape, shape)):
    if have == want:
      continue
    if have == 0 or want % have:
      raise ValueError(f'Cannot broadcast between {tuple(x.shape)} {shape}')
    x = x.repeat_interleave(want // have, dim=axis) if have != 1 else x.expand(*[want if a == axis else d for a, d in enumerate(x.shape)])
  return x


def broadcast_to(operand, target_shape):
  """qarray.py:447-467 for arrays and QArrays.  The values are repeated tile-wise; scale and zero point grow
  only where they were finer than per-tensor along a growing axis (each element keeps its own scale, the
  scale stays as small as it can), where the reference materialises them at the full target shape."""
  target_shape = tuple(int(d) for d in target_shape)
  if tuple(operand.shape) == target_shape:
    return operand
  if not isinstance(operand, QArray):
    return _broadcast_tensor(operand, target_shape)
  if isinstance(operand.qvalue, Int4Tensor):
    raise NotImplementedError('broadcasting packed int4 values is not supported')
  qs = tuple(operand.shape)
  if len(qs) != len(target_shape):
    raise ValueError(f'Cannot broadcast between {qs} {target_shape}')

  def small(x):
    if x is None:
      return None
    want = tuple(k if (s == t or k == 1) else k * (t // s) for k, s, t in zip(x.shape, qs, target_shape))
    return _broadcast_tensor(x, want).contiguous()

  return QArray(_broadcast_tensor(operand.qvalue, target_shape).contiguous(), small(operand.scale),
                small(operand.zero_point), operand.qtype)


# ------------------------------------------------------------------------------------------
# dtype rule
# ------------------------------------------------------------------------------------------

_INT_NAMES = ('int8', 'int4', 'uint8', 'int16', 'int32')


def _dtype_names(x) -> tuple[str, str]:
  """(qvalue dtype name, dequant dtype name) of an operand."""
  name = lambda d: str(d).replace('torch.', '')
  if isinstance(x, QArray):
    qn = 'int4' if isinstance(x.qvalue, Int4Tensor) else name(x.qvalue.dtype)
    return qn, name(x.scale.dtype)
  if isinstance(x, Int4Tensor):
    return 'int4', 'int4'
  return name(x.dtype), name(x.dtype)


_TORCH = {'float32': torch.float32, 'bfloat16': torch.bfloat16, 'int32': torch.int32}


def get_accumulator_and_result_type(*args, preferred_element_type=None):
  """(accumulator dtype, result dtype) of a quantized contraction (qarray.py:781-821).

  The result type depends only on the dequantized dtypes (raw 1-byte ints count as int32, other
  1-byte types as bf16) unless preferred_element_type is given; the accumulator is int32 iff every
  operand's stored values are integers, otherwise it equals the result type.
  """
  qnames, dnames = zip(*[_dtype_names(a) for a in args])
  result = preferred_element_type
  if result is None:
    ds = []
    for n in dnames:
      if n in ('int8', 'int4', 'uint8'):
        ds.append(torch.int32)
      elif n in ('bool', 'float8_e4m3fn', 'float8_e5m2'):
        ds.append(torch.bfloat16)
      else:
        ds.append(_TORCH[n])
    floats = [d for d in ds if d.is_floating_point]
    if not floats:
      result = torch.int32
    else:
      result = torch.float32 if torch.float32 in floats else torch.bfloat16
  acc = torch.int32 if all('int' in n for n in qnames) else result
  return acc, result
