"""Quantized dot_general on MI355X: the host-side operator in front of the MFMA GEMM kernels.

Mirror of qwix/_src/core/dot_general.py: `get_how_to_quantize` (:28-76), the dispatcher
`dot_general` (:407-491) with its 128 threshold (:404), `_fast_dot_general` (:135-261,
quantized contraction + dequantize on output) and `_slow_dot_general` (:264-275, dequantize
first).  Arguments are torch tensors / QArrays in HBM; `dimension_numbers` is
((lhs_contracting, rhs_contracting), (lhs_batch, rhs_batch)) as in jax.lax.dot_general.

What reaches a hand-written kernel:
  int8 x int8, e4m3 x e4m3 (per-row x per-column scales)          -> qwix_hip_qgemm
  int8 x int8/int4 with K-group scales (tile % 128 == 0)          -> qwix_hip_qgemm_grouped
  bf16 activations x int4/int8/e4m3 weight (weight-only, any group) -> qwix_hip_gemv_wq up to 32..80 rows,
      qwix_hip_gemm_bf16_wq (int4 up to 1024 rows, int8 and e4m3 up to one round of tiles),
      qwix_hip_dequantize_rm + qwix_hip_gemm_bf16 above
Everything else on the slow path is dequantized by the HIP dequantize kernel and contracted by
the vendor float GEMM.  Unsupported fast-path combinations raise; they never change path silently.
"""
from __future__ import annotations

import functools
import math
import weakref
from typing import Any, Mapping, Sequence

import torch

from qwix_amd import _lib
from qwix_amd.core import numerics
from qwix_amd.core import qarray
from qwix_amd.core.qarray import Int4Tensor, QArray

DotDimensionNumbers = tuple[tuple[Sequence[int], Sequence[int]], tuple[Sequence[int], Sequence[int]]]


def get_how_to_quantize(*, dimension_numbers: DotDimensionNumbers, ndims: tuple[int, int], for_lhs: bool,
                        tile_size: Mapping[int, int | float] | int | float | None, **kwargs: Any) -> qarray.HowToQuantize:
  """Channelwise on every non-contracting axis; sub-channel tiles on the last contracting axis
  when tile_size is given (a mapping is used verbatim)."""
  side = 0 if for_lhs else 1
  ndim, contracting = ndims[side], tuple(dimension_numbers[0][side])
  if isinstance(tile_size, Mapping):
    tiled = dict(tile_size)
  else:
    tiled = {contracting[-1]: tile_size} if tile_size else {}
  channelwise = sorted(set(range(ndim)) - set(contracting) - set(tiled))
  return qarray.HowToQuantize(channelwise_axes=channelwise, tiled_axes=tiled, **kwargs)


# If a contracting axis is tiled finer than this, dequantize the inputs instead (dot_general.py:404).
MIN_TILE_SIZE_TO_DEQUANT_ON_OUTPUT = 128


def _is_float_array(x) -> bool:
  return isinstance(x, torch.Tensor) and numerics.should_quantize(x.dtype)


def _use_fast_path(lhs, rhs, dimension_numbers) -> bool:
  for operand, ca in zip((lhs, rhs), dimension_numbers[0]):
    if not isinstance(operand, QArray):
      if _is_float_array(operand):
        return False
      continue
    qarray.validate_qarray(operand)
    if not numerics.can_dequant_on_output(operand.qtype):
      return False
    for axis in ca:
      if operand.scale.shape[axis] > 1:
        if operand.shape[axis] // operand.scale.shape[axis] < MIN_TILE_SIZE_TO_DEQUANT_ON_OUTPUT:
          return False
  return True


# ------------------------------------------------------------------------------------------
# 2-D canonical form
# ------------------------------------------------------------------------------------------


def _broadcast_free(s: torch.Tensor, shape: Sequence[int], free: Sequence[int]) -> torch.Tensor:
  """Brings the scale (or zero point) to full size along the non-contracted axes: a per-tensor entry is
  expanded, a tiled axis repeats each entry over its tile -- the generic broadcast the reference applies to
  the result (qarray.py:425-444), done on the small array instead."""
  if all(s.shape[a] == shape[a] for a in free):
    return s
  for a in free:
    if s.shape[a] not in (1, shape[a]):
      s = s.repeat_interleave(shape[a] // s.shape[a], dim=a)
  return s.expand(*[shape[a] if a in free else s.shape[a] for a in range(s.ndim)])


class _Canon:
  """lhs as (M, K) row-major, rhs as (N, K) K-contiguous, plus scales in kernel order."""

  def __init__(self, lhs, rhs, dimension_numbers):
    (lca, rca), (lba, rba) = dimension_numbers
    lca, rca = [int(a) for a in lca], [int(a) for a in rca]
    if len(lba) or len(rba):
      raise ValueError('batch dimensions are peeled off before the 2-D canonical form')
    if len(lca) != len(rca) or not lca:
      raise ValueError(f'bad contracting axes {lca} {rca}')
    lshape, rshape = tuple(lhs.shape), tuple(rhs.shape)
    for l, r in zip(lca, rca):
      if lshape[l] != rshape[r]:
        raise ValueError(f'contracting dimensions differ: lhs {lshape} axis {l} vs rhs {rshape} axis {r}')
    pairs = sorted(zip(lca, rca))
    self.lca = [p[0] for p in pairs]
    self.rca = [p[1] for p in pairs]
    self.lfree = [a for a in range(len(lshape)) if a not in self.lca]
    self.rfree = [a for a in range(len(rshape)) if a not in self.rca]
    self.M = math.prod(lshape[a] for a in self.lfree)
    self.N = math.prod(rshape[a] for a in self.rfree)
    self.K = math.prod(lshape[a] for a in self.lca)
    self.out_shape = tuple(lshape[a] for a in self.lfree) + tuple(rshape[a] for a in self.rfree)

  # -- values
  def lhs_values(self, lhs) -> torch.Tensor:
    v = lhs.qvalue if isinstance(lhs, QArray) else lhs
    if isinstance(v, Int4Tensor):
      v = v.unpack()  # int4 activations are widened to int8 (exact); the MFMA kernels take int8 rows
    v = v.permute(*(self.lfree + self.lca))  # contracting axes last (a no-op view in the usual layout)
    v = v if v.is_contiguous() else v.contiguous()
    if v.data_ptr() % 16:  # a contiguous view that starts inside a 16-byte unit: the kernels load 16 bytes per lane
      v = v.clone()
    v = v.reshape(self.M, self.K)
    if self.M == 1 and v.stride(0) != self.K:  # a single row keeps whatever pitch its parent had
      v = v.as_strided((1, self.K), (self.K, 1))
    return v

  def rhs_values(self, rhs) -> tuple[torch.Tensor, bool]:
    """(N, K) K-contiguous storage (for int4: (N, K/2) bytes), is_int4."""
    v = rhs.qvalue if isinstance(rhs, QArray) else rhs
    order = self.rfree + self.rca
    if isinstance(v, Int4Tensor):
      p = v.permute(*order)
      if p.packed_axis == len(order) - 1 and p.data.is_contiguous():
        return p.data.reshape(self.N, self.K // 2), True
      nat = v.permute(*(self.rca + self.rfree))
      if nat.packed_axis == len(order) - 1 and nat.data.is_contiguous():
        dst = torch.empty(self.N, self.K // 2, dtype=torch.uint8, device=v.device)
        _lib.call('qwix_hip_transpose_q', nat.data.data_ptr(), _lib.INT4, self.K, self.N, dst.data_ptr(),
                  _lib.stream_of(dst))
        return dst, True
      raise qarray.Int4LayoutError(f'int4 weight layout {v} cannot be brought to K-contiguous form')
    p = v.permute(*order)
    if p.is_contiguous():
      return p.reshape(self.N, self.K), False
    nat = v.permute(*(self.rca + self.rfree))
    if nat.is_contiguous() and v.element_size() == 1:
      dst = torch.empty(self.N, self.K, dtype=v.dtype, device=v.device)
      _lib.call('qwix_hip_transpose_q', nat.data_ptr(), _lib.INT8, self.K, self.N, dst.data_ptr(), _lib.stream_of(dst))
      return dst, False
    return p.contiguous().reshape(self.N, self.K), False

  # -- scales
  def lhs_scale(self, lhs: QArray) -> tuple[torch.Tensor | None, int]:
    """(scale as (M, ga) contiguous, ga)."""
    s = lhs.scale
    for a in self.lca[:-1]:
      if s.shape[a] != 1:
        raise NotImplementedError('only the last contracting axis of the lhs may carry sub-channel scales')
    ga = s.shape[self.lca[-1]]
    if ga > 1 and len(self.lca) > 1:
      raise NotImplementedError('sub-channel lhs scales with several contracting axes are not supported')
    s = _broadcast_free(s, lhs.shape, self.lfree)
    return s.permute(*(self.lfree + self.lca)).reshape(self.M, ga).contiguous(), ga

  def rhs_scale(self, rhs: QArray) -> tuple[torch.Tensor | None, int]:
    """(scale as (gb, N) contiguous, gb)."""
    s = rhs.scale
    for a in self.rca[:-1]:
      if s.shape[a] != 1:
        raise NotImplementedError('only the last contracting axis of the rhs may carry sub-channel scales')
    gb = s.shape[self.rca[-1]]
    if gb > 1 and len(self.rca) > 1:
      raise NotImplementedError('sub-channel rhs scales with several contracting axes are not supported')
    s = _broadcast_free(s, rhs.shape, self.rfree)
    s = s.permute(*([self.rca[-1]] + self.rfree + self.rca[:-1]))
    return s.reshape(gb, self.N).contiguous(), gb


  # -- zero points: shaped like the scales; int32 for the kernels
  def lhs_zero_point(self, lhs: QArray) -> tuple[torch.Tensor, int]:
    """(zero points as (M, gz) int32 contiguous, gz): gz > 1 when the last contracting axis is tiled."""
    z = lhs.zero_point
    if any(z.shape[a] != 1 for a in self.lca[:-1]):
      raise NotImplementedError('only the last contracting axis of the lhs may carry sub-channel zero points')
    gz = z.shape[self.lca[-1]]
    if gz > 1 and len(self.lca) > 1:
      raise NotImplementedError('sub-channel lhs zero points with several contracting axes are not supported')
    z = _broadcast_free(z, lhs.shape, self.lfree)
    return z.permute(*(self.lfree + self.lca)).reshape(self.M, gz).to(torch.int32).contiguous(), gz

  def rhs_zero_point(self, rhs: QArray) -> tuple[torch.Tensor, int]:
    """(zero points as (gz, N) int32 contiguous, gz)."""
    z = rhs.zero_point
    if any(z.shape[a] != 1 for a in self.rca[:-1]):
      raise NotImplementedError('only the last contracting axis of the rhs may carry sub-channel zero points')
    gz = z.shape[self.rca[-1]]
    if gz > 1 and len(self.rca) > 1:
      raise NotImplementedError('sub-channel rhs zero points with several contracting axes are not supported')
    z = _broadcast_free(z, rhs.shape, self.rfree)
    z = z.permute(*([self.rca[-1]] + self.rfree + self.rca[:-1]))
    return z.reshape(gz, self.N).to(torch.int32).contiguous(), gz


# ------------------------------------------------------------------------------------------
# batch dimensions
# ------------------------------------------------------------------------------------------


def _index_batch(x, axes: Sequence[int], idx: Sequence[int]):
  """x[..., idx_k at axes_k, ...] for a tensor or a QArray (scale / zero point axes of size 1 broadcast)."""
  def take(t):
    if isinstance(t, Int4Tensor):  # index the packed bytes; the pairs must not run along a batch axis
      if t.packed_axis in axes:
        raise qarray.Int4LayoutError('int4 values packed along a batch axis are not supported')
      sel = [slice(None)] * t.ndim
      for a, i in zip(axes, idx):
        sel[a] = i
      kept = [a for a in range(t.ndim) if a not in axes]
      return Int4Tensor(t.data[tuple(sel)], tuple(t.shape[a] for a in kept), kept.index(t.packed_axis))
    sel = [slice(None)] * t.ndim
    for a, i in zip(axes, idx):
      sel[a] = i if t.shape[a] != 1 else 0
    return t[tuple(sel)]
  if isinstance(x, QArray):
    return QArray(take(x.qvalue), take(x.scale), None if x.zero_point is None else take(x.zero_point), x.qtype)
  return take(x)


def _drop_axes(axes: Sequence[int], dropped: Sequence[int]) -> list[int]:
  """Axis numbers after the `dropped` axes have been indexed away."""
  return [a - sum(1 for d in dropped if d < a) for a in axes]


def _over_batch(fn, lhs, rhs, dimension_numbers, **kwargs) -> torch.Tensor:
  """Runs the 2-D operator once per batch element: out[b..., lhs free..., rhs free...], the layout of
  lax.dot_general.  One kernel launch per element; the quantized values are sliced as views."""
  (lca, rca), (lba, rba) = dimension_numbers
  lba, rba = [int(a) for a in lba], [int(a) for a in rba]
  if len(lba) != len(rba):
    raise ValueError(f'batch axes differ in number: {lba} {rba}')
  bshape = [lhs.shape[a] for a in lba]
  if bshape != [rhs.shape[a] for a in rba]:
    raise ValueError(f'batch dimensions differ: lhs {tuple(lhs.shape)} axes {lba} vs rhs {tuple(rhs.shape)} axes {rba}')
  dn = ((_drop_axes(lca, lba), _drop_axes(rca, rba)), ((), ()))
  outs = []
  for flat in range(math.prod(bshape)):
    idx, rem = [], flat
    for d in reversed(bshape):
      idx.append(rem % d)
      rem //= d
    idx.reverse()
    outs.append(fn(_index_batch(lhs, lba, idx), _index_batch(rhs, rba, idx), dn, **kwargs))
  return torch.stack(outs).reshape(*bshape, *outs[0].shape)


def _batched_qgemm(lhs, rhs, dimension_numbers, preferred_element_type):
  """All batch elements in one launch (qwix_hip_qgemm_batched) for the common case: two QArrays of int8
  or e4m3 values with per-row / per-column scales and no zero point.  Returns None when the operands
  need the general route (one launch per batch element)."""
  if not (isinstance(lhs, QArray) and isinstance(rhs, QArray)):
    return None
  if lhs.zero_point is not None or rhs.zero_point is not None:
    return None
  if isinstance(lhs.qvalue, Int4Tensor) or isinstance(rhs.qvalue, Int4Tensor):
    return None
  lq, rq = _qtype_of(lhs), _qtype_of(rhs)
  if (lq, rq) == (numerics.INT8, numerics.INT8):
    qt = _lib.INT8
  elif (lq, rq) == (numerics.E4M3, numerics.E4M3):
    qt = _lib.E4M3
  else:
    return None
  (lca, rca), (lba, rba) = dimension_numbers
  lca, rca, lba, rba = ([int(a) for a in x] for x in (lca, rca, lba, rba))
  lshape, rshape = tuple(lhs.shape), tuple(rhs.shape)
  if len(lba) != len(rba) or [lshape[a] for a in lba] != [rshape[a] for a in rba]:
    return None  # the general route reports the error
  if len(lca) != len(rca) or not lca or [lshape[a] for a in lca] != [rshape[a] for a in rca]:
    return None
  if any(lhs.scale.shape[a] != 1 for a in lca) or any(rhs.scale.shape[a] != 1 for a in rca):
    return None  # sub-channel scales
  lfree = [a for a in range(len(lshape)) if a not in lca and a not in lba]
  rfree = [a for a in range(len(rshape)) if a not in rca and a not in rba]
  bshape = [lshape[a] for a in lba]
  Bt, M, N, K = (math.prod(bshape), math.prod(lshape[a] for a in lfree), math.prod(rshape[a] for a in rfree),
                 math.prod(lshape[a] for a in lca))
  if not (0 < Bt <= 65535) or M == 0 or N == 0 or K % 16:
    return None
  acc_t, res_t = qarray.get_accumulator_and_result_type(lhs, rhs, preferred_element_type=preferred_element_type)

  def values(q, order, rows):
    v = q.qvalue.permute(*order)
    return (v if v.is_contiguous() else v.contiguous()).reshape(Bt, rows, K)

  def scales(q, shape, contracting, order, rows):
    s = q.scale.expand(*[1 if a in contracting else shape[a] for a in range(len(shape))])
    return s.permute(*order).reshape(Bt, rows).contiguous()

  a = values(lhs, lba + lfree + lca, M)
  b = values(rhs, rba + rfree + rca, N)
  sa = scales(lhs, lshape, lca, lba + lfree + lca, M)
  sb = scales(rhs, rshape, rca, rba + rfree + rca, N)
  out = torch.empty(Bt, M, N, dtype=res_t, device=a.device)
  _lib.call('qwix_hip_qgemm_batched', a.data_ptr(), K, M * K, b.data_ptr(), K, N * K, qt, Bt, M, N, K,
            sa.data_ptr(), _lib.float_tag(sa.dtype), M, sb.data_ptr(), _lib.float_tag(sb.dtype), N,
            _tag_of(acc_t) if acc_t != torch.int32 else 0, out.data_ptr(), _tag_of(res_t), N, M * N,
            _lib.stream_of(a))
  return out.reshape(*bshape, *[lshape[a] for a in lfree], *[rshape[a] for a in rfree])


def fused_act_dot_general(lhs, rhs, dimension_numbers, preferred_element_type=None, act_qtype=numerics.INT8):
  """Dynamic per-token quantization of a float lhs (absmax over the whole contraction, to the weight's own
  qtype: int8 or e4m3) and the quantized contraction against a per-channel weight in one library call
  (qwix_hip_qgemm_dynamic_act): one launch at decode sizes, the quantize kernel and the GEMM back to back on a
  scratch buffer otherwise.  Bit-identical to quantize(lhs, channelwise over the non-contracting axes)
  followed by dot_general.  Returns None when the operands are not of that kind; the caller then takes the
  two-step route."""
  if not (_is_float_array(lhs) and lhs.dtype in (torch.bfloat16, torch.float32) and isinstance(rhs, QArray)):
    return None
  if rhs.zero_point is not None or isinstance(rhs.qvalue, Int4Tensor):
    return None
  if act_qtype not in (numerics.INT8, numerics.E4M3) or _qtype_of(rhs) != act_qtype:
    return None
  (lca, rca), (lba, rba) = dimension_numbers
  if len(lba) or len(rba) or any(rhs.scale.shape[int(a)] != 1 for a in rca):
    return None
  try:
    c = _Canon(lhs, rhs, dimension_numbers)
  except ValueError:
    return None
  if c.M <= 0 or c.K % 16:
    return None
  # qarray.py:781-821 for a (quantized lhs with scales in lhs.dtype, rhs) pair: integer values accumulate in
  # int32, e4m3 values in the result type.
  res_t = preferred_element_type or torch.promote_types(lhs.dtype, rhs.scale.dtype)
  acc_t = torch.int32 if act_qtype == numerics.INT8 else res_t
  if res_t not in (torch.bfloat16, torch.float32):
    return None
  x = c.lhs_values(lhs)
  if x.stride(1) != 1 or x.stride(0) != c.K:
    x = x.contiguous()
  b, _ = c.rhs_values(rhs)
  sb, _ = c.rhs_scale(rhs)
  out = torch.empty(c.M, c.N, dtype=res_t, device=x.device)
  nws = _dynamic_act_bytes(c.M, c.N, c.K, _lib.float_tag(x.dtype))
  ws = torch.empty(nws, dtype=torch.uint8, device=x.device) if nws else None
  _lib.call('qwix_hip_qgemm_dynamic_act', x.data_ptr(), _lib.float_tag(x.dtype), x.stride(0), b.data_ptr(), b.stride(0),
            _lib.INT8 if act_qtype == numerics.INT8 else _lib.E4M3, c.M, c.N, c.K, sb.data_ptr(),
            _lib.float_tag(sb.dtype), _tag_of(acc_t) if acc_t != torch.int32 else 0, out.data_ptr(),
            _lib.float_tag(res_t), c.N, _lib.ptr(ws), nws, _lib.stream_of(x))
  return out.reshape(c.out_shape)


@functools.lru_cache(maxsize=4096)
def _dynamic_act_bytes(M: int, N: int, K: int, x_tag: int) -> int:
  return int(_lib.load().qwix_hip_qgemm_dynamic_act_workspace_bytes(M, N, K, x_tag))


@functools.lru_cache(maxsize=4096)
def _splitk_bytes(M: int, N: int, K: int) -> int:
  """Scratch bytes with which the GEMM may split K for this shape (0: it would not)."""
  return int(_lib.load().qwix_hip_qgemm_workspace_bytes(M, N, K))


def _tag_of(dtype: torch.dtype) -> int:
  if dtype == torch.int32:
    return _lib.I32
  return _lib.float_tag(dtype)


def _qtype_of(x) -> str:
  if isinstance(x, QArray):
    return numerics.canonical_qtype(x.qtype)
  if isinstance(x, Int4Tensor):
    return numerics.INT4
  return numerics.canonical_qtype(x.dtype)


def _narrow_tiles(x, tiles: Mapping[int, tuple[int, int]]):
  """The operand restricted to tile `i` of `n` elements along every axis of `tiles` ({axis: (i, n)}): values are
  narrowed, scale and zero point keep the one entry of that tile (or their single entry when this operand is not
  tiled along the axis).  Packed int4 values are narrowed in bytes and copied (the kernels need rows that start at
  a byte)."""
  def values(v):
    if isinstance(v, Int4Tensor):
      data, shape = v.data, list(v.shape)
      for a, (i, n) in tiles.items():
        if a == v.packed_axis:
          if n % 2:
            raise NotImplementedError('int4 values tiled by an odd tile size along their packed axis')
          data = data.narrow(a, i * n // 2, n // 2)
        else:
          data = data.narrow(a, i * n, n)
        shape[a] = n
      return Int4Tensor(data.contiguous(), tuple(shape), v.packed_axis)
    for a, (i, n) in tiles.items():
      v = v.narrow(a, i * n, n)
    return v

  def per_tile(t):
    for a, (i, _) in tiles.items():
      if t.shape[a] != 1:
        t = t.narrow(a, i, 1)
    return t

  if isinstance(x, QArray):
    return QArray(values(x.qvalue), per_tile(x.scale), None if x.zero_point is None else per_tile(x.zero_point), x.qtype)
  return values(x)


def _tile_by_tile(lhs, rhs, dimension_numbers, tiled, preferred_element_type, exact) -> torch.Tensor:
  """The tiled contraction of dot_general.py:186-226, 255-260 as the reference writes it, for the operand kinds
  that the sub-channel MFMA kernel does not take (several contracting axes, e4m3 values, tile sizes that are not
  multiples of 128): every tile combination is an untiled contraction of its own (one launch each), scaled by that
  tile's scales with the roundings of the untiled path; the partials are summed in f32 in row-major order of the
  tile axes (the order of the contracting axes) and rounded once to the type the scaled partials have, then cast
  to the result type.  `tiled` lists (lhs axis, rhs axis, tile size)."""
  import itertools
  acc_t, res_t = qarray.get_accumulator_and_result_type(lhs, rhs, preferred_element_type=preferred_element_type)
  cur = acc_t  # dtype of a scaled partial: the accumulator's, promoted by every scale it meets
  for operand in (lhs, rhs):
    if isinstance(operand, QArray):
      sd = operand.scale.dtype
      cur = sd if cur == torch.int32 else torch.promote_types(cur, sd)
  counts = [lhs.shape[l] // n for l, _, n in tiled]
  total = None
  for combo in itertools.product(*[range(c) for c in counts]):
    lsel = {l: (i, n) for (l, _, n), i in zip(tiled, combo)}
    rsel = {r: (i, n) for (_, r, n), i in zip(tiled, combo)}
    part = _fast_dot_general(_narrow_tiles(lhs, lsel), _narrow_tiles(rhs, rsel), dimension_numbers,
                             preferred_element_type=preferred_element_type, exact=exact, _partial_dtype=cur)
    part = part.to(torch.float32) if cur != torch.int32 else part
    total = part if total is None else total + part
  return total.to(cur).to(res_t)


# K-sums of a weight's quantized values (the zero-point correction of an asymmetric activation, dot_general.py:228-253,
# multiplies them with the activation's zero points): weights are static, so the sums are kept per values tensor while it
# is alive and unchanged (identity + torch version counter; entries leave with their tensor).
_KSUM_CACHE: dict = {}


def _weight_ksums(values_owner, b: torch.Tensor, key_extra: tuple, compute) -> torch.Tensor:
  """`values_owner`: the tensor object the weight's QArray holds (its identity and version key the entry; `b` may be a
  re-laid-out copy of it); `compute()` launches the sum kernel and returns the result."""
  store = values_owner.data if isinstance(values_owner, Int4Tensor) else values_owner
  key = (id(store),) + key_extra
  hit = _KSUM_CACHE.get(key)
  if hit is not None and hit[0]() is store and hit[1] == store._version:
    return hit[2]
  out = compute()
  _KSUM_CACHE[key] = (weakref.ref(store, lambda _, k=key: _KSUM_CACHE.pop(k, None)), store._version, out)
  return out


def _fast_dot_general(lhs, rhs, dimension_numbers, preferred_element_type=None, *, exact: bool = False,
                      return_accumulators: bool = False, _partial_dtype=None, **kwargs) -> torch.Tensor:
  """Contract the quantized values on the matrix cores, then scale: out = ((acc * sx) * sy).
  `_partial_dtype` (internal, set by the tile-by-tile route): the dtype the result is delivered in, in place of the
  result type, while the accumulator type still follows `preferred_element_type`."""
  del kwargs
  if _is_float_array(lhs) or _is_float_array(rhs):
    # The reference contracts a raw float operand with the other side's quantized values and scales the
    # result (dot_general.py:135-261 with lhs_scale / rhs_scale None); the dispatcher never sends such a pair
    # here.  It is served by the dequantize-first kernels: the same value up to the rounding of a float dot.
    if return_accumulators:
      raise NotImplementedError('raw accumulators need quantized operands on both sides')
    return _slow_dot_general(lhs, rhs, dimension_numbers, preferred_element_type=preferred_element_type)
  lzp = lhs.zero_point if isinstance(lhs, QArray) else None
  rzp = rhs.zero_point if isinstance(rhs, QArray) else None
  if lzp is not None and rzp is not None:
    raise ValueError('Only one operand can be asymmetric.')
  if len(dimension_numbers[1][0]) or len(dimension_numbers[1][1]):
    if return_accumulators:
      raise NotImplementedError('raw accumulators are not returned for batched contractions')
    out = _batched_qgemm(lhs, rhs, dimension_numbers, preferred_element_type)
    if out is not None:
      return out
    return _over_batch(_fast_dot_general, lhs, rhs, dimension_numbers, preferred_element_type=preferred_element_type,
                       exact=exact)
  c = _Canon(lhs, rhs, dimension_numbers)
  lt = qarray.get_tiled_axes(lhs) if isinstance(lhs, QArray) else {}
  rt = qarray.get_tiled_axes(rhs) if isinstance(rhs, QArray) else {}
  for l, r in zip(c.lca, c.rca):
    if lt.get(l) and rt.get(r) and lt[l] != rt[r]:
      raise ValueError(f'Contracting axes must be tiled with the same tile size. lhs_tiled_axes={lt} rhs_tiled_axes={rt} {dimension_numbers=}')
  acc_t, res_t = qarray.get_accumulator_and_result_type(lhs, rhs, preferred_element_type=preferred_element_type)
  if _partial_dtype is not None:
    res_t = _partial_dtype
  lq, rq = _qtype_of(lhs), _qtype_of(rhs)
  if lq == numerics.INT4:
    lq = numerics.INT8  # lhs_values widens int4 rows
  tiled = [(l, r, lt.get(l) or rt.get(r)) for l, r in zip(c.lca, c.rca) if lt.get(l) or rt.get(r)]
  int_pair = lq == numerics.INT8 and rq in (numerics.INT8, numerics.INT4)
  f8_pair = lq == numerics.E4M3 and rq == numerics.E4M3
  if tiled and (len(c.lca) > 1 or not (int_pair or f8_pair) or any(n % 128 for _, _, n in tiled)):
    # what the sub-channel MFMA kernel does not take runs tile by tile on the untiled kernels
    if return_accumulators:
      raise NotImplementedError('raw accumulators are returned for one tiled contracting axis of int8 x int8/int4 only')
    return _tile_by_tile(lhs, rhs, dimension_numbers, tiled, preferred_element_type, exact)
  a = c.lhs_values(lhs)
  b, b_is4 = c.rhs_values(rhs)
  sa, ga = c.lhs_scale(lhs) if isinstance(lhs, QArray) else (None, 1)
  sb, gb = c.rhs_scale(rhs) if isinstance(rhs, QArray) else (None, 1)
  if b_is4 and ga == 1 and gb == 1 and c.K % 128:
    # per-channel int4 weights whose K the sub-channel kernel does not take: widened to int8 (the same integers)
    b = rhs.qvalue.unpack().permute(*(c.rfree + c.rca)).contiguous().reshape(c.N, c.K)
    b_is4, rq = False, numerics.INT8
  dev = a.device
  st = _lib.stream_of(a)
  out = torch.empty(c.M, c.N, dtype=res_t, device=dev)
  grouped = ga > 1 or gb > 1 or b_is4
  K = c.K
  if not grouped and K % 16:
    # The kernels read K in 16-byte pieces: zero columns (+0 in e4m3 too) add nothing to any sum.
    pad = 16 - K % 16
    a = torch.nn.functional.pad(a.view(torch.uint8), (0, pad)).view(a.dtype)
    b = torch.nn.functional.pad(b.view(torch.uint8), (0, pad)).view(b.dtype)
    K += pad
  if not grouped:
    if (lq, rq) == (numerics.INT8, numerics.INT8):
      qt = _lib.INT8
    elif (lq, rq) == (numerics.E4M3, numerics.E4M3):
      qt = _lib.E4M3
    else:
      raise NotImplementedError(f'no MFMA kernel for {lq} x {rq} operands')
    if lzp is not None or rzp is not None:
      # dot_general.py:228-253: subtract dot(zp, q_other) from the int32 accumulator.  With one zero
      # point per row (lhs) / column (rhs) that is the outer product zero_point x K-sum.
      if qt != _lib.INT8:
        raise NotImplementedError('zero-point operands need int8 x int8 values on the quantized path')
      if return_accumulators:
        raise NotImplementedError('raw accumulators are not returned for zero-point operands')
      if lzp is not None:
        zu = c.lhs_zero_point(lhs)[0].reshape(c.M)

        def ksum():
          zv = torch.empty(c.N, dtype=torch.int32, device=dev)
          _lib.call('qwix_hip_ksum_i8', b.data_ptr(), b.stride(0), c.N, K, zv.data_ptr(), st)
          return zv
        zv = _weight_ksums(rhs.qvalue, b, (tuple(c.rca), tuple(c.rfree), K), ksum)
      else:
        zv = c.rhs_zero_point(rhs)[0].reshape(c.N)
        zu = torch.empty(c.M, dtype=torch.int32, device=dev)
        _lib.call('qwix_hip_ksum_i8', a.data_ptr(), a.stride(0), c.M, K, zu.data_ptr(), st)
      _lib.call('qwix_hip_qgemm_zp', a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), c.M, c.N, K,
                _lib.ptr(sa), 0 if sa is None else _lib.float_tag(sa.dtype), _lib.ptr(sb),
                0 if sb is None else _lib.float_tag(sb.dtype), zu.data_ptr(), zv.data_ptr(), out.data_ptr(),
                _tag_of(res_t), c.N, st)
      return out.reshape(c.out_shape)
    if return_accumulators:
      acc = torch.empty(c.M, c.N, dtype=torch.int32, device=dev)
      _lib.call('qwix_hip_qgemm', a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), qt, c.M, c.N, K, None, 0,
                None, 0, 0, acc.data_ptr(), _lib.I32, c.N, st)
    nws = _splitk_bytes(c.M, c.N, K)
    ws = torch.empty(nws, dtype=torch.uint8, device=dev) if nws else None
    _lib.call('qwix_hip_qgemm_ws', a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), qt, c.M, c.N, K,
              _lib.ptr(sa), 0 if sa is None else _lib.float_tag(sa.dtype), _lib.ptr(sb),
              0 if sb is None else _lib.float_tag(sb.dtype), _tag_of(acc_t) if acc_t != torch.int32 else 0,
              out.data_ptr(), _tag_of(res_t), c.N, _lib.ptr(ws), nws, st)
    out = out.reshape(c.out_shape)
    return (out, acc.reshape(c.out_shape)) if return_accumulators else out
  # sub-channel / int4 weights
  if not (int_pair or f8_pair):
    raise NotImplementedError(f'sub-channel MFMA kernel needs int8 x int8/int4 or e4m3 x e4m3 operands, got {lq} x {rq}')
  if f8_pair and return_accumulators:
    raise NotImplementedError('raw accumulators are int32 partials; e4m3 operands have none')
  ngroups = max(ga, gb)
  if c.K % ngroups or (c.K // ngroups) % 128:
    raise NotImplementedError(f'K-group size {c.K / ngroups} must be a multiple of 128')
  group = c.K // ngroups
  if sb is None:
    raise NotImplementedError('grouped GEMM needs rhs scales')
  if gb != ngroups:  # rhs per-channel, lhs tiled: repeat the rhs scale per group
    sb = sb.expand(ngroups, c.N).contiguous()
  acc = torch.empty(ngroups, c.M, c.N, dtype=torch.int32, device=dev) if return_accumulators else None
  bq = _lib.E4M3 if f8_pair else _lib.INT4 if b_is4 else _lib.INT8
  if lzp is not None or rzp is not None:
    # dot_general.py:196-203, 228-253: the zero point is split with the tiles and every tile's partial is
    # corrected by zero_point x (K-sum of the other operand over that tile) before it is scaled.
    if lzp is not None:
      zu, gz = c.lhs_zero_point(lhs)                       # (M, gz)
      zu_strides = (gz, 1 if gz > 1 else 0)

      def ksum():
        zv = torch.empty(c.N, ngroups, dtype=torch.int32, device=dev)
        _lib.call('qwix_hip_ksum_groups', b.data_ptr(), bq, b.stride(0), c.N, c.K, group, zv.data_ptr(), st)
        return zv
      zv = _weight_ksums(rhs.qvalue, b, (tuple(c.rca), tuple(c.rfree), group), ksum)
      zv_strides = (ngroups, 1)
    else:
      zv, gz = c.rhs_zero_point(rhs)                       # (gz, N)
      zv_strides = (1, c.N if gz > 1 else 0)
      zu = torch.empty(c.M, ngroups, dtype=torch.int32, device=dev)
      _lib.call('qwix_hip_ksum_groups', a.data_ptr(), _lib.INT8, a.stride(0), c.M, c.K, group, zu.data_ptr(), st)
      zu_strides = (ngroups, 1)
    if gz not in (1, ngroups):
      raise ValueError(f'zero points come in {gz} groups along K, the scales in {ngroups}')
    _lib.call('qwix_hip_qgemm_grouped_zp', a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), bq, c.M, c.N, c.K,
              group, _lib.ptr(sa), 0 if sa is None else _lib.float_tag(sa.dtype), ga, sb.data_ptr(),
              _lib.float_tag(sb.dtype), zu.data_ptr(), zu_strides[0], zu_strides[1], zv.data_ptr(), zv_strides[0],
              zv_strides[1], out.data_ptr(), _tag_of(res_t), c.N, int(exact), _lib.ptr(acc), st)
  else:
    # few tiles: K in ranges with f32 partial sums in a workspace (0 bytes: not split; never with `exact`)
    nws = 0 if exact or acc is not None else int(_lib.load().qwix_hip_qgemm_grouped_workspace_bytes(c.M, c.N, c.K, group, bq))
    ws = torch.empty(nws, dtype=torch.uint8, device=dev) if nws else None
    _lib.call('qwix_hip_qgemm_grouped_ws', a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), bq, c.M, c.N, c.K, group,
              _lib.ptr(sa), 0 if sa is None else _lib.float_tag(sa.dtype), ga, sb.data_ptr(), _lib.float_tag(sb.dtype),
              out.data_ptr(), _tag_of(res_t), c.N, int(exact), _lib.ptr(acc), _lib.ptr(ws), nws, st)
  out = out.reshape(c.out_shape)
  return (out, acc.reshape((ngroups,) + c.out_shape)) if return_accumulators else out


# The zero points of a weight in the form the weight-only kernels read ((groups, N) int8, contiguous), kept per
# zero-point tensor and operand order: weights are static, and re-laying them out costs three small launches,
# more than the decode kernel itself takes.
_ZP8_CACHE: dict = {}


def _rhs_zero_point_i8(c: '_Canon', rhs: QArray) -> tuple[torch.Tensor, int]:
  z = rhs.zero_point
  key = (id(z), tuple(c.rca), tuple(c.rfree))
  hit = _ZP8_CACHE.get(key)
  if hit is not None and hit[0]() is z and hit[1] == z._version:
    return hit[2], hit[3]
  z32, gz = c.rhs_zero_point(rhs)
  zp = z32.to(torch.int8).contiguous()
  _ZP8_CACHE[key] = (weakref.ref(z, lambda _, k=key: _ZP8_CACHE.pop(k, None)), z._version, zp, gz)
  return zp, gz


def _weight_only_fit(lhs, rhs, dimension_numbers):
  """The canonical form when the fused weight-only kernels (dequantize in registers, bf16 MFMA) take this pair,
  else None.  The conditions are the kernels' own: a bf16 activation, an int4 / int8 / e4m3 weight whose scales (and zero
  points, if any, in the same groups) are tiled along the last contracting axis only, in groups that are
  multiples of 128."""
  if not (_is_float_array(lhs) and lhs.dtype == torch.bfloat16 and isinstance(rhs, QArray)):
    return None
  if _qtype_of(rhs) not in (numerics.INT4, numerics.INT8, numerics.E4M3):
    return None
  if _qtype_of(rhs) == numerics.E4M3 and rhs.zero_point is not None:
    return None
  c = _Canon(lhs, rhs, dimension_numbers)
  if rhs.zero_point is not None and tuple(rhs.zero_point.shape) != tuple(rhs.scale.shape):
    return None
  if any(rhs.scale.shape[a] != 1 for a in c.rca[:-1]):
    return None
  gb = rhs.scale.shape[c.rca[-1]]
  if (gb > 1 and len(c.rca) > 1) or c.K % 128 or (c.K // gb) % 128:
    return None
  if isinstance(rhs.qvalue, Int4Tensor):  # packed pairs must run along K or along N (one re-layout)
    order = c.rfree + c.rca
    packed = (rhs.qvalue.permute(*order).packed_axis, rhs.qvalue.permute(*(c.rca + c.rfree)).packed_axis)
    if len(order) - 1 not in packed:
      return None
  return c


_I31 = (1 << 31) - 1


def _decode_kernel_limits_ok(ldx: int, ldb_bytes: int, n: int, k: int, group: int, int4: bool, scale_bytes: int) -> bool:
  """The address arithmetic of `qwix_hip_gemv_wq`: 31-bit lane offsets over 32 activation rows, 64 weight rows and the
  whole scale array.  Calls beyond it take the dequantize-first route."""
  brow = k // 2 if int4 else k
  return 32 * ldx * 2 + 2 * k <= _I31 and 64 * ldb_bytes + brow <= _I31 and (k // group) * n * scale_bytes <= _I31


def _bf16_gemm_limits_ok(m: int, lda: int, n: int, ldb_bytes: int) -> bool:
  """`qwix_hip_gemm_bf16` / `qwix_hip_gemm_bf16_wq` address each operand with 31-bit byte offsets."""
  return m * lda * 2 <= _I31 and n * ldb_bytes <= _I31


def _aligned_rows(x: torch.Tensor) -> torch.Tensor:
  """The activation as the kernels want it: unit stride along K, row pitch a multiple of 8 elements, 16-byte aligned
  base.  A view that is not (a slice that starts inside a row) is copied."""
  if x.stride(-1) == 1 and x.data_ptr() % 16 == 0:
    if x.stride(0) % 8 == 0:
      return x
    if x.shape[0] == 1:  # the pitch of a single row means nothing: state a valid one
      return x.as_strided(tuple(x.shape), (x.shape[1], 1))
  # (`contiguous()` would hand a single row back as it is, whatever its pitch and base)
  y = torch.empty(tuple(x.shape), dtype=x.dtype, device=x.device)
  y.copy_(x)
  return y


# Rows up to which the fused weight-only kernel (one pass over the weight per 16 or 32 rows) is used; above
# it the weight is dequantized once (HIP kernel) and contracted by the float GEMM.
WEIGHT_ONLY_MAX_ROWS = 256


# Decode-size calls x (M, K) @ w (K, N) against a static weight spend more time in this module than in the kernel (24 us
# of host work per call against 8.4 us on the device), most of it on the weight: operand checks, layout views, the
# zero-point re-layout.  That part is done once per weight object and kept while the weight is alive and unchanged.
_DECODE_PLANS: dict = {}


def _weight_signature(rhs: QArray) -> tuple:
  """Identity and torch version counter of every tensor a kept plan may hold a re-laid-out COPY of: an in-place update
  (`copy_`, a state reload into existing tensors) keeps the object and bumps the counter."""
  def sig(t):
    if t is None:
      return None
    store = t.data if isinstance(t, Int4Tensor) else t
    return (id(t), id(store), store._version)
  return (sig(rhs.qvalue), sig(rhs.scale), sig(rhs.zero_point))


def _decode_plan(lhs, rhs, dimension_numbers):
  key = id(rhs)
  hit = _DECODE_PLANS.get(key)
  if hit is not None and hit[0]() is rhs and hit[1] == _weight_signature(rhs):
    return hit[2]
  plan = None
  c = _weight_only_fit(lhs, rhs, dimension_numbers)
  if c is not None:
    b, b_is4 = c.rhs_values(rhs)
    sb, gb = c.rhs_scale(rhs)
    zp = _rhs_zero_point_i8(c, rhs)[0] if rhs.zero_point is not None else None
    plan = (b, numerics.qtype_tag(_qtype_of(rhs)), sb, _lib.float_tag(sb.dtype), zp, c.N, c.K, c.K // gb,
            fused_wq_min_rows(c.N, b_is4, c.K, c.K // gb))
  _DECODE_PLANS[key] = (weakref.ref(rhs, lambda _, k=key: _DECODE_PLANS.pop(k, None)),
                        _weight_signature(rhs), plan)
  return plan


def _decode_dot(lhs, rhs, dimension_numbers, preferred_element_type):
  """The decode kernel on a 2-D bf16 activation and a 2-D weight with a kept plan; None when the call is not of that
  kind (the general code below then decides)."""
  (lca, rca), _ = dimension_numbers
  if not (type(lhs) is torch.Tensor and lhs.ndim == 2 and lhs.dtype == torch.bfloat16 and isinstance(rhs, QArray)
          and len(lca) == 1 and lca[0] == 1 and rca[0] == 0 and lhs.shape[0] <= WEIGHT_ONLY_MAX_ROWS):
    return None
  plan = _decode_plan(lhs, rhs, dimension_numbers)
  if plan is None:
    return None
  b, b_tag, sb, sb_tag, zp, n, k, group, fused_min = plan
  m = lhs.shape[0]
  if lhs.shape[1] != k or len(rhs.shape) != 2 or m > fused_min:
    return None
  lhs = _aligned_rows(lhs)
  if not _decode_kernel_limits_ok(lhs.stride(0), b.stride(0), n, k, group, b_tag == _lib.INT4, sb.element_size()):
    return None
  res_t = preferred_element_type or torch.promote_types(lhs.dtype, sb.dtype)
  out = torch.empty(m, n, dtype=res_t, device=lhs.device)
  if zp is not None:
    _lib.call('qwix_hip_gemv_wq_zp', lhs.data_ptr(), lhs.stride(0), b.data_ptr(), b.stride(0), b_tag, m, n, k, group,
              sb.data_ptr(), sb_tag, zp.data_ptr(), out.data_ptr(), _lib.float_tag(res_t), n, _lib.stream_of(lhs))
  else:
    _lib.call('qwix_hip_gemv_wq', lhs.data_ptr(), lhs.stride(0), b.data_ptr(), b.stride(0), b_tag, m, n, k, group,
              sb.data_ptr(), sb_tag, out.data_ptr(), _lib.float_tag(res_t), n, _lib.stream_of(lhs))
  return out


def _slow_dot_general(lhs, rhs, dimension_numbers, preferred_element_type=None, **kwargs) -> torch.Tensor:
  """Dequantize-first path (dot_general.py:264-275).  A bf16 activation against an int4/int8 weight runs in one
  fused kernel (dequantize in registers, bf16 MFMA) when `_weight_only_fit` says the kernel takes it; every
  other combination is dequantized by the HIP dequantize kernel and contracted by the float GEMM.  Which of
  the two runs is decided here from the operands alone; a kernel that refuses its arguments raises."""
  del kwargs
  if len(dimension_numbers[1][0]) or len(dimension_numbers[1][1]):
    return _over_batch(_slow_dot_general, lhs, rhs, dimension_numbers, preferred_element_type=preferred_element_type)
  out = _decode_dot(lhs, rhs, dimension_numbers, preferred_element_type)
  if out is not None:
    return out
  c = _weight_only_fit(lhs, rhs, dimension_numbers)
  if c is not None and (fused_wq_min_rows(c.N, isinstance(rhs.qvalue, Int4Tensor), c.K, c.K // rhs.scale.shape[c.rca[-1]])
                        < c.M <= WEIGHT_ONLY_MAX_ROWS):
    # one row tile of the dequantizing tile GEMM beats the decode kernel from here on
    out = _dequantize_then_bf16_gemm(lhs, rhs, dimension_numbers, preferred_element_type, fused_only=True)
    if out is not None:
      return out
  if c is not None and c.M <= WEIGHT_ONLY_MAX_ROWS and _decode_fits_limits(c, rhs):
    sb, gb = c.rhs_scale(rhs)
    x = c.lhs_values(lhs)
    b, b_is4 = c.rhs_values(rhs)
    res_t = preferred_element_type or torch.promote_types(lhs.dtype, rhs.scale.dtype)
    out = torch.empty(c.M, c.N, dtype=res_t, device=x.device)
    if rhs.zero_point is not None:  # asymmetric weights: (q - zp) * scale, the zero point per group and column
      zp, _ = _rhs_zero_point_i8(c, rhs)
      _lib.call('qwix_hip_gemv_wq_zp', x.data_ptr(), x.stride(0), b.data_ptr(), b.stride(0),
                numerics.qtype_tag(_qtype_of(rhs)), c.M, c.N, c.K, c.K // gb, sb.data_ptr(), _lib.float_tag(sb.dtype),
                zp.data_ptr(), out.data_ptr(), _lib.float_tag(res_t), c.N, _lib.stream_of(x))
      return out.reshape(c.out_shape)
    _lib.call('qwix_hip_gemv_wq', x.data_ptr(), x.stride(0), b.data_ptr(), b.stride(0),
              numerics.qtype_tag(_qtype_of(rhs)), c.M, c.N, c.K, c.K // gb, sb.data_ptr(), _lib.float_tag(sb.dtype),
              out.data_ptr(), _lib.float_tag(res_t), c.N, _lib.stream_of(x))
    return out.reshape(c.out_shape)
  out = _dequantize_then_bf16_gemm(lhs, rhs, dimension_numbers, preferred_element_type)
  if out is not None:
    return out
  if isinstance(lhs, QArray):
    lhs = qarray.dequantize(lhs)
  if isinstance(rhs, QArray):
    rhs = qarray.dequantize(rhs)
  res_t = preferred_element_type or torch.promote_types(lhs.dtype, rhs.dtype)
  return float_dot_general(lhs, rhs, dimension_numbers, res_t)


def _decode_fits_limits(c, rhs: QArray) -> bool:
  """`_decode_kernel_limits_ok` from the shapes alone (K-contiguous weight rows, contiguous activation rows)."""
  int4 = isinstance(rhs.qvalue, Int4Tensor)
  gb = rhs.scale.shape[c.rca[-1]]
  return _decode_kernel_limits_ok(c.K, c.K // 2 if int4 else c.K, c.N, c.K, c.K // gb, int4, rhs.scale.element_size())


# The tile GEMM that dequantizes the weight inside its workgroups converts it once per row tile of 256; above these
# sizes dequantizing it once into memory and running the dense bf16 GEMM is faster.  int4 (K 4096, N 14336, per
# call): 512 rows 79 us against 114, 1024 rows 154 against 156, 2048 rows 293 against 260.  int8: one round of
# 256 x 128 tiles (N 14336: 512 rows 82 against 118, 1024 rows 170 against 159; N 4096: 2048 rows 90 against 94).
_FUSED_WQ_MAX_ROWS = 1024


def _fused_wq_takes(m: int, n: int, int4: bool) -> bool:
  if int4:
    return m <= _FUSED_WQ_MAX_ROWS
  return -(-m // 256) * -(-n // 128) <= _FUSED_W8_MAX_TILES


_FUSED_W8_MAX_TILES = 256


def fused_wq_min_rows(n: int, int4: bool = True, k: int = 0, group: int = 0) -> int:
  """Rows above which the dequantizing tile GEMM beats the decode kernel (`qwix_hip_gemv_wq`).  The time of one row
  tile does not depend on the rows (K 4096, up to 128 rows, tiles of 128 x 64: int4 29 / 26 us at N 14336 / 4096, int8
  29 / 25 us; 129-256 rows, tiles of 256 x 64: 45 us); the decode kernel's grows with them in steps of 16 rows and
  falls with N (K 4096, int4, 64 / 80 / 96 / 128 rows: N 14336 26 / 35 / 38 / 48 us, N 4096 21 / 23 / 28 / 35 us; int8,
  32 / 48 / 64 / 80 rows: N 14336 23 / 31 / 35 / 46 us, N 4096 12 / 17 / 21 / 26 us).
  Where the tile GEMM cuts K into ranges (given `k` and `group`: few tiles, `qwix_hip_gemm_bf16_wq_ws`) it wins earlier.
  Weights from HBM, decode kernel at 32 / 48 / 64 rows against the tile GEMM's one time up to 128 rows: int4 K 4096,
  N 4096 12 / 15 / 21 against 15 us; K 8192, N 8192 23 / 29 / 40 against 33; K 14336, N 4096 34 / 45 / 64 against 31;
  int8 13 / 17 / 21 against 15; 25 / 40 / 48 against 34; 35 / 55 / 67 against 32."""
  if k and group and _lib.load().qwix_hip_gemm_bf16_wq_workspace_bytes(64, n, k, group):
    return 48 if int4 else 32
  if int4:
    return 64 if n >= 12288 else 80
  return 32 if n >= 12288 else 64


def _dequantize_then_bf16_gemm(lhs, rhs, dimension_numbers, preferred_element_type, fused_only=False):
  """The dequantize-first path on this library's own kernels, for a bf16 activation against a quantized weight
  of any of the three qtypes, with or without zero point: the weight is dequantized into a K-contiguous bf16
  array (qwix_hip_dequantize_rm, the reference's D(D(q - zp) * scale) in the scale dtype; an f32 result rounded
  once more to bf16) and contracted by the bf16 MFMA GEMM with f32 accumulation (qwix_hip_gemm_bf16).  Returns
  None when the operands are not of that kind (then: HIP dequantize + the float GEMM of the vendor library).
  int4 / int8 weights skip the dequantized copy while `_fused_wq_takes` (qwix_hip_gemm_bf16_wq);
  with `fused_only` nothing else is run."""
  if not (_is_float_array(lhs) and lhs.dtype == torch.bfloat16 and isinstance(rhs, QArray)):
    return None
  if _qtype_of(rhs) not in (numerics.INT4, numerics.INT8, numerics.E4M3):
    return None
  c = _Canon(lhs, rhs, dimension_numbers)
  if any(rhs.scale.shape[a] != 1 for a in c.rca[:-1]) or c.K % 64:
    return None
  gb = rhs.scale.shape[c.rca[-1]]
  if (gb > 1 and len(c.rca) > 1) or (c.K // gb) % 8 or rhs.scale.dtype not in (torch.bfloat16, torch.float32):
    return None
  if isinstance(rhs.qvalue, Int4Tensor):
    order = c.rfree + c.rca
    packed = (rhs.qvalue.permute(*order).packed_axis, rhs.qvalue.permute(*(c.rca + c.rfree)).packed_axis)
    if len(order) - 1 not in packed:
      return None
  if not _bf16_gemm_limits_ok(c.M, c.K, c.N, 2 * c.K):  # beyond the kernels' 31-bit offsets: HIP dequantize + float GEMM
    return None
  x = c.lhs_values(lhs)
  b, b_is4 = c.rhs_values(rhs)
  sb, _ = c.rhs_scale(rhs)
  zp = None
  if rhs.zero_point is not None:
    zp, gz = _rhs_zero_point_i8(c, rhs)
    if gz != gb:
      return None
  dev, st = x.device, _lib.stream_of(x)
  res_t = preferred_element_type or torch.promote_types(lhs.dtype, rhs.scale.dtype)
  if res_t not in (torch.bfloat16, torch.float32):
    return None
  if (_fused_wq_takes(c.M, c.N, b_is4)
      and c.K % 256 == 0 and (c.K // gb) % 64 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0):
    # int4 / int8 with or without zero points, e4m3: dequantized inside the GEMM's workgroups, slab by slab (the same
    # bf16 weights, the same products in the same order, no dequantized copy of the weight in memory)
    out = torch.empty(c.M, c.N, dtype=res_t, device=dev)
    # few tiles: K in ranges over more workgroups, f32 partials in a workspace (0 bytes = not split)
    nws = int(_lib.load().qwix_hip_gemm_bf16_wq_workspace_bytes(c.M, c.N, c.K, c.K // gb))
    ws = torch.empty(nws, dtype=torch.uint8, device=dev) if nws else None
    _lib.call('qwix_hip_gemm_bf16_wq_ws', x.data_ptr(), x.stride(0), b.data_ptr(), b.stride(0),
              numerics.qtype_tag(_qtype_of(rhs)), c.M, c.N, c.K, c.K // gb, sb.data_ptr(), _lib.float_tag(sb.dtype),
              _lib.ptr(zp), out.data_ptr(), _lib.float_tag(res_t), c.N, _lib.ptr(ws), nws, st)
    return out.reshape(c.out_shape)
  if fused_only:
    return None
  w = torch.empty(c.N, c.K, dtype=torch.bfloat16, device=dev)
  _lib.call('qwix_hip_dequantize_rm', b.data_ptr(), numerics.qtype_tag(_qtype_of(rhs)), 1, c.K, c.N, c.K // gb,
            sb.data_ptr(), _lib.ptr(zp), _lib.float_tag(sb.dtype), w.data_ptr(), _lib.BF16, st)
  out = torch.empty(c.M, c.N, dtype=res_t, device=dev)
  _lib.call('qwix_hip_gemm_bf16', x.data_ptr(), x.stride(0), w.data_ptr(), c.K, c.M, c.N, c.K, out.data_ptr(),
            _lib.float_tag(res_t), c.N, st)
  return out.reshape(c.out_shape)


def float_dot_general(lhs: torch.Tensor, rhs: torch.Tensor, dimension_numbers, preferred_element_type=None) -> torch.Tensor:
  """lax.dot_general on two float tensors: contracting AND batch axes honoured, result laid out as
  (batch..., lhs free..., rhs free...).  The float GEMM itself is the vendor library's (torch.einsum)."""
  (lca, rca), (lba, rba) = dimension_numbers
  lca, rca, lba, rba = ([int(a) for a in x] for x in (lca, rca, lba, rba))
  if len(lca) != len(rca) or len(lba) != len(rba):
    raise TypeError(f'dot_general: contracting / batch axes differ in number: {dimension_numbers}')
  letters = iter('abcdefghijklmnopqrstuvwxyzABCDEFGHIJKLMNOPQRSTUVWXYZ')
  lsub = [next(letters) for _ in range(lhs.ndim)]
  rsub = [None] * rhs.ndim
  for l, r in list(zip(lca, rca)) + list(zip(lba, rba)):
    if lhs.shape[l] != rhs.shape[r]:
      raise TypeError(f'dot_general: sizes of {tuple(lhs.shape)} axis {l} and {tuple(rhs.shape)} axis {r} differ')
    rsub[r] = lsub[l]
  rsub = [c if c is not None else next(letters) for c in rsub]
  out = ([lsub[a] for a in lba] + [lsub[a] for a in range(lhs.ndim) if a not in lca and a not in lba] +
         [rsub[a] for a in range(rhs.ndim) if a not in rca and a not in rba])
  ct = torch.promote_types(lhs.dtype, rhs.dtype)
  if preferred_element_type == torch.float32:
    ct = torch.float32  # bf16 operands with an f32 result: f32 sums delivered as they are, not rounded to bf16 on the way
  res = torch.einsum(f"{''.join(lsub)},{''.join(rsub)}->{''.join(out)}", lhs.to(ct), rhs.to(ct))
  return res if preferred_element_type is None else res.to(preferred_element_type)


def _degenerate(lhs, rhs, dimension_numbers, preferred_element_type):
  """The result when an operand has no elements (nothing to launch): an empty array, or zeros when only
  the contracted axes are empty -- what lax.dot_general returns for such shapes.  None otherwise."""
  ls, rs = tuple(lhs.shape), tuple(rhs.shape)
  if math.prod(ls) and math.prod(rs):
    return None
  (lc, rc), (lb, rb) = dimension_numbers
  if [ls[a] for a in lc] != [rs[a] for a in rc] or [ls[a] for a in lb] != [rs[a] for a in rb]:
    raise TypeError(f'dot_general: contracting / batch sizes of {ls} and {rs} differ for {dimension_numbers}')
  out = ([ls[a] for a in lb] + [d for a, d in enumerate(ls) if a not in lc and a not in lb] +
         [d for a, d in enumerate(rs) if a not in rc and a not in rb])
  _, res_t = qarray.get_accumulator_and_result_type(lhs, rhs, preferred_element_type=preferred_element_type)
  dev = (lhs.scale if isinstance(lhs, qarray.QArray) else lhs).device
  return torch.zeros(out, dtype=res_t, device=dev)


def dot_general(lhs: MaybeQ, rhs: MaybeQ, dimension_numbers: DotDimensionNumbers, precision=None,
                preferred_element_type=None, **kwargs) -> torch.Tensor:
  """Drop-in for lax.dot_general that accepts QArray operands.

  Takes the dequantize-first path iff an operand is a raw float array, a qtype cannot be scaled
  on output, or a contracting axis is tiled finer than 128; otherwise contracts the quantized
  values directly.  `precision` and extra keywords (e.g. out_sharding) are accepted and ignored.
  """
  del precision
  empty = _degenerate(lhs, rhs, dimension_numbers, preferred_element_type)
  if empty is not None:
    return empty
  fn = _fast_dot_general if _use_fast_path(lhs, rhs, dimension_numbers) else _slow_dot_general
  try:
    return fn(lhs, rhs, dimension_numbers, preferred_element_type=preferred_element_type, **kwargs)
  except qarray.Int4LayoutError:
    # packed int4 values that no kernel reads where they lie (pairs along a batch axis, or along an axis that is
    # neither the last contracting one nor the last free one): the same integers as int8, one byte each
    wl, wr = _widen_int4(lhs), _widen_int4(rhs)
    if wl is lhs and wr is rhs:
      raise
    return fn(wl, wr, dimension_numbers, preferred_element_type=preferred_element_type, **kwargs)


def _widen_int4(x):
  if isinstance(x, QArray) and isinstance(x.qvalue, Int4Tensor):
    return QArray(x.qvalue.unpack().contiguous(), x.scale, x.zero_point, numerics.INT8)
  return x


MaybeQ = Any
