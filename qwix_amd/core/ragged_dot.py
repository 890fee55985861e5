"""Quantized ragged dot (mixture-of-experts matmul) on MI355X: host side of the ragged MFMA GEMM.

Mirror of qwix/_src/core/ragged_dot.py: `ragged_dot` (:316-353), the dispatcher
`ragged_dot_general` (:244-313: quantized path unless an operand has a zero point or is a raw float
array), `_fast_ragged_dot_general` (:123-226) and `_slow_ragged_dot_general` (:229-241).

lhs is (M, K), rhs is (G, K, N); the rows of lhs form G consecutive groups of `group_sizes` rows
and group g is multiplied with rhs[g].  `group_sizes` stays in device memory: the kernel reads it,
so the quantized path never synchronises with the host.  Rows past the last group come out as
zeros.  int4 expert weights and the dequantize-first path run the dense kernels of dot_general group by
group (these need the group boundaries on the host).  Other dimension numbers with the ragged axis as the only
free axis of the lhs and one group axis on the rhs (batch axes, several contracting axes, any axis order) run one
dense contraction per group (`_general_ragged`); a ragged contracting or batch axis raises.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Sequence

import torch

from qwix_amd import _lib
from qwix_amd.core import numerics
from qwix_amd.core import qarray
from qwix_amd.core import dot_general as _dot_general
from qwix_amd.core.dot_general import DotDimensionNumbers, _is_float_array, _qtype_of, _tag_of
from qwix_amd.core.qarray import Int4Tensor, QArray


@dataclasses.dataclass(frozen=True)
class RaggedDotDimensionNumbers:
  """Counterpart of jax.lax.RaggedDotDimensionNumbers."""

  dot_dimension_numbers: DotDimensionNumbers
  lhs_ragged_dimensions: Sequence[int]
  rhs_group_dimensions: Sequence[int]


_BASIC_RAGGED_DOT_DIMENSION_NUMBERS = RaggedDotDimensionNumbers(
    dot_dimension_numbers=(((1,), (1,)), ((), ())), lhs_ragged_dimensions=(0,), rhs_group_dimensions=(0,))


def _check_basic(dn: RaggedDotDimensionNumbers, lhs, rhs, group_sizes, group_offset):
  (lca, rca), (lba, rba) = dn.dot_dimension_numbers
  basic = (tuple(lca), tuple(rca), tuple(lba), tuple(rba), tuple(dn.lhs_ragged_dimensions),
           tuple(dn.rhs_group_dimensions)) == ((1,), (1,), (), (), (0,), (0,))
  if not basic:
    raise NotImplementedError(f'only the dimension numbers of ragged_dot are supported, got {dn}')
  if group_offset is not None:
    raise NotImplementedError('group_offset is not supported')
  if len(lhs.shape) != 2 or len(rhs.shape) != 3 or lhs.shape[1] != rhs.shape[1]:
    raise ValueError(f'ragged_dot expects lhs (M, K) and rhs (G, K, N), got {tuple(lhs.shape)} and {tuple(rhs.shape)}')
  if group_sizes.ndim != 1 or group_sizes.shape[0] != rhs.shape[0]:
    raise ValueError(f'group_sizes must have one entry per group: {tuple(group_sizes.shape)} vs G={rhs.shape[0]}')
  if group_sizes.dtype not in (torch.int32, torch.int64):
    raise TypeError(f'group_sizes must be an integer tensor, got {group_sizes.dtype}')


def _rhs_values(v: torch.Tensor) -> torch.Tensor:
  """(G, K, N) values as (G, N, K) K-contiguous storage: a view if the tensor already is a permuted
  view of such storage, else one transposing pass per group."""
  G, K, N = v.shape
  p = v.permute(0, 2, 1)
  if p.is_contiguous():
    return p
  if not v.is_contiguous():
    v = v.contiguous()
  dst = torch.empty(G, N, K, dtype=v.dtype, device=v.device)
  for g in range(G):
    _lib.call('qwix_hip_transpose_q', v[g].data_ptr(), _lib.INT8, K, N, dst[g].data_ptr(), _lib.stream_of(dst))
  return dst


_PLAIN_DOT = (((1,), (0,)), ((), ()))


def _rows(x, start: int, stop: int):
  """Rows start .. stop - 1 of an (M, K) operand: a view, scales and zero points sliced where they are per row."""
  if not isinstance(x, QArray):
    return x[start:stop]
  cut = lambda t: None if t is None else (t[start:stop] if t.shape[0] > 1 else t)
  q = x.qvalue
  if isinstance(q, Int4Tensor):
    if q.packed_axis == 0:
      raise NotImplementedError('int4 rows packed along the ragged axis cannot be sliced by groups')
    q = Int4Tensor(q.data[start:stop], (stop - start,) + tuple(q.shape[1:]), q.packed_axis)
  else:
    q = q[start:stop]
  return QArray(qvalue=q, scale=cut(x.scale), zero_point=cut(x.zero_point), qtype=x.qtype)


def _group(w, g: int):
  """Group g of a (G, K, N) operand as a (K, N) operand: a view."""
  if not isinstance(w, QArray):
    return w[g]
  pick = lambda t: None if t is None else t[g if t.shape[0] > 1 else 0]
  q = w.qvalue
  if isinstance(q, Int4Tensor):
    if q.packed_axis == 0:
      raise NotImplementedError('int4 weights packed along the group axis cannot be sliced by groups')
    q = Int4Tensor(q.data[g], tuple(q.shape[1:]), q.packed_axis - 1)
  else:
    q = q[g]
  return QArray(qvalue=q, scale=pick(w.scale), zero_point=pick(w.zero_point), qtype=w.qtype)


def _group_by_group(fn, lhs, rhs, group_sizes, res_t, **kwargs) -> torch.Tensor:
  """out[rows of group g] = fn(those rows of lhs, rhs[g]): one call of a dense kernel path per non-empty group.
  The group boundaries are needed on the host to slice the rows, so this waits for `group_sizes` to arrive there.
  Rows past the last group stay zero."""
  M, N = lhs.shape[0], rhs.shape[2]
  dev = (lhs.scale if isinstance(lhs, QArray) else lhs).device
  out = torch.zeros(M, N, dtype=res_t, device=dev)
  start = 0
  for g, size in enumerate(group_sizes.tolist()):
    stop = min(start + max(int(size), 0), M)
    if stop > start:
      out[start:stop] = fn(_rows(lhs, start, stop), _group(rhs, g), _PLAIN_DOT, preferred_element_type=res_t, **kwargs)
    start = stop
  return out


def _is_basic(dn: RaggedDotDimensionNumbers) -> bool:
  (lca, rca), (lba, rba) = dn.dot_dimension_numbers
  return (tuple(lca), tuple(rca), tuple(lba), tuple(rba), tuple(dn.lhs_ragged_dimensions),
          tuple(dn.rhs_group_dimensions)) == ((1,), (1,), (), (), (0,), (0,))


def _narrow(x, axis: int, start: int, stop: int):
  """Positions start .. stop - 1 along `axis` of a tensor or QArray: views; scales and zero points are cut where they
  have one entry per position and kept where they have one in all."""
  full = x.shape[axis]

  def cut(t):
    if t is None or t.shape[axis] == 1:
      return t
    if t.shape[axis] != full:
      raise NotImplementedError('scales tiled along the ragged axis cannot be sliced by groups')
    return t.narrow(axis, start, stop - start)

  def values(q):
    if isinstance(q, Int4Tensor):
      if q.packed_axis == axis:
        raise NotImplementedError('int4 values packed along the ragged axis cannot be sliced by groups')
      shape = tuple(stop - start if a == axis else d for a, d in enumerate(q.shape))
      return Int4Tensor(q.data.narrow(axis, start, stop - start), shape, q.packed_axis)
    return q.narrow(axis, start, stop - start)

  if isinstance(x, QArray):
    return QArray(qvalue=values(x.qvalue), scale=cut(x.scale), zero_point=cut(x.zero_point), qtype=x.qtype)
  return values(x)


def _select(w, axis: int, g: int):
  """Entry g along `axis` of a tensor or QArray, the axis removed: views."""
  full = w.shape[axis]

  def pick(t):
    if t is None:
      return None
    if t.shape[axis] not in (1, full):
      raise NotImplementedError('scales tiled along the group axis cannot be sliced by groups')
    return t.select(axis, g if t.shape[axis] > 1 else 0)

  def values(q):
    if isinstance(q, Int4Tensor):
      if q.packed_axis == axis:
        raise NotImplementedError('int4 weights packed along the group axis cannot be sliced by groups')
      shape = tuple(d for a, d in enumerate(q.shape) if a != axis)
      return Int4Tensor(q.data.select(axis, g), shape, q.packed_axis - (q.packed_axis > axis))
    return q.select(axis, g)

  if isinstance(w, QArray):
    return QArray(qvalue=values(w.qvalue), scale=pick(w.scale), zero_point=pick(w.zero_point), qtype=w.qtype)
  return values(w)


def _check_general(dn: RaggedDotDimensionNumbers, lhs, rhs, group_sizes, group_offset):
  """The ragged axis is a free axis of the lhs (its rows form the groups) and the rhs has one group axis: the first of
  the three modes of lax.ragged_dot_general, with batch axes, several contracting axes and any axis order.  Returns
  (ragged axis, group axis, dimension numbers of one group's dense contraction)."""
  (lca, rca), (lba, rba) = dn.dot_dimension_numbers
  lca, rca, lba, rba = ([int(a) for a in x] for x in (lca, rca, lba, rba))
  if group_offset is not None:
    raise NotImplementedError('group_offset is not supported')
  if len(dn.lhs_ragged_dimensions) != 1 or len(dn.rhs_group_dimensions) != 1:
    raise NotImplementedError(f'one ragged axis on the lhs and one group axis on the rhs are supported, got {dn}')
  ragged, group = int(dn.lhs_ragged_dimensions[0]), int(dn.rhs_group_dimensions[0])
  if ragged in lca or ragged in lba:
    raise NotImplementedError('a ragged contracting or batch axis (the modes without an rhs group axis) is not supported')
  if group in rca or group in rba:
    raise ValueError(f'the rhs group axis {group} cannot be a contracting or batch axis')
  lfree = [a for a in range(len(lhs.shape)) if a not in lca and a not in lba]
  if lfree != [ragged]:
    raise NotImplementedError(f'the ragged axis has to be the only free axis of the lhs, got free axes {lfree}')
  if len(lca) != len(rca) or len(lba) != len(rba):
    raise ValueError(f'contracting / batch axes differ in number: {dn}')
  for l, r in list(zip(lca, rca)) + list(zip(lba, rba)):
    if lhs.shape[l] != rhs.shape[r]:
      raise ValueError(f'sizes of lhs axis {l} and rhs axis {r} differ: {tuple(lhs.shape)} and {tuple(rhs.shape)}')
  if group_sizes.ndim != 1 or group_sizes.shape[0] != rhs.shape[group]:
    raise ValueError(f'group_sizes must have one entry per group: {tuple(group_sizes.shape)} vs G={rhs.shape[group]}')
  if group_sizes.dtype not in (torch.int32, torch.int64):
    raise TypeError(f'group_sizes must be an integer tensor, got {group_sizes.dtype}')
  drop = lambda a: a - (a > group)
  return ragged, group, ((tuple(lca), tuple(drop(a) for a in rca)), (tuple(lba), tuple(drop(a) for a in rba)))


def _general_ragged(fn, lhs, rhs, group_sizes, dimension_numbers, res_t, group_offset, **kwargs) -> torch.Tensor:
  """Dimension numbers other than ragged_dot's (ragged_dot.py:123-226 hands any to lax.ragged_dot_general): one dense
  contraction per non-empty group on views of the operands -- the rows of the group along the ragged axis against
  that group's slice of the rhs -- written to the group's rows of the result (batch axes, the ragged axis, the free
  axes of the rhs).  Per element the same arithmetic as the reference's: the group's accumulator scaled by the row's
  lhs scale, then by the group's rhs scale, tile partials summed last.  The group boundaries are needed on the host."""
  ragged, group, dn = _check_general(dimension_numbers, lhs, rhs, group_sizes, group_offset)
  (_, _), (lba, rba) = dn
  M = lhs.shape[ragged]
  rfree = [d for a, d in enumerate(rhs.shape) if a != group and (a - (a > group)) not in dn[0][1] and (a - (a > group)) not in rba]
  dev = (lhs.scale if isinstance(lhs, QArray) else lhs).device
  out = torch.zeros([lhs.shape[a] for a in lba] + [M] + rfree, dtype=res_t, device=dev)
  start = 0
  for g, size in enumerate(group_sizes.tolist()):
    stop = min(start + max(int(size), 0), M)
    if stop > start:
      part = fn(_narrow(lhs, ragged, start, stop), _select(rhs, group, g), dn, preferred_element_type=res_t, **kwargs)
      out.narrow(len(lba), start, stop - start).copy_(part)
    start = stop
  return out


def _fast_ragged_dot_general(lhs, rhs, group_sizes, dimension_numbers=_BASIC_RAGGED_DOT_DIMENSION_NUMBERS,
                             precision=None, preferred_element_type=None, group_offset=None) -> torch.Tensor:
  """Contract the quantized values group by group on the matrix cores, then scale:
  out = ((acc * lhs_scale) * rhs_scale[group of the row]), tile partials summed last."""
  del precision
  if not _is_basic(dimension_numbers):
    for x in (lhs, rhs):
      if isinstance(x, QArray) and x.zero_point is not None:
        raise NotImplementedError('zero-point operands take the dequantize-first ragged dot')
    _, res_t = qarray.get_accumulator_and_result_type(lhs, rhs, preferred_element_type=preferred_element_type)
    return _general_ragged(_dot_general._fast_dot_general, lhs, rhs, group_sizes, dimension_numbers, res_t, group_offset)
  _check_basic(dimension_numbers, lhs, rhs, group_sizes, group_offset)
  for x in (lhs, rhs):
    if isinstance(x, QArray) and x.zero_point is not None:
      raise NotImplementedError('zero-point operands take the dequantize-first ragged dot')
  if any(isinstance(x.qvalue if isinstance(x, QArray) else x, Int4Tensor) for x in (lhs, rhs)):
    # int4 values (int8 activations x int4 expert weights): the sub-channel MFMA GEMM of dot_general, group by
    # group; the ragged kernel itself reads int8 / e4m3 values only
    _, res_t = qarray.get_accumulator_and_result_type(lhs, rhs, preferred_element_type=preferred_element_type)
    return _group_by_group(_dot_general._fast_dot_general, lhs, rhs, group_sizes, res_t)
  lq, rq = _qtype_of(lhs), _qtype_of(rhs)
  if (lq, rq) == (numerics.INT8, numerics.INT8):
    qt = _lib.INT8
  elif (lq, rq) == (numerics.E4M3, numerics.E4M3):
    qt = _lib.E4M3
  else:
    raise NotImplementedError(f'no ragged MFMA kernel for {lq} x {rq} operands')
  lt = qarray.get_tiled_axes(lhs) if isinstance(lhs, QArray) else {}
  rt = qarray.get_tiled_axes(rhs) if isinstance(rhs, QArray) else {}
  if lt.get(1) and rt.get(1) and lt[1] != rt[1]:
    raise ValueError(f'Contracting axes must be tiled with the same tile size. lhs_tiled_axes={lt} rhs_tiled_axes={rt} {dimension_numbers=}')
  acc_t, res_t = qarray.get_accumulator_and_result_type(lhs, rhs, preferred_element_type=preferred_element_type)
  M, K = lhs.shape
  G, _, N = rhs.shape
  tile = lt.get(1) or rt.get(1) or K
  ntiles = K // tile
  a = lhs.qvalue if isinstance(lhs, QArray) else lhs
  a = a if a.is_contiguous() else a.contiguous()
  b = _rhs_values(rhs.qvalue if isinstance(rhs, QArray) else rhs)
  dev = a.device
  st = _lib.stream_of(a)
  gs = group_sizes.to(device=dev, dtype=torch.int32).contiguous()

  # scales in kernel order: sa (M, ntiles or 1), sb (G or 1, ntiles or 1, N)
  sa = sb = None
  if isinstance(lhs, QArray):
    sa = lhs.scale.expand(M, lhs.scale.shape[1]).contiguous()
  if isinstance(rhs, QArray):
    sb = rhs.scale
    if sb.shape[2] not in (1, N):
      sb = sb.repeat_interleave(N // sb.shape[2], dim=2)
    sb = sb.expand(sb.shape[0], sb.shape[1], N).contiguous()
  # dtype in which the scaled partials live: the accumulator's, promoted with each scale in turn
  cur_t = None if acc_t == torch.int32 else acc_t
  for s in (sa, sb):
    if s is not None:
      cur_t = s.dtype if cur_t is None else torch.promote_types(cur_t, s.dtype)
  cur_t = cur_t or torch.int32

  def launch(t: int, out: torch.Tensor):
    sa_t = None if sa is None else sa[:, min(t, sa.shape[1] - 1)].contiguous()
    sb_t = None if sb is None else sb[:, min(t, sb.shape[1] - 1), :].contiguous()
    _lib.call('qwix_hip_qgemm_ragged', a.data_ptr() + t * tile, a.stride(0), b.data_ptr() + t * tile, b.stride(1),
              b.stride(0), qt, M, N, tile, gs.data_ptr(), G, _lib.ptr(sa_t),
              0 if sa_t is None else _lib.float_tag(sa_t.dtype), _lib.ptr(sb_t),
              0 if sb_t is None else _lib.float_tag(sb_t.dtype), N if (sb_t is not None and sb_t.shape[0] > 1) else 0,
              _tag_of(acc_t) if acc_t != torch.int32 else 0, out.data_ptr(), _tag_of(out.dtype), N, st)

  if ntiles == 1:
    out = torch.empty(M, N, dtype=res_t, device=dev)
    launch(0, out)
    return out
  # Sub-channel scales along K: one launch per K tile, each partial scaled with its own scales; the
  # partials are summed in f32 in tile order and rounded once (ragged_dot.py:222-224).
  part = torch.empty(M, N, dtype=cur_t, device=dev)
  total = torch.zeros(M, N, dtype=torch.int32 if cur_t == torch.int32 else torch.float32, device=dev)
  for t in range(ntiles):
    launch(t, part)
    total += part
  return total.to(cur_t).to(res_t)


def _slow_ragged_dot_general(lhs, rhs, group_sizes, dimension_numbers=_BASIC_RAGGED_DOT_DIMENSION_NUMBERS,
                             precision=None, preferred_element_type=None, group_offset=None) -> torch.Tensor:
  """Dequantize first (ragged_dot.py:229-241), group by group on the dense dequantize-first path: a bf16
  activation against an expert's int4 / int8 / e4m3 weight runs on this library's weight-only kernels (the fused
  dequantize + bf16 MFMA kernel up to 256 rows, dequantize + the bf16 MFMA GEMM beyond), every other combination
  is dequantized by the HIP kernel and contracted by the float GEMM."""
  del precision
  basic = _is_basic(dimension_numbers)
  if basic:
    _check_basic(dimension_numbers, lhs, rhs, group_sizes, group_offset)
  else:
    _check_general(dimension_numbers, lhs, rhs, group_sizes, group_offset)
  if isinstance(lhs, QArray):
    lhs = qarray.dequantize(lhs)
  rhs_t = rhs.scale.dtype if isinstance(rhs, QArray) else rhs.dtype
  res_t = preferred_element_type or torch.promote_types(lhs.dtype, rhs_t)
  if not basic:
    return _general_ragged(_dot_general._slow_dot_general, lhs, rhs, group_sizes, dimension_numbers, res_t, group_offset)
  return _group_by_group(_dot_general._slow_dot_general, lhs, rhs, group_sizes, res_t)


def ragged_dot_general(lhs, rhs, group_sizes: torch.Tensor, dimension_numbers: RaggedDotDimensionNumbers,
                       precision=None, preferred_element_type=None, group_offset=None) -> torch.Tensor:
  """Drop-in for lax.ragged_dot_general that accepts QArray operands."""
  if math.prod(lhs.shape) == 0 or math.prod(rhs.shape) == 0:
    # nothing to launch: no rows or no columns give an empty result, an empty contraction gives zeros
    _, res_t = qarray.get_accumulator_and_result_type(lhs, rhs, preferred_element_type=preferred_element_type)
    dev = (lhs.scale if isinstance(lhs, QArray) else lhs).device
    if _is_basic(dimension_numbers):
      _check_basic(dimension_numbers, lhs, rhs, group_sizes, group_offset)
      return torch.zeros(lhs.shape[0], rhs.shape[2], dtype=res_t, device=dev)
    ragged, group, dn = _check_general(dimension_numbers, lhs, rhs, group_sizes, group_offset)
    rfree = [d for a, d in enumerate(rhs.shape)
             if a != group and (a - (a > group)) not in dn[0][1] and (a - (a > group)) not in dn[1][1]]
    return torch.zeros([lhs.shape[a] for a in dn[1][0]] + [lhs.shape[ragged]] + rfree, dtype=res_t, device=dev)
  use_fast_path = True
  for operand in (lhs, rhs):
    if isinstance(operand, QArray):
      if operand.zero_point is not None:
        use_fast_path = False
        break
    elif _is_float_array(operand):
      use_fast_path = False
      break
  fn = _fast_ragged_dot_general if use_fast_path else _slow_ragged_dot_general
  return fn(lhs, rhs, group_sizes, dimension_numbers, precision=precision,
            preferred_element_type=preferred_element_type, group_offset=group_offset)


def ragged_dot(lhs, rhs, group_sizes: torch.Tensor, precision=None, preferred_element_type=None,
               group_offset=None) -> torch.Tensor:
  """Drop-in for lax.ragged_dot: lhs (M, K) . rhs (G, K, N) with the rows of lhs in G groups."""
  return ragged_dot_general(lhs, rhs, group_sizes, _BASIC_RAGGED_DOT_DIMENSION_NUMBERS, precision=precision,
                            preferred_element_type=preferred_element_type, group_offset=group_offset)
