"""Quantized einsum: string -> dimension numbers -> the HIP dot_general (host glue).

Mirror of qwix/_src/core/einsum.py: `get_how_to_quantize` (:27-81) and `einsum` (:106-188) for
the binary case; the contraction itself is `_qwix_dot_general` (default: the MFMA-backed
qwix_amd dot_general).  N-ary einsums are contracted pairwise left to right.
"""
from __future__ import annotations

from typing import Any, Mapping

import torch

from qwix_amd.core import dot_general as _dg
from qwix_amd.core import einsum_info
from qwix_amd.core import qarray


def get_how_to_quantize(*, einsum_str: str, ndims: tuple[int, int], for_lhs: bool,
                        tile_size: Mapping[int, int | float] | int | float | None, **kwargs: Any) -> qarray.HowToQuantize:
  """Channelwise for every non-contracted subscript; tiles on the last contracted axis if tile_size."""
  info = einsum_info.EinsumInfo.parse(einsum_str, ndims=ndims)
  subs = info.lhs if for_lhs else info.rhs
  channelwise, last = [], None
  for axis, ch in enumerate(subs):
    if ch in info.contract_chars:
      last = axis
    else:
      channelwise.append(axis)
  tiled: dict = {}
  if isinstance(tile_size, Mapping):
    tiled = dict(tile_size)
    channelwise = [a for a in channelwise if a not in tiled]
  elif tile_size and last is not None:
    tiled[last] = tile_size
  return qarray.HowToQuantize(channelwise_axes=channelwise, tiled_axes=tiled, **kwargs)


def _binary(lhs, rhs, einsum_str: str, dot_general_fn, preferred_element_type, **kwargs):
  info = einsum_info.EinsumInfo.parse(einsum_str, ndims=(len(lhs.shape), len(rhs.shape)))
  out = dot_general_fn(lhs, rhs, info.dimension_numbers, preferred_element_type=preferred_element_type, **kwargs)
  if info.output_perm is not None:
    out = out.permute(*info.output_perm)
  return out


def broadcast_operands(operands: list, subs_list: list[str]) -> list:
  """einsum_info.py:197-241: operands that share a subscript with different sizes are brought to the
  largest one when it is a multiple of the others (size 1 included), values repeated tile-wise."""
  size = {}
  for op, subs in zip(operands, subs_list):
    if len(subs) != len(op.shape):
      return operands  # ellipsis or rank mismatch: left to the parser
    for ch, d in zip(subs, op.shape):
      d = int(d)
      if ch not in size or size[ch] == 1 or (d > size[ch] and d % size[ch] == 0):
        size[ch] = d
  return [qarray.broadcast_to(op, tuple(size[c] for c in subs)) for op, subs in zip(operands, subs_list)]


def einsum(*args, _qwix_dot_general=_dg.dot_general, preferred_element_type=None, **kwargs) -> torch.Tensor:
  """Drop-in for jnp.einsum('subscripts', a, b) with QArray operands; the result dtype follows the
  dequantized dtypes unless preferred_element_type is given."""
  if not args or not isinstance(args[0], str):
    raise NotImplementedError('einsum expects the subscripts string first')
  einsum_str, operands = args[0], list(args[1:])
  _, res_t = qarray.get_accumulator_and_result_type(*operands, preferred_element_type=preferred_element_type)
  flat = einsum_str.replace(' ', '')
  if '.' not in flat:
    operands = broadcast_operands(operands, flat.split('->')[0].split(','))
  if len(operands) == 1:
    op = operands[0]
    return torch.einsum(einsum_str, qarray.dequantize(op) if isinstance(op, qarray.QArray) else op).to(res_t)
  if len(operands) != 2:
    return _nary(einsum_str, operands, _qwix_dot_general, res_t, **kwargs)
  return _binary(operands[0], operands[1], einsum_str, _qwix_dot_general, res_t, **kwargs)


def _nary(einsum_str: str, operands: list, dot_general_fn, res_t, **kwargs):
  """Three or more operands: contracted pairwise from the left (the reference follows the path chosen
  by opt_einsum, einsum.py:137-152; the result is the same up to the order of the float roundings).
  An intermediate keeps every subscript that a later operand or the output still needs."""
  s = einsum_str.replace(' ', '')
  if '->' not in s or '.' in s:
    raise NotImplementedError(f'einsum with {len(operands)} operands needs explicit subscripts: "{einsum_str}"')
  ins, out = s.split('->')
  terms = ins.split(',')
  if len(terms) != len(operands):
    raise ValueError(f'"{einsum_str}" names {len(terms)} operands, got {len(operands)}')
  cur, cur_sub = operands[0], terms[0]
  for k in range(1, len(operands)):
    later = set(out).union(*[set(t) for t in terms[k + 1:]])
    keep = [c for c in cur_sub if c in later] + [c for c in terms[k] if c in later and c not in cur_sub]
    last = k == len(operands) - 1
    sub = out if last else ''.join(keep)
    step = f'{cur_sub},{terms[k]}->{sub}'
    cur = _binary(cur, operands[k], step, dot_general_fn, res_t if last else None, **kwargs)
    cur_sub = sub
  return cur
