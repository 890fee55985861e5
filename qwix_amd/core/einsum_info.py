"""Binary einsum -> dot_general bookkeeping (host only).

Mirror of qwix/_src/core/einsum_info.py:26-174: splits 'lhs,rhs->out' into batch characters
(in all three), contraction characters (in both inputs, not in the output), the dot_general
dimension numbers, and the permutation that brings dot_general's (batch, lhs free, rhs free)
result into the requested output order.  Ellipsis and implicit outputs are expanded here when
`ndims` is given (the reference delegates that to opt_einsum's parser).
"""
from __future__ import annotations

import dataclasses
import re
import string


def expand_einsum(einsum_str: str, ndims: tuple[int, int]) -> str:
  """Rewrites '...' and a missing '->out' into explicit subscripts, the way numpy/opt_einsum do."""
  s = einsum_str.replace(' ', '')
  ins, arrow, out = s.partition('->')
  terms = ins.split(',')
  if len(terms) != 2:
    raise NotImplementedError(f'Unsupported einsum string: "{einsum_str}" (binary einsums only).')
  used = set(c for c in s if c.isalpha())
  spare = [c for c in string.ascii_lowercase + string.ascii_uppercase if c not in used]
  ell_len = 0
  for t, nd in zip(terms, ndims):
    if '...' in t:
      ell_len = max(ell_len, nd - (len(t) - 3))
  ell = ''.join(spare[:ell_len])
  new_terms = []
  for t, nd in zip(terms, ndims):
    if '...' in t:
      k = nd - (len(t) - 3)
      t = t.replace('...', ell[ell_len - k:] if k else '')
    new_terms.append(t)
  if arrow:
    out = out.replace('...', ell)
  else:
    counts = {}
    for t in new_terms:
      for c in t:
        counts[c] = counts.get(c, 0) + 1
    out = ell + ''.join(sorted(c for c, n in counts.items() if n == 1 and c not in ell))
  return f'{new_terms[0]},{new_terms[1]}->{out}'


@dataclasses.dataclass(slots=True)
class EinsumInfo:
  """lhs / rhs / out subscripts of a binary einsum, e.g. 'abc,bcd->acd' (a free, b contract, c batch)."""

  lhs: str
  rhs: str
  out: str

  @classmethod
  def parse(cls, einsum_str: str, ndims: tuple[int, int] | None = None) -> 'EinsumInfo':
    if ndims is not None:
      einsum_str = expand_einsum(einsum_str, ndims)
    s = einsum_str.replace(' ', '')
    if not re.match(r'^[a-zA-Z]*,[a-zA-Z]*->[a-zA-Z]*$', s):
      raise NotImplementedError(
          f'Unsupported einsum string: "{einsum_str}". EinsumInfo only supports binary einsums with explicit '
          'output subscripts (e.g., "abc,bcd->acd").'
      )
    ins, out = s.split('->')
    lhs, rhs = ins.split(',')
    for name, subs in (('lhs', lhs), ('rhs', rhs), ('out', out)):
      if len(set(subs)) != len(subs):
        raise NotImplementedError(f'Repeated indices in {name} ("{subs}") are not supported. Einsum string: "{s}".')
    return cls(lhs, rhs, out)

  @property
  def batch_chars(self) -> list[str]:
    return sorted(set(self.lhs) & set(self.rhs) & set(self.out))

  @property
  def contract_chars(self) -> list[str]:
    return sorted((set(self.lhs) & set(self.rhs)) - set(self.out))

  @property
  def dimension_numbers(self):
    li = {c: i for i, c in enumerate(self.lhs)}
    ri = {c: i for i, c in enumerate(self.rhs)}
    cc, bc = self.contract_chars, self.batch_chars
    return ((tuple(li[c] for c in cc), tuple(ri[c] for c in cc)), (tuple(li[c] for c in bc), tuple(ri[c] for c in bc)))

  @property
  def output_perm(self) -> tuple[int, ...] | None:
    bc = self.batch_chars
    natural = bc + [c for c in self.lhs if c in self.out and c not in bc] + [c for c in self.rhs if c in self.out and c not in bc]
    pos = {c: i for i, c in enumerate(natural)}
    perm = tuple(pos[c] for c in self.out)
    return None if perm == tuple(range(len(perm))) else perm
