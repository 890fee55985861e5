"""Quantized jnp.dot (mirror of qwix/_src/core/dot.py:24-71): contracts the last axis of `a` with
the second-to-last (or only) axis of `b` through the injected dot_general."""
from __future__ import annotations

from qwix_amd.core import dot_general as _dg


def dot(a, b, precision=None, preferred_element_type=None, out_sharding=None, *, _qwix_dot_general=_dg.dot_general):
  if a.ndim == 0 or b.ndim == 0:
    contract = ((), ())
  elif b.ndim == 1:
    contract = ((a.ndim - 1,), (0,))
  else:
    contract = ((a.ndim - 1,), (b.ndim - 2,))
  return _qwix_dot_general(a, b, dimension_numbers=(contract, ((), ())), precision=precision,
                           preferred_element_type=preferred_element_type, out_sharding=out_sharding)
