"""Host-side numerics tables: which dtypes can be quantized, and the value bounds per qtype.

Mirrors the parts of qwix/_src/core/numerics.py (:29-61 eligibility, :64-136 bounds) that the
int8 / int4 / float8_e4m3fn path uses.  The arithmetic itself (round, clip, cast) runs in the HIP
kernels; nothing here touches device memory.
"""
from __future__ import annotations

import torch

from qwix_amd import _lib

INT8 = 'int8'
INT4 = 'int4'
E4M3 = 'float8_e4m3fn'

_QUANTIZABLE = (torch.bfloat16, torch.float32)
_ALIASES = {
    'int8': INT8, 'torch.int8': INT8, 'jnp.int8': INT8,
    'int4': INT4, 'torch.int4': INT4, 'jnp.int4': INT4,
    'float8_e4m3fn': E4M3, 'torch.float8_e4m3fn': E4M3, 'jnp.float8_e4m3fn': E4M3, 'e4m3': E4M3,
}


def canonical_qtype(qtype) -> str:
  """Normalises a qtype given as a string or a torch dtype to 'int8' / 'int4' / 'float8_e4m3fn'."""
  key = str(qtype)
  if key not in _ALIASES:
    raise ValueError(
        f'qtype {qtype!r} is not served by the HIP path (int8, int4, float8_e4m3fn).'
    )
  return _ALIASES[key]


def qtype_tag(qtype) -> int:
  return {INT8: _lib.INT8, INT4: _lib.INT4, E4M3: _lib.E4M3}[canonical_qtype(qtype)]


def storage_dtype(qtype) -> torch.dtype:
  """The torch dtype holding the quantized values (int4 is packed into uint8 bytes)."""
  return {INT8: torch.int8, INT4: torch.uint8, E4M3: torch.float8_e4m3fn}[canonical_qtype(qtype)]


def should_quantize(dtype) -> bool:
  """Whether arrays of this dtype are eligible for quantization (numerics.py:29-41).

  The reference also lists float16/float64; the HIP kernels take bf16 and f32.
  """
  return dtype in _QUANTIZABLE


def can_dequant_on_output(qtype) -> bool:
  """numerics.py:44-61: uniform qtypes can be scaled after the integer/fp8 contraction."""
  return str(qtype) != 'nf4'


def get_asymmetric_bound(qtype) -> tuple[float, float]:
  """(qmin, qmax) of the integer grid used by asymmetric quantization (numerics.py:64-92)."""
  try:
    q = canonical_qtype(qtype)
  except ValueError as e:
    raise ValueError(f"{qtype} doesn't support asymmetric quantization.") from e
  if q == INT8:
    return (-128.0, 127.0)
  if q == INT4:
    return (-8.0, 7.0)
  raise ValueError(f"{qtype} doesn't support asymmetric quantization.")


def get_symmetric_bound(qtype) -> float:
  """Largest magnitude before rounding: qmax + 0.5 for ints, finfo.max for fp8 (numerics.py:95-136)."""
  return {INT8: 127.5, INT4: 7.5, E4M3: 448.0}[canonical_qtype(qtype)]
