"""Randomised Walsh-Hadamard rotation of the two operands of a contraction, on MI355X.

Host-side mirror of qwix/contrib/hadamard_rot.py (`hadamard_rotate_inputs` :133-190): the
activation is multiplied by had = H * row_signs[:, None] * col_signs[None, :] along its reduction
axis (unnormalised), the weight by had^T / n, so that act' @ weight' == act @ weight.  The
reference builds the dense n x n matrix and calls einsum; here an in-LDS fast Walsh-Hadamard
transform does the same sums in n log n adds (qwix_hip_fwht), and `rotate_and_quantize` fuses the
quantization behind it (qwix_hip_fwht_quantize) so the rotated tensors never reach HBM.

Sign vectors: the reference draws them with jax.random from a PRNG key.  Here `key` is a
torch.Generator or an int seed (or None when no flips are requested); the vectors are drawn from
it on the host and uploaded, and are also returned so that callers can keep them.
"""
from __future__ import annotations

import math

import torch

from qwix_amd import _lib
from qwix_amd.core import numerics
from qwix_amd.core import qarray


def _generator(key) -> torch.Generator | None:
  if key is None or isinstance(key, torch.Generator):
    return key
  g = torch.Generator(device='cpu')
  g.manual_seed(int(key))
  return g


def random_signs(key, n: int, dtype: torch.dtype, device) -> torch.Tensor:
  """A +-1 vector of length n drawn from `key` (torch.Generator or int seed)."""
  g = _generator(key)
  if g is None:
    raise ValueError('Key must be provided if row_sign_flip or col_sign_flip is True.')
  s = torch.randint(0, 2, (n,), generator=g, dtype=torch.int32) * 2 - 1
  return s.to(dtype).to(device)


def _check_dims(act, weight, lhs_reduction_dim, rhs_reduction_dim) -> int:
  if not isinstance(lhs_reduction_dim, int):
    raise ValueError(f'Expected lhs_reduction_dim to be an integer, but got {lhs_reduction_dim}')
  if not isinstance(rhs_reduction_dim, int):
    raise ValueError(f'Expected rhs_reduction_dim to be an integer, but got {rhs_reduction_dim}')
  n = act.shape[lhs_reduction_dim]
  if n != weight.shape[rhs_reduction_dim]:
    raise ValueError(f'Expected reduction dimension sizes to be the same, but got {n} and {weight.shape[rhs_reduction_dim]}')
  if 2 ** int(math.log2(n)) != n:
    raise ValueError(f'Expected reduction dimension size to be a power of 2, but got {n}')
  return n


def _rows_view(x: torch.Tensor, dim: int) -> torch.Tensor:
  """x with `dim` moved last, contiguous: the FWHT kernels transform along contiguous rows."""
  y = x.movedim(dim, -1)
  return y if y.is_contiguous() else y.contiguous()


def fwht(x: torch.Tensor, dim: int, pre_sign=None, post_sign=None, out_scale: float = 1.0) -> torch.Tensor:
  """((x * pre_sign) H_n) * post_sign * out_scale along `dim`; returns a view with x's logical shape."""
  rows = _rows_view(x, dim)
  n = rows.shape[-1]
  y = torch.empty_like(rows)
  _lib.call('qwix_hip_fwht', rows.data_ptr(), _lib.float_tag(x.dtype), rows.numel() // n, n, _lib.ptr(pre_sign),
            _lib.ptr(post_sign), float(out_scale), y.data_ptr(), _lib.stream_of(rows))
  return y.movedim(-1, dim)


def hadamard_rotate_inputs(act: torch.Tensor, weight: torch.Tensor, key, *, row_sign_flip: bool, col_sign_flip: bool,
                           lhs_reduction_dim: int, rhs_reduction_dim: int):
  """Returns (rotated act, rotated weight, key).  The rotated weight is a K-contiguous view."""
  n = _check_dims(act, weight, lhs_reduction_dim, rhs_reduction_dim)
  g = _generator(key)
  rs = random_signs(g, n, act.dtype, act.device) if row_sign_flip else None
  cs = random_signs(g, n, act.dtype, act.device) if col_sign_flip else None
  act_r = fwht(act, lhs_reduction_dim, rs, cs, 1.0)
  rs_w = None if rs is None else rs.to(weight.dtype)
  cs_w = None if cs is None else cs.to(weight.dtype)
  w_r = fwht(weight, rhs_reduction_dim, rs_w, cs_w, 1.0 / n)
  return act_r, w_r, g


def rotate_and_quantize(x: torch.Tensor, dim: int, how: qarray.HowToQuantize, pre_sign=None, post_sign=None,
                        out_scale: float = 1.0) -> qarray.QArray:
  """quantize(fwht(x, dim, ...), how) in one kernel, for `how` that reduces exactly along `dim`
  (per-row: every other axis channelwise; or tiles of a power-of-two size along `dim`)."""
  dim = dim % x.ndim
  shape = tuple(x.shape)
  n = shape[dim]
  sshape = qarray.get_scale_shape(shape, how)
  tiles = tuple(d // s for d, s in zip(shape, sshape))
  if any(t != 1 for a, t in enumerate(tiles) if a != dim and shape[a] != 1):
    raise NotImplementedError('rotate_and_quantize needs every axis other than `dim` to be channelwise')
  if how.calibration_method.lower() != 'absmax':
    raise NotImplementedError('rotate_and_quantize supports plain absmax calibration')
  tile = tiles[dim]
  q = numerics.canonical_qtype(how.qtype)
  if n < 8 or (tile != n and tile > 512) or tile & (tile - 1):
    # outside the fused kernel's shapes (rows of fewer than 8, tiles of more than 512 short of the row): two launches
    return qarray.quantize(fwht(x, dim, pre_sign, post_sign, out_scale).contiguous(), how)
  rows = _rows_view(x, dim)
  nrows = rows.numel() // n
  lead = tuple(rows.shape[:-1])
  if q == numerics.INT4:
    data = torch.empty(*lead, n // 2, dtype=torch.uint8, device=x.device)
  else:
    data = torch.empty(*lead, n, dtype=numerics.storage_dtype(q), device=x.device)
  scale = torch.empty(*lead, n // tile, dtype=x.dtype, device=x.device)
  _lib.call('qwix_hip_fwht_quantize', rows.data_ptr(), _lib.float_tag(x.dtype), nrows, n, _lib.ptr(pre_sign),
            _lib.ptr(post_sign), float(out_scale), tile, numerics.qtype_tag(q), data.data_ptr(), scale.data_ptr(),
            _lib.stream_of(rows))
  if q == numerics.INT4:
    qv = qarray.Int4Tensor(data, lead + (n,), len(lead)).permute(*_inverse_movedim(x.ndim, dim))
  else:
    qv = data.movedim(-1, dim)
  return qarray.QArray(qv, scale.movedim(-1, dim).contiguous(), None, q)


def _inverse_movedim(ndim: int, dim: int) -> tuple[int, ...]:
  """Permutation p with y.permute(p) == y.movedim(-1, dim)."""
  order = list(range(ndim - 1))
  order.insert(dim, ndim - 1)
  return tuple(order)


def hadamard_quantized_matmul(act: torch.Tensor, weight: qarray.QArray, pre_sign=None, post_sign=None, *,
                              act_tile: int | None = None, preferred_element_type=None) -> torch.Tensor:
  """quantize_int8(fwht(act)) @ weight in one library call: the counterpart of `hadamard_quantize_multiply`
  (qwix/contrib/kernels/fused_hadamard_quantized_matmul.py:349-414) with the numerics of `rotate_and_quantize`
  followed by the sub-channel quantized dot (dot_general.py:186-203,255-260).

  act: (M, K) bf16 / f32, K a power of two; weight: a symmetric int8 / int4 QArray of logical shape (K, N) with
  scales per output channel and group of `group` rows (tiles along K only), K-contiguous storage as
  `quantize(..., reduce-minor)` writes it; act_tile: None = one scale per token, else the weight's group."""
  from qwix_amd.core import dot_general as dg
  if act.ndim != 2 or not isinstance(weight, qarray.QArray) or weight.zero_point is not None:
    raise NotImplementedError('hadamard_quantized_matmul takes a 2-D activation and a symmetric quantized weight')
  dn = (((1,), (0,)), ((), ()))
  c = dg._Canon(act, weight, dn)
  b, b_is4 = c.rhs_values(weight)
  sb, gb = c.rhs_scale(weight)
  group = c.K // gb
  tile = c.K if act_tile is None else int(act_tile)
  x = act if act.is_contiguous() else act.contiguous()
  res_t = preferred_element_type or act.dtype
  bq = _lib.INT4 if b_is4 else _lib.INT8
  need = int(_lib.load().qwix_hip_qgemm_hadamard_act_workspace_bytes(c.M, c.K, tile, _lib.float_tag(x.dtype)))
  # room behind it for the GEMM's K ranges (few tiles, one scale per token; 0 bytes otherwise)
  need += int(_lib.load().qwix_hip_qgemm_grouped_workspace_bytes(c.M, c.N, c.K, group, bq)) if tile == c.K else 0
  ws = torch.empty(max(int(need), 16), dtype=torch.uint8, device=x.device)
  out = torch.empty(c.M, c.N, dtype=res_t, device=x.device)
  _lib.call('qwix_hip_qgemm_hadamard_act', x.data_ptr(), _lib.float_tag(x.dtype), c.M, c.N, c.K, _lib.ptr(pre_sign),
            _lib.ptr(post_sign), 1.0, tile, b.data_ptr(), b.stride(0), bq, group,
            sb.data_ptr(), _lib.float_tag(sb.dtype), out.data_ptr(), _lib.float_tag(res_t), c.N, ws.data_ptr(), int(need),
            _lib.stream_of(x))
  return out
