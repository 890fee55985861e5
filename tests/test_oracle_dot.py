"""Pins the oracle's dot_general / einsum / hadamard restatement (no GPU needed)."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import qwix_oracle as O

GOLD = json.load(
    open(os.path.join(os.path.dirname(__file__), 'golden', 'known_answers.json'))
)
DN2D = (((1,), (0,)), ((), ()))


def _operand(spec):
  if isinstance(spec, str):
    if spec == 'bool':
      return np.ones((10, 10), np.bool_)
    return O.FArr(np.ones((10, 10), np.float32), spec)
  qt, st = spec
  q = np.ones((10, 10), np.uint8 if qt == O.E4M3 else np.int8)
  if qt == O.E4M3:
    q[:] = 0x38  # 1.0
  return O.QArray(q, O.FArr(np.ones((1, 1), np.float32), st), None, qt)


@pytest.mark.parametrize('case', GOLD['result_dtype'])
def test_output_dtype_table(case):
  """dot_general_test.py:28-146."""
  lhs, rhs = _operand(case['lhs']), _operand(case['rhs'])
  for pref in (None, O.BF16, O.F32):
    want = pref or case['expect']
    _, res = O.get_accumulator_and_result_type(lhs, rhs, preferred_element_type=pref)
    assert res == want, case['src']
    if isinstance(lhs, np.ndarray):
      continue
    assert O.slow_dot_general(lhs, rhs, DN2D, pref).dtype == want if not (
        isinstance(lhs, O.QArray) and False
    ) else True
    assert O.fast_dot_general(lhs, rhs, DN2D, pref).dtype == want
    assert O.einsum('ab,bc->ac', lhs, rhs, pref).dtype == want


def test_accumulator_is_int32_only_for_int_times_int():
  i8 = _operand(['int8', 'bf16'])
  i4 = _operand(['int4', 'f32'])
  f8 = _operand(['float8_e4m3fn', 'bf16'])
  assert O.get_accumulator_and_result_type(i8, i4, preferred_element_type=None) == ('int32', 'f32')
  assert O.get_accumulator_and_result_type(f8, f8, preferred_element_type=None) == ('bf16', 'bf16')
  assert O.get_accumulator_and_result_type(i8, f8, preferred_element_type='f32') == ('f32', 'f32')


def test_innermost_tiling_heuristic():
  c = GOLD['innermost_tiling']
  dn = tuple(tuple(tuple(a) for a in p) for p in c['dimension_numbers'])
  hl = O.dg_get_how_to_quantize(dimension_numbers=dn, ndims=tuple(c['ndims']), for_lhs=True, qtype='int8', tile_size=c['tile_size'])
  hr = O.dg_get_how_to_quantize(dimension_numbers=dn, ndims=tuple(c['ndims']), for_lhs=False, qtype='int8', tile_size=c['tile_size'])
  assert dict(hl.tiled_axes) == {int(k): v for k, v in c['lhs_tiled'].items()}
  assert dict(hr.tiled_axes) == {int(k): v for k, v in c['rhs_tiled'].items()}
  assert list(hl.channelwise_axes) == [0, 1] and list(hr.channelwise_axes) == [2]
  # einsum_test.py:450-473
  hl = O.einsum_get_how_to_quantize(einsum_str='BTNH,NHO->BTO', ndims=(4, 3), for_lhs=True, qtype='int8', tile_size=32)
  hr = O.einsum_get_how_to_quantize(einsum_str='BTNH,NHO->BTO', ndims=(4, 3), for_lhs=False, qtype='int8', tile_size=32)
  assert dict(hl.tiled_axes) == {3: 32} and dict(hr.tiled_axes) == {1: 32}
  assert list(hl.channelwise_axes) == [0, 1] and list(hr.channelwise_axes) == [2]


@pytest.mark.parametrize(
    's,lhs,rhs,out,batch,contract',
    [
        ('abc,bcd->acd', 'abc', 'bcd', 'acd', ['c'], ['b']),
        ('ab,bc->ac', 'ab', 'bc', 'ac', [], ['b']),
        ('bth,thk->btk', 'bth', 'thk', 'btk', ['t'], ['h']),
        (',i->i', '', 'i', 'i', [], []),
    ],
)
def test_einsum_info_parse_table(s, lhs, rhs, out, batch, contract):
  """einsum_info_test.py:66-100."""
  info = O.EinsumInfo.parse(s)
  assert (info.lhs, info.rhs, info.out) == (lhs, rhs, out)
  assert info.batch_chars == batch and info.contract_chars == contract


def test_einsum_info_dimension_numbers_and_perm():
  c = GOLD['einsum_info'][0]
  info = O.EinsumInfo.parse(c['einsum'])
  dn = info.dimension_numbers
  assert [[list(a) for a in p] for p in dn] == c['dimension_numbers']
  assert list(info.output_perm) == c['output_perm']
  assert O.EinsumInfo.parse('ab,bc->ac').output_perm is None
  with pytest.raises(NotImplementedError):
    O.EinsumInfo.parse('ab,bc')
  with pytest.raises(NotImplementedError):
    O.EinsumInfo.parse('aab,bc->ac')


# ------------------------------------------------------------------ integer dot


def test_int_dot_is_exact():
  rng = np.random.default_rng(0)
  a = rng.integers(-128, 128, (37, 4096), dtype=np.int8)
  b = rng.integers(-128, 128, (4096, 29), dtype=np.int8)
  want = a.astype(np.int64) @ b.astype(np.int64)
  la = O.QArray(a, O.FArr(np.ones((37, 1), np.float32)), None, 'int8')
  rb = O.QArray(b, O.FArr(np.ones((1, 29), np.float32)), None, 'int8')
  out, acc = O.fast_dot_general(la, rb, DN2D, return_acc=True)
  assert acc.dtype == np.int32 and np.array_equal(acc, want)
  assert np.array_equal(out.v, want.astype(np.float32))


def test_fast_epilogue_order_and_bf16_rounding_vs_torch():
  """out = bf16(bf16(bf16(f32(acc)) * sx) * sy) — torch-CPU bf16 as the judge."""
  rng = np.random.default_rng(1)
  a = rng.integers(-128, 128, (16, 256), dtype=np.int8)
  b = rng.integers(-128, 128, (256, 24), dtype=np.int8)
  sx = O.round_to_bf16(rng.uniform(0.001, 0.1, (16, 1)).astype(np.float32))
  sy = O.round_to_bf16(rng.uniform(0.001, 0.1, (1, 24)).astype(np.float32))
  out = O.fast_dot_general(
      O.QArray(a, O.FArr(sx, O.BF16), None, 'int8'),
      O.QArray(b, O.FArr(sy, O.BF16), None, 'int8'),
      DN2D,
  )
  acc = torch.from_numpy((a.astype(np.int64) @ b.astype(np.int64)).astype(np.int32))
  t = acc.to(torch.float32).to(torch.bfloat16)
  t = t * torch.from_numpy(sx).to(torch.bfloat16)
  t = t * torch.from_numpy(sy).to(torch.bfloat16)
  assert out.dtype == O.BF16
  assert np.array_equal(out.v, t.to(torch.float32).numpy())


def test_fast_slow_dequant_agree_2d_scales():
  """two_dim_scales_test.py:57-93 invariant: fast == slow == dequant @ dequant."""
  rng = np.random.default_rng(2)
  l = rng.standard_normal((128, 128)).astype(np.float32)
  r = rng.standard_normal((128, 128)).astype(np.float32)
  how = O.HowToQuantize(qtype='int8', tiled_axes={0: 8, 1: 8})
  lq, rq = O.quantize(O.FArr(l), how), O.quantize(O.FArr(r), how)
  assert lq.scale.shape == (16, 16)
  true = O.dequantize(lq).v.astype(np.float64) @ O.dequantize(rq).v.astype(np.float64)
  fast = O.fast_dot_general(lq, rq, DN2D).v
  slow = O.slow_dot_general(lq, rq, DN2D).v
  assert np.allclose(fast, true, rtol=1e-4, atol=1e-4)
  assert np.allclose(slow, true, rtol=1e-4, atol=1e-4)
  assert not O.use_fast_path(lq, rq, DN2D)  # tile 8 < 128 -> dispatcher picks slow


def test_subchannel_fast_path_bruteforce():
  """K split in groups of 128: per-group int32 partials, scaled, then summed."""
  rng = np.random.default_rng(3)
  m, k, n, g = 24, 384, 40, 128
  x = rng.standard_normal((m, k)).astype(np.float32)
  w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
  xq = O.quantize(O.FArr(x), O.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  wq = O.quantize(O.FArr(w), O.HowToQuantize(qtype='int4', channelwise_axes=[1], tiled_axes={0: g}))
  assert wq.scale.shape == (3, n)
  assert O.use_fast_path(xq, wq, DN2D)
  out, acc = O.fast_dot_general(xq, wq, DN2D, return_acc=True)
  assert acc.shape == (3, m, n) and acc.dtype == np.int32
  want = np.zeros((m, n), np.float32)
  for gi in range(3):
    part = xq.qvalue[:, gi * g : (gi + 1) * g].astype(np.int64) @ wq.qvalue[gi * g : (gi + 1) * g].astype(np.int64)
    assert np.array_equal(acc[gi], part)
    want = want + (part.astype(np.float32) * xq.scale.v) * wq.scale.v[gi][None, :]
  assert np.array_equal(out.v, want)
  # and it approximates the float product
  ref = x.astype(np.float64) @ w.astype(np.float64)
  assert np.abs(out.v - ref).mean() / np.abs(ref).mean() < 0.13  # einsum_test.py w4a8 ceiling is 0.12 at full size


def test_lhs_tile_mismatch_and_two_asymmetric_raise():
  a = np.ones((4, 256), np.int8)
  b = np.ones((256, 4), np.int8)
  la = O.QArray(a, O.FArr(np.ones((4, 2), np.float32)), None, 'int8')
  rb = O.QArray(b, O.FArr(np.ones((4, 4), np.float32)), None, 'int8')
  with pytest.raises(ValueError, match='same tile size'):
    O.fast_dot_general(la, rb, DN2D)
  la = O.QArray(a, O.FArr(np.ones((4, 1), np.float32)), np.zeros((4, 1), np.int8), 'int8')
  rb = O.QArray(b, O.FArr(np.ones((1, 4), np.float32)), np.zeros((1, 4), np.int8), 'int8')
  with pytest.raises(ValueError, match='Only one operand can be asymmetric'):
    O.fast_dot_general(la, rb, DN2D)


def test_zero_point_correction_equals_dequantized_product():
  rng = np.random.default_rng(4)
  x = (rng.standard_normal((6, 256)) + 0.7).astype(np.float32)
  w = rng.standard_normal((256, 9)).astype(np.float32)
  xq = O.quantize(O.FArr(x), O.HowToQuantize(qtype='int8', channelwise_axes=[0], calibration_method='minmax'))
  wq = O.quantize(O.FArr(w), O.HowToQuantize(qtype='int8', channelwise_axes=[1]))
  fast = O.fast_dot_general(xq, wq, DN2D).v
  true = O.dequantize(xq).v.astype(np.float64) @ O.dequantize(wq).v.astype(np.float64)
  assert np.allclose(fast, true, rtol=1e-5, atol=1e-5)


def test_dispatcher_rule():
  """dot_general.py:439-472."""
  q = O.QArray(np.ones((256, 8), np.int8), O.FArr(np.ones((2, 8), np.float32)), None, 'int4')
  assert not O.use_fast_path(O.FArr(np.ones((4, 256), np.float32), O.BF16), q, DN2D)  # raw float lhs
  assert O.use_fast_path(np.ones((4, 256), np.int8), q, DN2D)  # raw int8 lhs stays fast
  q64 = O.QArray(np.ones((256, 8), np.int8), O.FArr(np.ones((4, 8), np.float32)), None, 'int4')
  lq = O.QArray(np.ones((4, 256), np.int8), O.FArr(np.ones((4, 1), np.float32)), None, 'int8')
  assert O.use_fast_path(lq, q, DN2D) and not O.use_fast_path(lq, q64, DN2D)


def test_weight_only_slow_path_matches_float_dot():
  rng = np.random.default_rng(5)
  x = O.round_to_bf16(rng.standard_normal((8, 256)).astype(np.float32))
  w = O.round_to_bf16((rng.standard_normal((256, 16)) * 0.02).astype(np.float32))
  wq = O.quantize_api(O.FArr(w, O.BF16), 'int4', channelwise_axes=[1], tiled_axes={0: 128}, scale_dtype=O.F32)
  out = O.dot_general(O.FArr(x, O.BF16), wq, DN2D, O.BF16)
  assert out.dtype == O.BF16
  ref = x.astype(np.float64) @ w.astype(np.float64)
  assert np.abs(out.v - ref).mean() / np.abs(ref).mean() < 0.12


def test_einsum_with_batch_and_output_perm():
  rng = np.random.default_rng(6)
  a = rng.standard_normal((3, 256, 4)).astype(np.float32)   # a b c
  b = rng.standard_normal((256, 4, 5)).astype(np.float32)   # b c d
  how_l = O.einsum_get_how_to_quantize(einsum_str='abc,bcd->acd', ndims=(3, 3), for_lhs=True, qtype='int8', tile_size=None)
  how_r = O.einsum_get_how_to_quantize(einsum_str='abc,bcd->acd', ndims=(3, 3), for_lhs=False, qtype='int8', tile_size=None)
  assert list(how_l.channelwise_axes) == [0, 2] and list(how_r.channelwise_axes) == [1, 2]
  out = O.einsum('abc,bcd->acd', O.quantize(O.FArr(a), how_l), O.quantize(O.FArr(b), how_r))
  ref = np.einsum('abc,bcd->acd', a.astype(np.float64), b.astype(np.float64))
  assert out.shape == (3, 4, 5)
  assert np.abs(out.v - ref).mean() / np.abs(ref).mean() < 0.02  # einsum_test.py w8a8 ceiling


def test_fp8_fast_path_close_to_float():
  rng = np.random.default_rng(7)
  x = O.round_to_bf16(rng.standard_normal((16, 512)).astype(np.float32))
  w = O.round_to_bf16((rng.standard_normal((512, 32)) * 0.02).astype(np.float32))
  xq = O.quantize(O.FArr(x, O.BF16), O.HowToQuantize(qtype='float8_e4m3fn', channelwise_axes=[0]))
  wq = O.quantize(O.FArr(w, O.BF16), O.HowToQuantize(qtype='float8_e4m3fn', channelwise_axes=[1]))
  out = O.dot_general(xq, wq, DN2D, O.BF16)
  ref = x.astype(np.float64) @ w.astype(np.float64)
  assert np.abs(out.v - ref).mean() / np.abs(ref).mean() < 0.045  # einsum_test.py fp8-act ceiling is 0.038 at full size
  # dequantized product is the exact target of the fp8 path
  deq = O.dequantize(xq).v.astype(np.float64) @ O.dequantize(wq).v.astype(np.float64)
  assert np.allclose(out.v, deq, rtol=3e-2, atol=1e-2)


# ------------------------------------------------------------------ hadamard


@pytest.mark.parametrize('p', [0, 1, 3, 6])
def test_hadamard_matrix_properties(p):
  """hadamard_rot_test.py:24-41 + popcount closed form."""
  h = O.hadamard_matrix(p)
  n = 2**p
  assert np.array_equal(h @ h.T, n * np.eye(n, dtype=np.float32))
  i, j = np.meshgrid(np.arange(n), np.arange(n), indexing='ij')
  pc = np.array([[bin(int(v)).count('1') for v in row] for row in (i & j)])
  assert np.array_equal(h, (-1.0) ** pc)


@pytest.mark.parametrize('row,col', [(False, False), (True, False), (False, True), (True, True)])
def test_hadamard_rotation_preserves_product(row, col):
  """hadamard_rot_test.py:92-147: (x had)(had^T w / n) == x w within 1e-4."""
  rng = np.random.default_rng(8)
  n = 64
  x = rng.standard_normal((8, n)).astype(np.float32)
  w = rng.standard_normal((n, 16)).astype(np.float32)
  rs = rng.choice([-1.0, 1.0], n) if row else None
  cs = rng.choice([-1.0, 1.0], n) if col else None
  xr, wr = O.hadamard_rotate_inputs(O.FArr(x), O.FArr(w), rs, cs, lhs_reduction_dim=1, rhs_reduction_dim=0)
  assert np.allclose(xr.v @ wr.v, x @ w, atol=1e-4)
  # closed form on a unit vector: row i of had.
  e = np.zeros((1, n), np.float32)
  e[0, 5] = 1
  xr, _ = O.hadamard_rotate_inputs(O.FArr(e), O.FArr(w), rs, cs, lhs_reduction_dim=1, rhs_reduction_dim=0)
  want = O.hadamard_matrix(6)[5] * (rs[5] if row else 1) * (cs if col else 1)
  assert np.array_equal(xr.v[0], want)


def test_hadamard_rejects_bad_sizes():
  with pytest.raises(ValueError, match='power of 2'):
    O.hadamard_rotate_inputs(O.FArr(np.ones((2, 6))), O.FArr(np.ones((6, 2))), None, None, lhs_reduction_dim=1, rhs_reduction_dim=0)
  with pytest.raises(ValueError, match='to be the same'):
    O.hadamard_rotate_inputs(O.FArr(np.ones((2, 8))), O.FArr(np.ones((4, 2))), None, None, lhs_reduction_dim=1, rhs_reduction_dim=0)


def test_contraction_to_a_scalar():
  """Operands without free or batch axes contract to a 0-d result (bf16 rounding and reshapes keep the shape ())."""
  x = O.FArr(O.round_to_bf16(np.arange(32, dtype=np.float32) / 7), O.BF16)
  w = O.FArr(O.round_to_bf16(np.arange(32, dtype=np.float32)[::-1] / 9), O.BF16)
  how = O.HowToQuantize(qtype='int8', channelwise_axes=[])
  xq, wq = O.quantize(x, how), O.quantize(w, how)
  out = O.dot_general(xq, wq, (((0,), (0,)), ((), ())))
  assert out.v.shape == () and out.dtype == O.BF16
  acc = int(xq.qvalue.astype(np.int64) @ wq.qvalue.astype(np.int64))
  want = O.round_to_bf16(O.round_to_bf16(O.round_to_bf16(np.float32(acc)) * xq.scale.v.reshape(())) * wq.scale.v.reshape(()))
  assert float(out.v) == float(want)
