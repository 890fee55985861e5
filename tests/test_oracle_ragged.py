"""Pins the oracle's ragged dot (CPU only).

The reference's own tests for this operator hold no known-answer vectors (their inputs come from
jax.random and they assert error ceilings: ragged_dot_test.py:36-330), so the restatement is pinned
by what the operator must reduce to: group by group it is the already pinned dot_general on a row
slice, tiny cases are recomputed with explicit Python loops, and the group_sizes patterns of the
reference's tests (empty groups, sizes that stop short of or reach past the last row) are covered."""
import numpy as np
import pytest

from oracle import qwix_oracle as O
from tests import util

DN = (((1,), (0,)), ((), ()))

# (64,32,16,16), (128,100,0,28), (50,50,28,0), (128,0,0,0), (10,20,30,68): ragged_dot_test.py:36-228
GROUP_SIZES = [(64, 32, 16, 16), (128, 100, 0, 28), (50, 50, 28, 0), (128, 0, 0, 0), (10, 20, 30, 68), (5, 0, 7, 3)]


def _operands(dtype, seed, lhs_how, rhs_how, m=128, k=256, g=4, n=64):
  x = O.FArr(util.make_np((m, k), dtype, seed), dtype)
  w = O.FArr(util.make_np((g, k, n), dtype, seed + 1, scale=0.05), dtype)
  return O.quantize(x, lhs_how), O.quantize(w, rhs_how)


def _slice_rhs(q: O.QArray, g: int) -> O.QArray:
  s = q.scale.v
  return O.QArray(q.qvalue[g], O.FArr(s[g if s.shape[0] > 1 else 0], q.scale.dtype), None, q.qtype)


def _slice_lhs(q: O.QArray, a: int, b: int) -> O.QArray:
  s = q.scale.v
  return O.QArray(q.qvalue[a:b], O.FArr(s[a:b] if s.shape[0] > 1 else s, q.scale.dtype), None, q.qtype)


HOWS = [
    ('per-tensor', O.HowToQuantize(qtype='int8'), O.HowToQuantize(qtype='int8')),
    ('channelwise', O.HowToQuantize(qtype='int8', channelwise_axes=[0]), O.HowToQuantize(qtype='int8', channelwise_axes=[2])),
    ('group+channel', O.HowToQuantize(qtype='int8', channelwise_axes=[0]), O.HowToQuantize(qtype='int8', channelwise_axes=[0, 2])),
    ('group only', O.HowToQuantize(qtype='int8'), O.HowToQuantize(qtype='int8', channelwise_axes=[0])),
    ('k tiled', O.HowToQuantize(qtype='int8', channelwise_axes=[0]),
     O.HowToQuantize(qtype='int8', channelwise_axes=[0, 2], tiled_axes={1: 128})),
    ('both tiled', O.HowToQuantize(qtype='int8', channelwise_axes=[0], tiled_axes={1: 128}),
     O.HowToQuantize(qtype='int8', channelwise_axes=[2], tiled_axes={1: 128})),
    ('fp8', O.HowToQuantize(qtype=O.E4M3, channelwise_axes=[0]), O.HowToQuantize(qtype=O.E4M3, channelwise_axes=[0, 2])),
]


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('sizes', GROUP_SIZES)
@pytest.mark.parametrize('name,lhs_how,rhs_how', HOWS)
def test_ragged_dot_is_dot_general_group_by_group(name, lhs_how, rhs_how, sizes, dtype):
  xq, wq = _operands(dtype, 11, lhs_how, rhs_how)
  got = O.fast_ragged_dot(xq, wq, sizes)
  m = xq.qvalue.shape[0]
  want = np.zeros_like(got.v)
  start = 0
  for g, size in enumerate(sizes):
    stop = min(start + size, m)
    if stop > start:
      want[start:stop] = O.fast_dot_general(_slice_lhs(xq, start, stop), _slice_rhs(wq, g), DN).v
    start = stop
  # also for fp8: both routes round one f64 sum, and the masked rows only add exact zeros to it
  assert np.array_equal(got.v, want)
  assert np.all(got.v[min(sum(sizes), m):] == 0)


def test_ragged_dot_brute_force_tiny():
  rng = util.rng(5)
  m, k, g, n = 9, 4, 3, 5
  a = rng.integers(-128, 128, (m, k)).astype(np.int8)
  b = rng.integers(-128, 128, (g, k, n)).astype(np.int8)
  sa = O.FArr(rng.uniform(0.5, 2, (m, 1)).astype(np.float32), O.F32)
  sb = O.FArr(rng.uniform(0.5, 2, (g, 1, n)).astype(np.float32), O.F32)
  sizes = (2, 0, 4)  # rows 6..8 belong to no group
  got = O.fast_ragged_dot(O.QArray(a, sa, None, 'int8'), O.QArray(b, sb, None, 'int8'), sizes)
  group_of = [0, 0, 2, 2, 2, 2, None, None, None]
  for i in range(m):
    for j in range(n):
      if group_of[i] is None:
        assert got.v[i, j] == 0
        continue
      acc = 0
      for kk in range(k):
        acc += int(a[i, kk]) * int(b[group_of[i], kk, j])
      want = np.float32(np.float32(np.float32(acc) * sa.v[i, 0]) * sb.v[group_of[i], 0, j])
      assert got.v[i, j] == want, (i, j)


def test_single_group_is_dot_general():
  xq, wq = _operands(O.BF16, 3, HOWS[1][1], HOWS[1][2], m=64, k=128, g=1, n=48)
  got = O.fast_ragged_dot(xq, wq, (64,))
  want = O.fast_dot_general(xq, _slice_rhs(wq, 0), DN)
  assert np.array_equal(got.v, want.v)


def test_raw_int8_operands_give_int32():
  rng = util.rng(9)
  a = rng.integers(-128, 128, (20, 16)).astype(np.int8)
  b = rng.integers(-128, 128, (2, 16, 8)).astype(np.int8)
  got = O.fast_ragged_dot(a, b, (12, 8))
  want = np.concatenate([a[:12].astype(np.int64) @ b[0].astype(np.int64), a[12:].astype(np.int64) @ b[1].astype(np.int64)])
  assert got.dtype == np.int32 and np.array_equal(got, want)


def test_dispatch_and_slow_path_agree_with_fast():
  # ragged_dot_test.py:281-330: the dequantize-first and the quantized path agree to 0.3 % of the mean magnitude
  xq, wq = _operands(O.F32, 21, HOWS[2][1], HOWS[2][2])
  fast = O.ragged_dot(xq, wq, (10, 20, 30, 68))
  slow = O.slow_ragged_dot(xq, wq, (10, 20, 30, 68))
  assert np.abs(fast.v - slow.v).mean() / np.abs(slow.v).mean() < 0.003
  # a zero point or a raw float operand sends the call to the dequantize-first path (ragged_dot.py:278-292)
  x = O.FArr(util.make_np((128, 256), O.F32, 4), O.F32)
  xz = O.quantize(x, O.HowToQuantize(qtype='int8', calibration_method='minmax'))
  assert np.array_equal(O.ragged_dot(xz, wq, (64, 64, 0, 0)).v, O.slow_ragged_dot(xz, wq, (64, 64, 0, 0)).v)
  assert np.array_equal(O.ragged_dot(x, wq, (64, 64, 0, 0)).v, O.slow_ragged_dot(x, wq, (64, 64, 0, 0)).v)


@pytest.mark.parametrize('dtype', [O.BF16, O.F32])
@pytest.mark.parametrize('name,lhs_how,rhs_how', HOWS[:4])
@pytest.mark.parametrize('sizes', [(128, 100, 0, 28), (10, 20, 30, 68), (5, 0, 7, 3)])
def test_general_dimension_numbers_reduce_to_ragged_dot(name, lhs_how, rhs_how, sizes, dtype):
  """ragged_dot_general on the dimension numbers of ragged_dot is fast_ragged_dot, bit for bit (the two are written
  independently: a masked sum with expanded scales against one dot_general per group)."""
  xq, wq = _operands(dtype, 11, lhs_how, rhs_how)
  want = O.ragged_dot(xq, wq, sizes)
  got = O.ragged_dot_general(xq, wq, sizes, (((1,), (1,)), ((), ())), 0, 0)
  assert got.dtype == want.dtype and np.array_equal(got.v, want.v)


def test_general_dimension_numbers_with_a_batch_axis_and_tiles():
  """The reference's non-basic case (tests/_src/core/ragged_dot_test.py:255-275): lhs (32, 620, 256) and rhs (32, 4, 256)
  int8 in tiles of 64 along K, batch axis 0, ragged axis 1, group axis 1, groups (60, 120, 190, 250).  Its inputs
  come from jax.random, so the reference's bound is what is checked: relative mean absolute error against the float
  result below 0.04 (a smaller batch keeps the CPU run short); and batch element by batch element the result is the
  basic ragged dot of that element."""
  dn, sizes = (((2,), (2,)), ((0,), (0,))), (60, 120, 190, 250)
  x = util.make_np((4, 620, 256), O.F32, 5)
  w = util.make_np((4, 4, 256), O.F32, 6)
  how = O.HowToQuantize(qtype='int8', tiled_axes={2: 64})
  xq, wq = O.quantize(O.FArr(x, O.F32), how), O.quantize(O.FArr(w, O.F32), how)
  got = O.ragged_dot_general(xq, wq, sizes, dn, 1, 1)
  assert got.v.shape == (4, 620)
  rows_group = np.repeat(np.arange(4), sizes)
  want_fp = np.einsum('bmk,bmk->bm', x.astype(np.float64), w.astype(np.float64)[:, rows_group, :])
  assert np.abs(got.v - want_fp).mean() / np.abs(want_fp).mean() < 0.04
  for b in range(4):
    assert xq.scale.v.shape == (1, 1, 4) and wq.scale.v.shape == (1, 1, 4)      # one scale per K tile
    xb = O.QArray(xq.qvalue[b], O.FArr(xq.scale.v[0], O.F32), None, 'int8')
    wb = O.QArray(wq.qvalue[b][:, :, None], O.FArr(wq.scale.v[0][:, :, None], O.F32), None, 'int8')   # (G, K, N=1)
    assert np.array_equal(O.ragged_dot(xb, wb, sizes).v[:, 0], got.v[b])
