"""Helpers shared by the GPU parity tests: seeded inputs and torch <-> oracle conversions."""
import numpy as np
import torch

from oracle import qwix_oracle as O

DEV = 'cuda:0'
TORCH_DT = {O.F32: torch.float32, O.BF16: torch.bfloat16}
ORACLE_DT = {torch.float32: O.F32, torch.bfloat16: O.BF16}


def rng(seed):
  return np.random.Generator(np.random.PCG64(seed))


def make_np(shape, dtype, seed, scale=1.0, dist='normal'):
  """numpy f32 array holding dtype-representable values from a seeded PCG64 stream."""
  g = rng(seed)
  x = g.standard_normal(shape) if dist == 'normal' else g.uniform(0, 1, shape)
  x = (x * scale).astype(np.float32)
  if dtype == O.BF16:
    x = O.round_to_bf16(x)
  return x


def to_gpu(x: np.ndarray, dtype) -> torch.Tensor:
  return torch.from_numpy(x).to(TORCH_DT[dtype]).to(DEV)


def make(shape, dtype, seed, scale=1.0, dist='normal'):
  """(numpy f32 holding dtype-representable values, torch tensor on the GPU)."""
  x = make_np(shape, dtype, seed, scale, dist)
  return x, to_gpu(x, dtype)


def farr(t: torch.Tensor) -> O.FArr:
  return O.FArr(t.detach().to(torch.float32).cpu().numpy(), ORACLE_DT[t.dtype])


def qvalues_np(qa) -> np.ndarray:
  """Logical quantized values of a qwix_amd QArray: int8 for int8/int4, uint8 bits for e4m3."""
  from qwix_amd.core.qarray import Int4Tensor
  q = qa.qvalue
  if isinstance(q, Int4Tensor):
    return q.unpack().cpu().numpy()
  if q.dtype == torch.float8_e4m3fn:
    return q.contiguous().view(torch.uint8).cpu().numpy()
  return q.contiguous().cpu().numpy()


def f32np(t: torch.Tensor) -> np.ndarray:
  return t.detach().to(torch.float32).cpu().numpy()


def to_oracle_qarray(qa) -> O.QArray:
  zp = None if qa.zero_point is None else qa.zero_point.cpu().numpy()
  return O.QArray(qvalues_np(qa), farr(qa.scale), zp, qa.qtype)


def assert_qarray_equal(qa, want: O.QArray, what=''):
  got_s = f32np(qa.scale)
  assert got_s.shape == want.scale.shape, (what, got_s.shape, want.scale.shape)
  bad = np.flatnonzero(got_s.ravel() != want.scale.v.ravel())
  assert bad.size == 0, f'{what}: {bad.size} scales differ, first at {bad[:5]}: {got_s.ravel()[bad[:5]]} vs {want.scale.v.ravel()[bad[:5]]}'
  got_q = qvalues_np(qa)
  assert got_q.shape == want.qvalue.shape, (what, got_q.shape, want.qvalue.shape)
  bad = np.flatnonzero(got_q.ravel() != want.qvalue.ravel())
  assert bad.size == 0, f'{what}: {bad.size}/{got_q.size} qvalues differ, first at {bad[:5]}: {got_q.ravel()[bad[:5]]} vs {want.qvalue.ravel()[bad[:5]]}'
  if want.zero_point is not None:
    assert np.array_equal(qa.zero_point.cpu().numpy(), want.zero_point), f'{what}: zero points differ'
  else:
    assert qa.zero_point is None


def partials_envelope(acc, oxq, owq) -> np.ndarray:
  """Rounding envelope of the reference's own sub-channel epilogue.

  With bf16 scales the reference rounds every per-group partial three times (convert, * sx, * sy)
  before summing, so two faithful evaluations may differ by up to 3 * 2^-9 * sum_g |partial_g|.
  acc: (G, M, N) int32 partials.  Returns 2^-7 * sum_g |acc_g| * sx * sy_g (f32 scales: 2^-20).
  """
  sx = oxq.scale.v.reshape(oxq.scale.v.shape[0], -1)[:, :1]          # (M, 1)
  sy = owq.scale.v                                                    # (G, N)
  mag = (np.abs(acc).astype(np.float64) * sx[None] * sy[:, None, :]).sum(0)
  eps = 2.0**-7 if O.BF16 in (oxq.scale.dtype, owq.scale.dtype) and O.F32 not in (oxq.scale.dtype, owq.scale.dtype) else 2.0**-20
  return (eps * mag).astype(np.float32)
