"""Helpers shared by the GPU parity tests: seeded inputs and torch <-> oracle conversions."""
import numpy as np
import torch

from oracle import qwix_oracle as O

DEV = 'cuda:0'
TORCH_DT = {O.F32: torch.float32, O.BF16: torch.bfloat16}
ORACLE_DT = {torch.float32: O.F32, torch.bfloat16: O.BF16}


def rng(seed):
  return np.random.Generator(np.random.PCG64(seed))


def make(shape, dtype, seed, scale=1.0, dist='normal'):
  """(numpy f32 holding dtype-representable values, torch tensor on the GPU)."""
  g = rng(seed)
  x = g.standard_normal(shape) if dist == 'normal' else g.uniform(0, 1, shape)
  x = (x * scale).astype(np.float32)
  if dtype == O.BF16:
    x = O.round_to_bf16(x)
  return x, torch.from_numpy(x).to(TORCH_DT[dtype]).to(DEV)


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
