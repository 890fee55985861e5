"""A few functional layers whose contractions go through the active quantization provider.

The reference intercepts jax.lax.dot_general / jnp.einsum inside Flax modules; without Flax the
same effect is obtained by layers that call `ops.dot_general` / `ops.einsum`, which forward to the
provider installed by `quantize_model` (or run in floating point when none is installed).  Params
are plain nested dicts {module name: {'kernel': tensor}} like an unboxed Linen param tree.
"""
from __future__ import annotations

import threading

import torch

from qwix_amd import qconfig
from qwix_amd.providers.ptq import Param

_tls = threading.local()


def current_provider():
  return getattr(_tls, 'provider', None)


class _Ops:
  """Interception points: the two functions the provider overrides."""

  @staticmethod
  def dot_general(lhs, rhs, dimension_numbers, precision=None, preferred_element_type=None):
    p = current_provider()
    if p is not None:
      return p.dot_general(lhs, rhs, dimension_numbers, precision, preferred_element_type)
    rhs = rhs.value if isinstance(rhs, Param) else rhs
    (lc, rc), _ = dimension_numbers
    return torch.tensordot(lhs, rhs, dims=(list(lc), list(rc)))

  @staticmethod
  def einsum(einsum_str, lhs, rhs, **kw):
    p = current_provider()
    if p is not None:
      return p.einsum(einsum_str, lhs, rhs, **kw)
    return torch.einsum(einsum_str, lhs, rhs.value if isinstance(rhs, Param) else rhs)


ops = _Ops()


class Dense:
  """y = x @ kernel (+ bias); kernel is (in_features, features) as in flax.linen.Dense."""

  def __init__(self, features: int, use_bias: bool = False, name: str = 'Dense_0'):
    self.features, self.use_bias, self.name = features, use_bias, name

  def init(self, gen: torch.Generator, in_features: int, dtype=torch.float32, device='cpu', std: float = 0.02) -> dict:
    p = {'kernel': (torch.randn(in_features, self.features, generator=gen, dtype=torch.float32) * std).to(dtype).to(device)}
    if self.use_bias:
      p['bias'] = torch.zeros(self.features, dtype=dtype, device=device)
    return p

  def __call__(self, params: dict, x: torch.Tensor) -> torch.Tensor:
    with qconfig.module_scope(self.name):
      y = ops.dot_general(x, Param(params, 'kernel'), (((x.ndim - 1,), (0,)), ((), ())))
    if self.use_bias:
      y = y + params['bias'].to(y.dtype)
    return y


class Einsum:
  """y = einsum(subscripts, x, kernel), e.g. 'btd,dnh->btnh'."""

  def __init__(self, subscripts: str, shape, name: str = 'Einsum_0'):
    self.subscripts, self.shape, self.name = subscripts, tuple(shape), name

  def init(self, gen, dtype=torch.float32, device='cpu', std: float = 0.02) -> dict:
    return {'kernel': (torch.randn(*self.shape, generator=gen, dtype=torch.float32) * std).to(dtype).to(device)}

  def __call__(self, params: dict, x: torch.Tensor) -> torch.Tensor:
    with qconfig.module_scope(self.name):
      return ops.einsum(self.subscripts, x, Param(params, 'kernel'))


class MLP:
  """Dense -> ReLU -> Dense, the two-layer model of the PTQ example configuration."""

  def __init__(self, hidden: int, out: int):
    self.layers = [Dense(hidden, name='Dense_0'), Dense(out, name='Dense_1')]

  def init(self, gen, in_features: int, dtype=torch.float32, device='cpu') -> dict:
    p0 = self.layers[0].init(gen, in_features, dtype, device)
    p1 = self.layers[1].init(gen, self.layers[0].features, dtype, device)
    return {'Dense_0': p0, 'Dense_1': p1}

  def __call__(self, params: dict, x: torch.Tensor) -> torch.Tensor:
    h = self.layers[0](params['Dense_0'], x)
    h = torch.relu(h)
    return self.layers[1](params['Dense_1'], h)
