"""quantize_model: runs a model with a quantization provider installed.

Mirror of qwix/_src/model.py:51-89 in spirit: the returned object behaves like the model, but while
it runs, the contractions issued through `qwix_amd.nn.ops` are routed to the provider
(thread-locally, so other threads keep running in floating point, as with the reference's
per-thread interception).  Models are callables `model(params, *inputs)` over nested param dicts.
"""
from __future__ import annotations

from typing import Any

from qwix_amd import nn
from qwix_amd import qconfig


class QuantizedModel:
  def __init__(self, model, provider: qconfig.QuantizationProvider):
    self.model, self.provider = model, provider

  def apply(self, params: dict, *inputs, **kwargs):
    """Runs the model.  Float kernels in `params` that a rule covers are quantized in place (the
    dict is updated with WithAux[QArray] leaves), exactly once; quantized params are used as is."""
    old = nn.current_provider()
    nn._tls.provider = self.provider
    self.provider.reset_op_ids()
    try:
      out = self.model(params, *inputs, **kwargs)
      self.provider._initial_run_complete = True
      return out
    finally:
      nn._tls.provider = old

  __call__ = apply

  def init(self, params: dict, *inputs, **kwargs) -> dict:
    """Returns the PTQ param tree (WithAux leaves carrying `how`) obtained by running the model once
    on a copy of the float params; serves as `abstract_quantized_params` for quantize_params()."""
    p = _shallow_copy(params)  # structural copy: the tensors themselves are never mutated
    self.apply(p, *inputs, **kwargs)
    return p


def _shallow_copy(tree: Any):
  return {k: _shallow_copy(v) if isinstance(v, dict) else v for k, v in tree.items()}


def quantize_model(model, provider: qconfig.QuantizationProvider, *model_inputs, **kwargs) -> QuantizedModel:
  """Wraps `model` so that its ops are quantized according to `provider`'s rules."""
  del model_inputs, kwargs
  return QuantizedModel(model, provider)
