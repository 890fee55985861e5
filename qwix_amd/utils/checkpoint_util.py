"""Bringing pre-quantized checkpoints into a PTQ param tree.

Mirror of qwix/_src/utils/checkpoint_util.py: `process_prequantized_params` (:383-498) with its
three cases (:445-477), the leaf handling of `_process_quantized_param` (:212-273: cast to the
template's dtypes, block-wise scales broadcast to the template's scale shape, zero point required
iff the template has one), `_dequantize_quantized_param` (:276-349) and
`restore_quantization_rules` (:504-587).  `load_nested_safetensors` plays the part of the loader in
integration_tests/orbax_safetensors_test.py:41-83: a flat `a.b.c` safetensors file becomes a nested
dict whose quantized leaves are dicts {'qvalue', 'scale'[, 'zero_point']}.

The template is the PTQ param tree of this package (`QuantizedModel.init`): nested dicts whose
quantized leaves are `WithAux[QArray]` and whose other leaves are float tensors.  Everything here
is host glue around device tensors; the only arithmetic is `dequantize`, which is the HIP kernel.
"""
from __future__ import annotations

import logging
import os
from typing import Any, Mapping

import torch

from qwix_amd import qconfig
from qwix_amd.core import qarray
from qwix_amd.providers.ptq import WithAux

_PREQUANTIZED_ARRAY_LEAF_NAMES = frozenset(('qvalue', 'scale', 'zero_point'))
_log = logging.getLogger(__name__)


def _is_leaf(x) -> bool:
  return isinstance(x, dict) and 'qvalue' in x


def _flatten(tree: Mapping, prefix=()) -> dict[tuple, Any]:
  """Flattens nested dicts; a dict holding 'qvalue' is a (pre-quantized) leaf."""
  out = {}
  for k, v in tree.items():
    if isinstance(v, Mapping) and not _is_leaf(v):
      out.update(_flatten(v, prefix + (k,)))
    else:
      out[prefix + (k,)] = v
  return out


def _unflatten(flat: Mapping[tuple, Any]) -> dict:
  out: dict = {}
  for path, v in flat.items():
    d = out
    for k in path[:-1]:
      d = d.setdefault(k, {})
    d[path[-1]] = v
  return out


def _get(tree, path):
  for k in path:
    if not isinstance(tree, Mapping) or k not in tree:
      return None
    tree = tree[k]
  return tree


def load_nested_safetensors(path: str, device='cpu', rename_rules=None) -> dict:
  """Loads `path` (a .safetensors file, or a directory of them) as a nested dict: key 'a.b.c' becomes
  tree['a']['b']['c'].  `rename_rules` is a sequence of (regex, replacement) applied to the flat keys
  first.  Tensors are read with safetensors' own reader (no code from the file is executed)."""
  import re
  from safetensors import safe_open
  files = [path]
  if os.path.isdir(path):
    files = sorted(os.path.join(path, f) for f in os.listdir(path) if f.endswith('.safetensors'))
    if not files:
      raise FileNotFoundError(f'no .safetensors file in {path}')
  flat = {}
  for f in files:
    with safe_open(f, framework='pt', device='cpu') as sf:
      for key in sf.keys():
        name = key
        for pat, rep in rename_rules or ():
          name = re.sub(pat, rep, name)
        if name in flat:
          raise ValueError(f'duplicate tensor name {name!r} (from {key!r} in {f})')
        flat[name] = sf.get_tensor(key).to(device)
  return _unflatten({tuple(k.split('.')): v for k, v in flat.items()})


def broadcast_to(x: torch.Tensor, shape) -> torch.Tensor:
  """Tile-wise broadcast (qarray.py:447-467): an axis of size s grows to a multiple t*s by repeating
  each element t times, so a (4, 4) block scale of a 128 x 128 weight becomes (4, 128)."""
  try:
    return qarray._broadcast_tensor(x, tuple(shape))
  except ValueError:
    raise ValueError(f'cannot broadcast {tuple(x.shape)} to {tuple(shape)}') from None


def _validate_prequantized_dict(checkpoint_param, path) -> None:
  if not isinstance(checkpoint_param, dict):
    raise ValueError(f'{path} is quantized in the template_params. Expected a dict containing qvalue/scale leaves.')
  unsupported = set(checkpoint_param) - _PREQUANTIZED_ARRAY_LEAF_NAMES
  if unsupported:
    raise ValueError(f'{path} has unsupported quantized leaves {sorted(unsupported)}. Expected only '
                     f'{sorted(_PREQUANTIZED_ARRAY_LEAF_NAMES)}.')
  if 'qvalue' not in checkpoint_param or 'scale' not in checkpoint_param:
    summary = {k: (type(v), getattr(v, 'shape', None)) for k, v in checkpoint_param.items()}
    raise ValueError(f'{path} is missing required "qvalue" or "scale" in pre-quantized dictionary. Found keys: '
                     f'{list(checkpoint_param.keys())}, summary: {summary}')


def _as_tensor(x, device) -> torch.Tensor:
  if isinstance(x, torch.Tensor):
    return x.to(device)
  import numpy as np
  return torch.from_numpy(np.ascontiguousarray(x)).to(device)


def _coerce(value, template: torch.Tensor, path, allow_broadcast=False, follow_layout=False) -> torch.Tensor:
  """Device, dtype (a value conversion, e.g. int8 codes into an e4m3 template) and shape of the template.
  follow_layout: also the template's memory layout (a weight that quantize() stores with its contracted axis
  contiguous keeps that layout when its codes come from a file, so that no GEMM has to re-lay it out)."""
  if isinstance(template, qarray.Int4Tensor) or not isinstance(template, torch.Tensor):
    raise TypeError(f'{path} does not resolve to a dense tensor in the template_params.')
  value = _as_tensor(value, template.device)
  if value.dtype != template.dtype:
    value = value.to(template.dtype)
  if tuple(value.shape) != tuple(template.shape):
    if not allow_broadcast:
      raise ValueError(f'{path} has shape {tuple(value.shape)}, expected {tuple(template.shape)}.')
    try:
      value = broadcast_to(value, template.shape)
    except ValueError as e:
      raise ValueError(f'{path} has shape {tuple(value.shape)}, expected {tuple(template.shape)}.') from e
  if follow_layout and not template.is_contiguous() and value.numel() and _is_dense_permutation(template):
    out = torch.empty_strided(tuple(template.shape), template.stride(), dtype=value.dtype, device=value.device)
    out.copy_(value)  # one re-layout at load time
    return out
  return value.contiguous()


def _is_dense_permutation(t: torch.Tensor) -> bool:
  """True when t is a permuted view of a dense row-major block (what empty_strided can reproduce)."""
  order = sorted(range(t.ndim), key=lambda a: (-t.stride(a), a))
  return t.permute(*order).is_contiguous()


def _template_fields(template_param):
  """(qvalue, scale, zero_point) templates of a quantized template leaf."""
  t = template_param.array if isinstance(template_param, WithAux) else template_param
  if isinstance(t, qarray.QArray):
    return t.qvalue, t.scale, t.zero_point
  return t.get('qvalue'), t.get('scale'), t.get('zero_point')


def _process_quantized_param(checkpoint_param, template_param, path):
  _validate_prequantized_dict(checkpoint_param, path)
  t_q, t_s, t_zp = _template_fields(template_param)
  qvalue = _coerce(checkpoint_param['qvalue'], t_q, path, follow_layout=True)
  scale = _coerce(checkpoint_param['scale'], t_s, path, allow_broadcast=True)
  zero_point = checkpoint_param.get('zero_point')
  if t_zp is None and zero_point is not None:
    raise ValueError(f'{path} provided an unexpected "zero_point" for a symmetric quantized param.')
  if t_zp is not None and zero_point is None:
    raise ValueError(f'{path} is missing required quantized leaf "zero_point".')
  if t_zp is not None:
    zero_point = _coerce(zero_point, t_zp, path, allow_broadcast=True)
  tq = template_param.array if isinstance(template_param, WithAux) else template_param
  qtype = tq.qtype if isinstance(tq, qarray.QArray) else qvalue.dtype
  leaf = qarray.QArray(qvalue, scale, zero_point, qtype)
  qarray.validate_qarray(leaf)
  return template_param.replace(array=leaf) if isinstance(template_param, WithAux) else leaf


def _dequantize_quantized_param(checkpoint_param, template_param: torch.Tensor, path) -> torch.Tensor:
  _validate_prequantized_dict(checkpoint_param, path)
  dev = template_param.device
  qvalue = _as_tensor(checkpoint_param['qvalue'], dev).contiguous()
  scale = _as_tensor(checkpoint_param['scale'], dev).contiguous()
  if scale.ndim < qvalue.ndim:
    scale = scale.reshape((1,) * (qvalue.ndim - scale.ndim) + tuple(scale.shape))
  zp = checkpoint_param.get('zero_point')
  if zp is not None:
    zp = _as_tensor(zp, dev).contiguous()
  leaf = qarray.QArray(qvalue, scale, zp, qvalue.dtype)
  return _coerce(qarray.dequantize(leaf), template_param, path)


def process_prequantized_params(checkpoint_params: Mapping[str, Any], template_params: Mapping[str, Any], *,
                                allow_extra_params: bool = False) -> dict:
  """Turns an external pre-quantized payload into a param tree the PTQ model runs on.

  `checkpoint_params`: nested dict; a leaf is a tensor (or numpy array) or a dict
  {'qvalue', 'scale'[, 'zero_point']}.  `template_params`: the PTQ param tree.  For each payload
  leaf: quantized payload + quantized template -> a QArray coerced to the template (boxed like the
  template); quantized payload + float template -> dequantized; float + float -> cast; a float
  payload for a quantized template is an error (quantize_params handles that direction).  A payload
  path may end in 'array' where the template leaf is the boxed array itself."""
  if not isinstance(template_params, Mapping):
    raise TypeError(f'process_prequantized_params expects the PTQ param tree (nested dicts). Got {type(template_params)}.')
  out = {}
  for path, checkpoint_param in _flatten(checkpoint_params).items():
    resolved, template_param = path, _get(template_params, path)
    if template_param is None and path and path[-1] == 'array':
      resolved, template_param = path[:-1], _get(template_params, path[:-1])
    if template_param is None:
      if not allow_extra_params:
        raise ValueError(f'Found extra parameters in prequantized_params not present in template: {resolved}')
      _log.info('Skipping parameter not in template: %s', resolved)
      continue
    if isinstance(template_param, Mapping) and 'array' in template_param and not _is_leaf(template_param):
      template_param = template_param['array']
    template_quantized = isinstance(template_param, (WithAux, qarray.QArray)) or _is_leaf(template_param)
    if isinstance(checkpoint_param, dict) and template_quantized:
      processed = _process_quantized_param(checkpoint_param, template_param, resolved)
    elif isinstance(checkpoint_param, dict):
      processed = _dequantize_quantized_param(checkpoint_param, template_param, resolved)
    elif not template_quantized:
      processed = _coerce(checkpoint_param, template_param, resolved)
    else:
      raise ValueError(f'Unhandled or invalid parameter combination for {resolved}. checkpoint_param is '
                       f'{type(checkpoint_param)}, template_param is {type(template_param)}.')
    out[resolved] = processed
  return _unflatten(out)


_DEFAULT_ACT_QTYPE = object()


def restore_quantization_rules(checkpoint_params: Mapping[str, Any], rule_type=qconfig.QuantizationRule, *,
                               tile_size, act_qtype=_DEFAULT_ACT_QTYPE, **kwargs) -> list:
  """One rule per module that holds a pre-quantized weight: weight_qtype = the dtype of its qvalue,
  'minmax' if it has a zero point else 'absmax', numeric path components become wildcards, and
  act_qtype defaults to the weight's qtype."""
  rules = {}
  for path, checkpoint_param in _flatten(checkpoint_params).items():
    if not _is_leaf(checkpoint_param):
      continue
    module_path = path[:-1] if path and path[-1] == 'array' else path
    module_path = module_path[:-1]
    parts = ['[^/]+' if isinstance(p, int) or (isinstance(p, str) and p.isdigit()) else str(p) for p in module_path]
    module_path_str = '/'.join(parts)
    weight_qtype = checkpoint_param['qvalue'].dtype
    rule = rule_type(module_path=module_path_str, weight_qtype=weight_qtype,
                     act_qtype=weight_qtype if act_qtype is _DEFAULT_ACT_QTYPE else act_qtype,
                     weight_calibration_method='minmax' if checkpoint_param.get('zero_point') is not None else 'absmax',
                     tile_size=tile_size, **kwargs)
    if module_path_str in rules and rules[module_path_str] != rule:
      _log.warning('Conflicting quantization rules reconstructed for %s. Existing: %s, New: %s. The existing rule '
                   'will be overwritten.', module_path_str, rules[module_path_str], rule)
    rules[module_path_str] = rule
  return list(rules.values())
