"""Post-training quantization provider on top of the HIP quantize / dot_general kernels.

Mirror of qwix/_src/providers/ptq.py (`PtqProvider` :33-49, `quantize_params` :52-135) and of the
parts of providers/boxed_param.py it inherits: `WithAux` (:37-77), `BoxedParamProvider.__init__`
with its three injection points `_qarray_module`, `_dot_general_fn`, `_einsum_fn` (:92-107),
`dot_general` (:109-171), `einsum` (:173-236), `quantize_act` (:416-455, dynamic and static
range) and `create_quantized_param` (:458-499).

Weights reach the provider either as `WithAux[QArray]` (already quantized: used as is) or as a
`Param` (a named float tensor inside a params dict: quantized on first use and written back, which
is how the reference turns float checkpoints into PTQ params); any other float tensor is an
activation.  `precision` / `preferred_element_type` given by the caller are not forwarded, as in
the reference (boxed_param.py:169-171).
"""
from __future__ import annotations

import dataclasses
import functools
from typing import Any, Callable, Generic, Mapping, Sequence, TypeVar

import torch

from qwix_amd import averaging
from qwix_amd import qconfig
from qwix_amd.core import dot_general as _dot_general
from qwix_amd.core import einsum as _einsum
from qwix_amd.core import qarray as _qarray

T = TypeVar('T')


@dataclasses.dataclass
class WithAux(Generic[T]):
  """A (quantized) array plus how it was / is to be quantized, so that quantize_params() can
  quantize float weights without running the model."""

  array: T
  how: _qarray.HowToQuantize

  value = property(lambda self: self.array)
  shape = property(lambda self: tuple(self.array.shape))
  ndim = property(lambda self: len(self.array.shape))
  dtype = property(lambda self: self.array.dtype)

  def replace(self, **kw) -> 'WithAux':
    return dataclasses.replace(self, **kw)

  def reshape(self, *shape):
    if len(shape) == 1 and not isinstance(shape[0], int):
      shape = tuple(shape[0])
    if tuple(self.shape) != tuple(shape):
      raise ValueError(f'Boxed weights should already have the target shape. Got {self.shape=} but {shape=} is requested.')
    return self


@dataclasses.dataclass
class Param:
  """A float weight together with where it lives: `store[name]` (a mutable params dict)."""

  store: dict
  name: str

  value = property(lambda self: self.store[self.name])
  shape = property(lambda self: tuple(self.value.shape))
  ndim = property(lambda self: self.value.ndim)


def create_quantized_param(param: Param, how: _qarray.HowToQuantize, *, _qarray_module=_qarray) -> WithAux:
  """Quantizes a float weight, replaces it in its params dict, and returns the boxed QArray."""
  value = param.value
  if isinstance(value, WithAux):
    return value
  if not isinstance(value, torch.Tensor):
    raise ValueError(f'Cannot quantize param {param.name!r} of type {type(value)}; feed float tensors or WithAux.')
  boxed = WithAux(_qarray_module.quantize(value, how), how)
  param.store[param.name] = boxed
  return boxed


def quantize_act(array: torch.Tensor, how: _qarray.HowToQuantize, rule: qconfig.QuantizationRule, act_name: str, *,
                 store: dict | None = None, quant_stats: Mapping[str, Any] | None = None,
                 _qarray_module=_qarray) -> _qarray.QArray:
  """boxed_param.py:416-455.  Dynamic range: one fused quantize.  Static range (rule.act_static_scale): the
  scale is a parameter `<act_name>_scale` (a WithAux, so that quantize_params can read the qtype; plus
  `<act_name>_zero_point` for asymmetric methods) of the module that issues the op.  When it does not
  exist yet it is created: from collected statistics `quant_stats[act_name]` ({'count', 'sum_of_*'}) if
  there are any, else from the calibration of this very input averaged over rule.act_batch_axes.
  `store` is the module's param dict; ops without one (two activations) use `quant_stats` itself, where a
  precomputed `<act_name>_scale` may also be supplied directly."""
  if not rule.act_static_scale:
    return _qarray_module.quantize(array, how)
  where = store if store is not None else quant_stats
  if where is None:
    raise ValueError(f'static-range quantization of {act_name!r} needs a param store or quant_stats')
  name = act_name + '_scale'
  if name not in where and quant_stats is not None and name in quant_stats:
    where = quant_stats  # a scale computed offline and handed to the provider
  if name not in where:
    stat = None if quant_stats is None else quant_stats.get(act_name)
    if isinstance(stat, Mapping) and 'count' in stat:
      calibration = averaging.SimpleMovingAverage().get_calibration(stat)
      calibration = {k: v.to(array.dtype) for k, v in calibration.items()}
    else:
      calibration = _qarray_module.calibrate(array, how)
      axes = [a for a in rule.act_batch_axes]
      calibration = {k: v.to(torch.float32).mean(dim=axes, keepdim=True).to(v.dtype) for k, v in calibration.items()}
    scale, zp = _qarray_module.compute_scale_zero_point(calibration, how.qtype)
    where[name] = WithAux(scale, how)
    if zp is not None:
      where[act_name + '_zero_point'] = zp
  scale = where[name]
  scale = scale.array if isinstance(scale, WithAux) else scale
  zp = where.get(act_name + '_zero_point')
  return _qarray_module.quantize_with_scale_zero_point(array, how.qtype, scale, zp)


class BoxedParamProvider(qconfig.QuantizationProvider):
  """Runtime ops that substitute boxed (quantized) parameters; subclasses add policy."""

  def __init__(self, rules: Sequence[qconfig.QuantizationRule], *, disable_jit: bool = False, _qarray_module=_qarray,
               _dot_general_fn: Callable = _dot_general.dot_general, _einsum_fn: Callable = _einsum.einsum,
               _conv_general_dilated_fn: Callable | None = None):
    super().__init__(rules, disable_jit=disable_jit)
    self._qarray_module = _qarray_module
    self._dot_general_fn = _dot_general_fn
    self._einsum_fn = _einsum_fn
    self._conv_general_dilated_fn = _conv_general_dilated_fn
    self.quant_stats: dict[str, Any] = {}

  # -- helpers
  def _prepare(self, lhs, rhs, rule, op_id, get_how, quantize_lhs: bool = True):
    store = rhs.store if isinstance(rhs, Param) else None  # the issuing module's params: static scales live there
    if isinstance(rhs, WithAux):
      rhs = rhs.array
    elif isinstance(rhs, Param):
      if isinstance(rhs.value, WithAux):
        rhs = rhs.value.array
      else:
        how = get_how(for_lhs=False, qtype=rule.weight_qtype, calibration_method=rule.weight_calibration_method)
        rhs = create_quantized_param(rhs, how, _qarray_module=self._qarray_module).array
    elif rule.act_qtype is not None:
      how = get_how(for_lhs=False, qtype=rule.act_qtype, calibration_method=rule.act_calibration_method or 'absmax')
      rhs = quantize_act(rhs, how, rule, op_id + '_rhs', store=store, quant_stats=self.quant_stats,
                         _qarray_module=self._qarray_module)
    if rule.act_qtype is not None and quantize_lhs:
      how = get_how(for_lhs=True, qtype=rule.act_qtype, calibration_method=rule.act_calibration_method or 'absmax')
      lhs = quantize_act(lhs, how, rule, op_id + '_lhs', store=store, quant_stats=self.quant_stats,
                         _qarray_module=self._qarray_module)
    return lhs, rhs

  def _fusable(self, rule):
    """The qtype with which the lhs quantization and the GEMM run as one library call, else None: only with the
    stock kernels, dynamic per-token absmax to int8 or e4m3, and no sub-channel tiling."""
    if not (self._dot_general_fn is _dot_general.dot_general and self._qarray_module is _qarray):
      return None
    if rule.act_qtype is None or rule.act_static_scale or rule.tile_size:
      return None
    if (rule.act_calibration_method or 'absmax') != 'absmax':
      return None
    qt = str(rule.act_qtype).replace('torch.', '')
    return qt if qt in ('int8', 'float8_e4m3fn') else None

  @staticmethod
  def _unbox_float(x):
    if isinstance(x, Param):
      x = x.value
    if isinstance(x, WithAux):
      x = x.array
    return _qarray.dequantize(x) if isinstance(x, _qarray.QArray) else x

  # -- ops
  def dot_general(self, lhs, rhs, dimension_numbers, precision=None, preferred_element_type=None, *, out_sharding=None):
    rule, op_id = self._get_current_rule_and_op_id('dot_general')
    if rule is None or rule.weight_qtype is None:
      # no rule for this op: the float contraction, batch axes included (boxed_param.py:119-127)
      return _dot_general.float_dot_general(self._unbox_float(lhs), self._unbox_float(rhs), dimension_numbers,
                                            preferred_element_type)
    get_how = functools.partial(_dot_general.get_how_to_quantize, dimension_numbers=dimension_numbers,
                                ndims=(len(lhs.shape), len(rhs.shape)), tile_size=rule.tile_size)
    fused_qtype = self._fusable(rule)
    if fused_qtype is not None and isinstance(lhs, torch.Tensor):
      lhs, rhs = self._prepare(lhs, rhs, rule, op_id, get_how, quantize_lhs=False)
      out = _dot_general.fused_act_dot_general(lhs, rhs, dimension_numbers, act_qtype=fused_qtype)
      if out is not None:
        return out
      how = get_how(for_lhs=True, qtype=rule.act_qtype, calibration_method='absmax')
      lhs = quantize_act(lhs, how, rule, op_id + '_lhs', quant_stats=self.quant_stats, _qarray_module=self._qarray_module)
    else:
      lhs, rhs = self._prepare(lhs, rhs, rule, op_id, get_how)
    return self._dot_general_fn(lhs, rhs, dimension_numbers, out_sharding=out_sharding)

  def einsum(self, einsum_str: str, *operands, precision=None, preferred_element_type=None, out_sharding=None):
    rule, op_id = self._get_current_rule_and_op_id('einsum')
    if rule is None or rule.weight_qtype is None:
      out = torch.einsum(einsum_str, *[self._unbox_float(o) for o in operands])
      return out if preferred_element_type is None else out.to(preferred_element_type)
    if len(operands) != 2:
      raise ValueError(f'Unsupported einsum format: {einsum_str=} {operands=}')
    lhs, rhs = operands
    get_how = functools.partial(_einsum.get_how_to_quantize, einsum_str=einsum_str,
                                ndims=(len(lhs.shape), len(rhs.shape)), tile_size=rule.tile_size)
    lhs, rhs = self._prepare(lhs, rhs, rule, op_id, get_how)
    return self._einsum_fn(einsum_str, lhs, rhs)


class PtqProvider(BoxedParamProvider):
  """Quantization provider for PTQ: float weights are replaced by quantized ones when the ops run;
  `quantize_params` does the same offline from the `how` recorded in the quantized param tree."""


def _flatten(tree: Mapping, prefix=()) -> dict[tuple, Any]:
  out = {}
  for k, v in tree.items():
    if isinstance(v, Mapping):
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


def quantize_params(params: Mapping, abstract_quantized_params: Mapping, quant_stats: Mapping | None = None, *,
                    allow_extra_params: bool = False, _qarray_module=_qarray) -> dict:
  """Quantizes a float param tree offline.

  `abstract_quantized_params` is the param tree of the PTQ model (leaves that are `WithAux` carry
  the `how`; their arrays may be real or shape-only).  Float leaves whose template is a `WithAux`
  are reshaped to the template's shape and quantized with `_qarray_module.quantize`; other leaves
  are passed through; leaves missing from the template raise unless allow_extra_params.
  """
  abstract = _flatten(abstract_quantized_params)
  out = {}
  for path, param in _flatten(params).items():
    if not isinstance(param, torch.Tensor):
      raise TypeError(f'params is not a pure dict of tensors: {type(param)}')
    tmpl = abstract.get(path)
    if tmpl is None:
      if allow_extra_params:
        continue
      raise ValueError(f'{path} is not found in the abstract_quantized_params.')
    if isinstance(tmpl, WithAux):
      param = param.reshape(tmpl.shape)
      param = tmpl.replace(array=_qarray_module.quantize(param, tmpl.how))
    out[path] = param
  # Static-range activations (ptq.py:106-129): scale and zero point from the collected statistics
  # {module path...: {<act_name>: {'count', 'sum_of_absmax' | 'sum_of_min', 'sum_of_max'}}}.
  stats = _flatten(quant_stats or {})
  for path in sorted({p[:-1] for p in stats}):
    stat = {p[-1]: v for p, v in stats.items() if p[:-1] == path}
    if int(stat['count']) == 0:
      raise ValueError(f'quant_stats is not initialized for {path}.')
    scale_path = path[:-1] + (path[-1] + '_scale',)
    tmpl = abstract.get(scale_path)
    if not isinstance(tmpl, WithAux):
      raise ValueError(f'{scale_path} is not a static scale of the abstract_quantized_params.')
    calibration = averaging.SimpleMovingAverage().get_calibration(stat)
    calibration = {k: v.to(tmpl.array.dtype) for k, v in calibration.items()}
    scale, zero_point = _qarray_module.compute_scale_zero_point(calibration, tmpl.how.qtype)
    out[scale_path] = tmpl.replace(array=scale)
    if zero_point is not None:
      out[path[:-1] + (path[-1] + '_zero_point',)] = zero_point
  return _unflatten(out)
