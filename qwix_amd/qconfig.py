"""Quantization rules and the provider base class (host-side configuration only).

Mirror of qwix/_src/qconfig.py: `QuantizationRule` (:31-92, same field names and defaults) and
the rule lookup of `QuantizationProvider._get_current_rule_and_op_id` (:209-240): the first rule
whose `module_path` regex fully matches '/'.join(current module path) and whose `op_names` (if
any) contains the op wins; per (module, op) an op id '<op><n>' numbers repeated ops.

There is no Flax here, so the "current module path" comes from `module_scope`, a thread-local
stack that the bundled `qwix_amd.nn` modules (or user code) push while they run.
"""
from __future__ import annotations

import contextlib
import dataclasses
import re
import threading
from typing import Any, Collection, Sequence


@dataclasses.dataclass(frozen=True, kw_only=True)
class QuantizationRule:
  """Which modules / ops to quantize, and how.  Fields as in the reference."""

  module_path: str = '.*'
  op_names: Collection[str] = ()
  weight_qtype: Any = None
  act_qtype: Any = None
  tile_size: int | float | None = None
  act_static_scale: bool | None = None
  weight_calibration_method: str = 'absmax'
  act_calibration_method: str | None = None
  act_batch_axes: Collection[int] = (0,)


_tls = threading.local()


def current_module_path() -> tuple[str, ...]:
  return tuple(getattr(_tls, 'path', ()))


@contextlib.contextmanager
def module_scope(name: str):
  """Pushes `name` on this thread's module path for the duration of the block."""
  old = current_module_path()
  _tls.path = old + (name,)
  try:
    yield
  finally:
    _tls.path = old


class QuantizationProvider:
  """Holds the rules and resolves the rule that applies to the op being executed."""

  def __init__(self, rules: Sequence[QuantizationRule], *, disable_jit: bool = False):
    self._rules = [self._init_rule(rule) for rule in rules]
    self._rule_matches = [False] * len(self._rules)
    self._op_counts: dict[tuple[tuple[str, ...], str], int] = {}
    self._initial_run_complete = False  # set by the model wrapper once the model has run under this provider
    self.disable_jit = disable_jit

  @staticmethod
  def _init_rule(rule: QuantizationRule) -> QuantizationRule:
    """Validates a rule and fills its defaults (qconfig.py:122-135)."""
    if rule.act_qtype is None and rule.act_static_scale is not None:
      raise ValueError(f'Invalid rule: act_static_scale is set to {rule.act_static_scale} but act_qtype is None. '
                       'Please either unset act_static_scale, or set act_qtype to enable activation quantization. '
                       f'(Rule: {rule})')
    if rule.act_static_scale is None:
      rule = dataclasses.replace(rule, act_static_scale=False)
    if rule.act_calibration_method is None:
      rule = dataclasses.replace(rule, act_calibration_method='absmax')
    return rule

  def reset_op_ids(self) -> None:
    """Op ids restart at 0 for every model call, so that the same op gets the same id each time."""
    self._op_counts = {}

  def _get_current_rule_and_op_id(self, op_name: str, *, only_rule: bool = False):
    path = current_module_path()
    path_str = '/'.join(path)
    rule = None
    for i, r in enumerate(self._rules):
      if re.fullmatch(r.module_path, path_str) and (not r.op_names or op_name in r.op_names):
        rule = r
        self._rule_matches[i] = True
        break
    if only_rule:
      return rule, None
    n = self._op_counts.get((path, op_name), 0)
    self._op_counts[(path, op_name)] = n + 1
    return rule, f'{op_name}{n}'

  def get_unused_rules(self) -> list[QuantizationRule]:
    """Rules that never matched (qconfig.py:242-262); only meaningful once the model has run."""
    if not self._initial_run_complete:
      raise ValueError('Quantization is not completed yet. Please call `quantize_model` and run the model '
                       'before calling `get_unused_rules`.')
    return [r for r, used in zip(self._rules, self._rule_matches) if not used]
