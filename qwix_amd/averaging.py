"""Aggregation of calibration values over calibration steps (static-range quantization).

Mirror of qwix/_src/averaging.py:25-99: a quantization statistic is a dict {'count': int32 scalar,
'sum_of_<key>': float32 tensor} per calibration key ('absmax', or 'min' and 'max'); the calibration used
for the static scale is the plain average sum / count.  Host-side arithmetic on scale-shaped tensors.
"""
from __future__ import annotations

from typing import Mapping

import torch

Calibration = Mapping[str, torch.Tensor]
QuantStat = dict


class SimpleMovingAverage:
  """averaging.py:25-99."""

  def __init__(self, bootstrap_steps: int = 0):
    self._bootstrap_steps = bootstrap_steps

  def init(self, calibration: Calibration) -> QuantStat:
    """Empty statistics shaped like `calibration`.  The sums are float32 whatever the calibration dtype: a
    bf16 sum stops growing after a few hundred steps."""
    first = next(iter(calibration.values()))
    stat = {'count': torch.zeros((), dtype=torch.int32, device=first.device)}
    for key, value in calibration.items():
      stat[f'sum_of_{key}'] = torch.zeros(value.shape, dtype=torch.float32, device=value.device)
    return stat

  def update(self, quant_stat: QuantStat, calibration: Calibration) -> QuantStat:
    out = dict(quant_stat)
    out['count'] = quant_stat['count'] + 1
    for key, value in calibration.items():
      have = quant_stat[f'sum_of_{key}']
      if tuple(have.shape) != tuple(value.shape):  # no silent broadcasting: it usually hides a config error
        raise ValueError(f'Shape mismatch between {quant_stat} and {calibration}')
      out[f'sum_of_{key}'] = have + value.to(torch.float32)
    return out

  def get_calibration(self, quant_stat: QuantStat, default_calibration: Calibration | None = None) -> dict:
    """The average calibration; `default_calibration` (if given) is returned instead while no more than
    `bootstrap_steps` samples have been seen, and fixes the dtype of the result."""
    count = quant_stat['count']
    calibration = {key[len('sum_of_'):]: value / count for key, value in quant_stat.items() if key.startswith('sum_of_')}
    if default_calibration is None:
      return calibration
    if int(count) > self._bootstrap_steps:
      return {k: v.to(default_calibration[k].dtype) for k, v in calibration.items()}
    return dict(default_calibration)
