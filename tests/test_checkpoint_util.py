"""Pre-quantized checkpoint ingestion (host logic on CPU tensors; the GPU part is in test_gpu_checkpoint.py).

The rule-restoring cases are the tables of the reference's tests/_src/utils/checkpoint_util_test.py:809-1018
(payloads and expected rules restated with torch dtypes); the error cases follow :214-251,253-274."""
import logging

import numpy as np
import pytest
import torch

from qwix_amd import qconfig
from qwix_amd.core import qarray
from qwix_amd.providers.ptq import WithAux
from qwix_amd.utils import checkpoint_util as cu


def _q(dtype=torch.int8, zp=False):
  d = {'qvalue': torch.ones(4, 4, dtype=dtype), 'scale': torch.ones(1, 4, dtype=torch.float32)}
  if zp:
    d['zero_point'] = torch.zeros(1, 4, dtype=torch.int8)
  return d


def _rule(path, wq, aq, method='absmax'):
  return qconfig.QuantizationRule(module_path=path, weight_qtype=wq, act_qtype=aq, weight_calibration_method=method, tile_size=4)


def test_restore_rules_linear_and_nested():
  rules = cu.restore_quantization_rules({'kernel': _q(), 'bias': torch.zeros(4)}, qconfig.QuantizationRule, tile_size=4)
  assert rules == [_rule('', torch.int8, torch.int8)]
  rules = cu.restore_quantization_rules({'dense1': {'kernel': _q()}, 'dense2': {'kernel': _q(torch.int16)}}, tile_size=4)
  assert sorted(rules, key=lambda r: r.module_path) == [_rule('dense1', torch.int8, torch.int8), _rule('dense2', torch.int16, torch.int16)]


def test_restore_rules_wildcards(caplog):
  with caplog.at_level(logging.WARNING):
    rules = cu.restore_quantization_rules({'layers': {0: {'kernel': _q(torch.uint8)}, 1: {'kernel': _q()}}}, tile_size=4)
  assert rules == [_rule('layers/[^/]+', torch.int8, torch.int8)]
  assert 'Conflicting quantization rules reconstructed for layers/[^/]+' in caplog.text
  caplog.clear()
  with caplog.at_level(logging.WARNING):
    rules = cu.restore_quantization_rules({'layers': {0: {'kernel': _q()}, 1: {'kernel': _q()}}}, tile_size=4)
  assert rules == [_rule('layers/[^/]+', torch.int8, torch.int8)] and not caplog.text
  # keys read from a flat file are strings: '0' is a wildcard as well
  assert cu.restore_quantization_rules({'layers': {'0': {'kernel': {'array': _q()}}}}, tile_size=4) == [
      _rule('layers/[^/]+', torch.int8, torch.int8)]


def test_restore_rules_act_and_asymmetric():
  assert cu.restore_quantization_rules({'kernel': _q()}, tile_size=4, act_qtype=None) == [_rule('', torch.int8, None)]
  assert cu.restore_quantization_rules({'kernel': _q()}, tile_size=4, act_qtype=torch.uint8) == [_rule('', torch.int8, torch.uint8)]
  assert cu.restore_quantization_rules({'kernel': _q(zp=True)}, tile_size=4) == [_rule('', torch.int8, torch.int8, 'minmax')]


def _template(zp=False, scale_shape=(1, 6), qdtype=torch.int8):
  how = qarray.HowToQuantize(qtype='int8', channelwise_axes=[1])
  q = qarray.QArray(torch.zeros(12, 6, dtype=qdtype), torch.zeros(scale_shape, dtype=torch.float32),
                    torch.zeros(scale_shape, dtype=torch.int8) if zp else None, 'int8')
  return {'kernel': WithAux(q, how), 'bias': torch.zeros(6, dtype=torch.float32)}


def _payload(zp=False, scale_shape=(1, 6)):
  g = torch.Generator().manual_seed(0)
  p = {'qvalue': torch.randint(-128, 128, (12, 6), generator=g, dtype=torch.int8),
       'scale': torch.rand(scale_shape, generator=g) + 0.1}
  if zp:
    p['zero_point'] = torch.randint(-128, 128, scale_shape, generator=g, dtype=torch.int8)
  return {'kernel': {'array': p}, 'bias': torch.arange(6, dtype=torch.float64)}


@pytest.mark.parametrize('zp', [False, True])
def test_quantized_payload_into_quantized_template(zp):
  payload = _payload(zp)
  out = cu.process_prequantized_params(payload, _template(zp))
  leaf = out['kernel']
  assert isinstance(leaf, WithAux) and leaf.how.channelwise_axes == [1]
  assert torch.equal(leaf.array.qvalue, payload['kernel']['array']['qvalue'])
  assert torch.equal(leaf.array.scale, payload['kernel']['array']['scale'])
  assert (leaf.array.zero_point is None) == (not zp)
  if zp:
    assert torch.equal(leaf.array.zero_point, payload['kernel']['array']['zero_point'])
  # float payload, float template: cast to the template's dtype
  assert out['bias'].dtype == torch.float32 and torch.equal(out['bias'], torch.arange(6, dtype=torch.float32))
  # the path may also name the boxed leaf directly
  direct = {'kernel': payload['kernel']['array']}
  assert torch.equal(cu.process_prequantized_params(direct, _template(zp))['kernel'].array.qvalue, leaf.array.qvalue)


def test_block_scales_are_broadcast_to_the_template():
  # integration_tests/orbax_safetensors_test.py:275-340: (4, 4) block scales for a template with (4, 128) scales
  s2 = torch.rand(4, 4) + 0.1
  q = torch.randint(-128, 128, (128, 128), dtype=torch.int8)
  how = qarray.HowToQuantize(qtype='int8', channelwise_axes=[1], tiled_axes={0: 32})
  tmpl = {'w': WithAux(qarray.QArray(torch.zeros(128, 128, dtype=torch.int8), torch.zeros(4, 128), None, 'int8'), how)}
  out = cu.process_prequantized_params({'w': {'array': {'qvalue': q, 'scale': s2}}}, tmpl)
  assert torch.equal(out['w'].array.scale, s2.repeat_interleave(32, dim=1))
  assert torch.equal(cu.broadcast_to(torch.tensor([1., 2.]), (2, 4)), torch.tensor([[1., 1., 2., 2.], [1., 1., 2., 2.]]))
  with pytest.raises(ValueError, match='shape'):
    cu.process_prequantized_params({'w': {'array': {'qvalue': q, 'scale': torch.rand(3, 128)}}}, tmpl)


def test_codes_are_converted_to_the_template_dtype():
  # orbax_safetensors_test.py:222-273: int8 codes loaded into a float8_e4m3fn template keep their values
  q = torch.randint(-16, 16, (12, 6), dtype=torch.int8)
  out = cu.process_prequantized_params({'kernel': {'array': {'qvalue': q, 'scale': torch.ones(1, 6)}}},
                                       {'kernel': _template(qdtype=torch.float8_e4m3fn)['kernel']})
  assert out['kernel'].array.qvalue.dtype == torch.float8_e4m3fn
  assert torch.equal(out['kernel'].array.qvalue.float(), q.float())


@pytest.mark.parametrize('modify,regex', [
    (lambda p: p['kernel']['array'].pop('scale'), 'scale'),
    (lambda p: p['kernel']['array'].update({'qvalue': p['kernel']['array']['qvalue'][:-1]}), 'shape'),
    (lambda p: p['kernel']['array'].update({'zero_point': torch.zeros(1, 6, dtype=torch.int8)}), 'unexpected'),
    (lambda p: p['kernel']['array'].update({'codebook': torch.zeros(1)}), 'unsupported quantized leaves'),
])
def test_errors(modify, regex):
  payload = _payload()
  modify(payload)
  with pytest.raises(ValueError, match=regex):
    cu.process_prequantized_params(payload, _template())


def test_missing_zero_point_extra_params_and_bad_combinations():
  with pytest.raises(ValueError, match='missing required quantized leaf "zero_point"'):
    cu.process_prequantized_params(_payload(False), _template(True))
  payload = _payload()
  payload['other'] = torch.zeros(3)
  with pytest.raises(ValueError, match='extra'):
    cu.process_prequantized_params(payload, _template())
  out = cu.process_prequantized_params(payload, _template(), allow_extra_params=True)
  assert set(out) == {'kernel', 'bias'}
  with pytest.raises(ValueError, match='Unhandled or invalid parameter combination'):
    cu.process_prequantized_params({'kernel': torch.zeros(12, 6)}, _template())
  with pytest.raises(TypeError, match='PTQ param tree'):
    cu.process_prequantized_params({}, object())
  assert cu.process_prequantized_params({}, _template()) == {}


def test_load_nested_safetensors(tmp_path):
  from safetensors.torch import save_file
  flat = {'model.layers.0.q_proj.weight.array.qvalue': torch.ones(8, 8, dtype=torch.int8),
          'model.layers.0.q_proj.weight.array.scale': torch.ones(1, 8),
          'model.embed.weight': torch.ones(8, 8, dtype=torch.bfloat16)}
  save_file(flat, str(tmp_path / 'model.safetensors'))
  tree = cu.load_nested_safetensors(str(tmp_path))
  leaf = tree['model']['layers']['0']['q_proj']['weight']['array']
  assert set(leaf) == {'qvalue', 'scale'} and leaf['qvalue'].dtype == torch.int8
  assert tree['model']['embed']['weight'].dtype == torch.bfloat16
  renamed = cu.load_nested_safetensors(str(tmp_path / 'model.safetensors'), rename_rules=[(r'^model\.', '')])
  assert 'layers' in renamed and 'embed' in renamed
  rules = cu.restore_quantization_rules(tree, tile_size=None)
  assert [r.module_path for r in rules] == ['model/layers/[^/]+/q_proj']
