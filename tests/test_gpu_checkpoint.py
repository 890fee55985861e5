"""GPU: a pre-quantized checkpoint on disk (safetensors) -> process_prequantized_params -> the PTQ model,
checked against the params quantize_params produces and against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import qwix_oracle as O
from tests import util

pytestmark = pytest.mark.gpu
DN = (((1,), (0,)), ((), ()))


def _setup(tile_size=None):
  import qwix_amd
  from qwix_amd import nn
  model = nn.MLP(512, 256)
  g = torch.Generator().manual_seed(77)
  params = model.init(g, 256, torch.float32, util.DEV)
  x = torch.rand(64, 256, generator=g, dtype=torch.float32).to(util.DEV)
  rules = [qwix_amd.QuantizationRule(module_path='.*', weight_qtype='int8', act_qtype='int8', tile_size=tile_size)]
  ptq_model = qwix_amd.quantize_model(model, qwix_amd.PtqProvider(rules))
  template = ptq_model.init(params, x)
  return qwix_amd, model, ptq_model, params, template, x


def _save(qparams, path, drop_scale_repeat=None):
  from safetensors.torch import save_file
  flat = {}
  for name in ('Dense_0', 'Dense_1'):
    q = qparams[name]['kernel'].array
    flat[f'{name}.kernel.array.qvalue'] = q.qvalue.cpu().contiguous()
    flat[f'{name}.kernel.array.scale'] = q.scale.cpu().contiguous()
  save_file(flat, path)


def test_prequantized_safetensors_round_trip(tmp_path):
  from qwix_amd.utils import checkpoint_util as cu
  qwix_amd, model, ptq_model, params, template, x = _setup()
  qparams = qwix_amd.quantize_params(params, template)
  _save(qparams, str(tmp_path / 'model.safetensors'))
  loaded = cu.load_nested_safetensors(str(tmp_path), device='cpu')
  processed = cu.process_prequantized_params(loaded, template)
  for name in ('Dense_0', 'Dense_1'):
    a, b = processed[name]['kernel'].array, qparams[name]['kernel'].array
    assert a.qvalue.device.type == 'cuda' and torch.equal(a.qvalue, b.qvalue) and torch.equal(a.scale, b.scale)
  # codes from the file take the layout quantize() gives such a weight (contracted axis contiguous): the GEMM
  # reads them as they are, no per-call re-layout
  from qwix_amd import _lib
  from qwix_amd.core import qarray as qa_mod
  for name in ('Dense_0', 'Dense_1'):
    a, b = processed[name]['kernel'].array, qparams[name]['kernel'].array
    assert qa_mod.physical_layout(a)[1] == qa_mod.physical_layout(b)[1] == _lib.LAYOUT_REDUCE_MINOR
    assert a.qvalue.stride() == b.qvalue.stride()
  out = ptq_model.apply(processed, x)
  assert torch.equal(out, ptq_model.apply(qparams, x))
  # the rules can be rebuilt from the payload alone
  rules = cu.restore_quantization_rules(loaded, tile_size=None)
  assert sorted(r.module_path for r in rules) == ['Dense_0', 'Dense_1'] and all(r.weight_qtype == torch.int8 for r in rules)
  # and the whole flow equals the oracle's dot_general on the stored codes
  w1 = processed['Dense_0']['kernel'].array
  xq = O.quantize(util.farr(x), O.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  h = O.fast_dot_general(xq, util.to_oracle_qarray(w1), DN)
  hq = O.quantize(O.FArr(np.maximum(h.v, 0), O.F32), O.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  want = O.fast_dot_general(hq, util.to_oracle_qarray(processed['Dense_1']['kernel'].array), DN)
  assert np.array_equal(util.f32np(out), want.v)


def test_block_scaled_checkpoint_runs_like_its_expanded_form(tmp_path):
  """2-D block scales (one per 128 x 128 block) are broadcast to the template's (K / 128, N) scales."""
  from safetensors.torch import save_file
  from qwix_amd.utils import checkpoint_util as cu
  qwix_amd, model, ptq_model, params, template, x = _setup(tile_size=128)
  g = torch.Generator().manual_seed(5)
  flat_2d, flat_1d = {}, {}
  for name, (k, n) in (('Dense_0', (256, 512)), ('Dense_1', (512, 256))):
    q = torch.randint(-128, 128, (k, n), generator=g, dtype=torch.int8)
    s2 = torch.rand(k // 128, n // 128, generator=g) * 0.01 + 0.001
    for flat, s in ((flat_2d, s2), (flat_1d, s2.repeat_interleave(128, dim=1))):
      flat[f'{name}.kernel.array.qvalue'] = q
      flat[f'{name}.kernel.array.scale'] = s.contiguous()
  save_file(flat_2d, str(tmp_path / 'blocks.safetensors'))
  save_file(flat_1d, str(tmp_path / 'expanded.safetensors'))
  p2 = cu.process_prequantized_params(cu.load_nested_safetensors(str(tmp_path / 'blocks.safetensors')), template)
  p1 = cu.process_prequantized_params(cu.load_nested_safetensors(str(tmp_path / 'expanded.safetensors')), template)
  assert tuple(p2['Dense_0']['kernel'].array.scale.shape) == (2, 512)
  assert torch.equal(p2['Dense_0']['kernel'].array.scale, p1['Dense_0']['kernel'].array.scale)
  assert torch.equal(ptq_model.apply(p2, x), ptq_model.apply(p1, x))


@pytest.mark.parametrize('zp', [False, True])
def test_quantized_payload_for_a_float_template_is_dequantized(zp):
  from qwix_amd.utils import checkpoint_util as cu
  g = torch.Generator().manual_seed(9)
  q = torch.randint(-128, 128, (256, 384), generator=g, dtype=torch.int8)
  s = (torch.rand(2, 384, generator=g) * 0.01 + 0.001).to(torch.bfloat16)
  payload = {'qvalue': q, 'scale': s}
  if zp:
    payload['zero_point'] = torch.randint(-128, 128, (2, 384), generator=g, dtype=torch.int8)
  template = {'w': torch.zeros(256, 384, dtype=torch.bfloat16, device=util.DEV)}
  out = cu.process_prequantized_params({'w': payload}, template)['w']
  assert out.dtype == torch.bfloat16 and out.device.type == 'cuda'
  oq = O.QArray(q.numpy(), O.FArr(s.float().numpy(), O.BF16), payload['zero_point'].numpy() if zp else None, 'int8')
  assert np.array_equal(util.f32np(out), O.dequantize(oq).v)
