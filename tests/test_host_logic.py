"""CPU-only tests: host-side mirror of the reference interface, and the C-ABI library surface."""
import ctypes
import os
import re

import pytest
import torch

from oracle import qwix_oracle as O
from qwix_amd import _lib, qconfig
from qwix_amd.core import dot_general as dg
from qwix_amd.core import einsum as es
from qwix_amd.core import einsum_info, numerics, qarray

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_every_declared_symbol():
  header = open(os.path.join(ROOT, 'include', 'qwix_hip.h')).read()
  declared = sorted(set(re.findall(r'\b(qwix_hip_\w+)\s*\(', header)))
  assert len(declared) >= 15
  lib = _lib.load()
  for name in declared:
    assert hasattr(lib, name), f'{name} is declared in include/qwix_hip.h but not exported'
    assert name in _lib.SIGNATURES, f'{name} has no ctypes prototype'
  assert sorted(_lib.SIGNATURES) == declared
  assert lib.qwix_hip_abi_version() == 1
  # a pure host-side entry point (no GPU work): workspace size query
  assert lib.qwix_hip_quantize_workspace_bytes(1, 4096, 4096, 4096, _lib.ABSMAX) == 4096 * 4
  assert lib.qwix_hip_quantize_workspace_bytes(8, 4096, 1, 4096, _lib.ABSMAX) == 0
  assert lib.qwix_hip_quantize_workspace_bytes(1, 4096, 64, 128, _lib.MINMAX) == 32 * 64 * 4 * 2


def test_argument_validation_happens_before_any_launch():
  lib = _lib.load()
  # null pointers / bad geometry are rejected on the host, with a message
  assert lib.qwix_hip_quantize(None, 0, 1, 8, 1, 8, 0, 0, 0.0, 0, None, None, None, None, 0, None) == 1
  assert b'null' in lib.qwix_hip_last_error()
  assert lib.qwix_hip_fwht(ctypes.c_void_p(16), 0, 4, 6, None, None, 1.0, ctypes.c_void_p(16), None) == 1
  assert b'power of 2' in lib.qwix_hip_last_error()
  with pytest.raises(_lib.QwixHipError, match='no CPU path'):
    qarray.quantize(torch.zeros(4, 8), qarray.HowToQuantize(qtype='int8'))


def test_bounds_and_eligibility():
  assert numerics.get_symmetric_bound('int8') == 127.5 and numerics.get_symmetric_bound(torch.int8) == 127.5
  assert numerics.get_symmetric_bound('int4') == 7.5 and numerics.get_symmetric_bound(torch.float8_e4m3fn) == 448.0
  assert numerics.get_asymmetric_bound('int4') == (-8.0, 7.0)
  with pytest.raises(ValueError, match="doesn't support asymmetric"):
    numerics.get_asymmetric_bound('nf4')
  assert numerics.should_quantize(torch.bfloat16) and not numerics.should_quantize(torch.int8)
  assert not numerics.can_dequant_on_output('nf4') and numerics.can_dequant_on_output('int4')


def test_scale_shape_rules_match_oracle():
  for shape, cw, tiled in [((2, 2, 6), [0], {2: 2}), ((128, 128), [], {0: 8, 1: 8}), ((16, 64), [1], {}), ((4, 12), [0], {1: 1 / 3})]:
    a = qarray.get_scale_shape(shape, qarray.HowToQuantize(qtype='int8', channelwise_axes=cw, tiled_axes=tiled))
    b = O.get_scale_shape(shape, O.HowToQuantize(qtype='int8', channelwise_axes=cw, tiled_axes=tiled))
    assert a == b
  with pytest.raises(ValueError, match='cannot be tiled'):
    qarray.get_scale_shape((4, 10), qarray.HowToQuantize(qtype='int8', tiled_axes={1: 4}))
  with pytest.raises(ValueError, match='both channelwise and tiled'):
    qarray.get_scale_shape((4, 8), qarray.HowToQuantize(qtype='int8', channelwise_axes=[1], tiled_axes={1: 4}))


def test_plan_maps_patterns_to_kernel_views():
  P = qarray._plan
  assert P((64, 4096), (1, 4096)).dims == (64, 4096, 1)
  assert P((512, 256), (128, 1)).dims == (1, 512, 256) and P((512, 256), (128, 1)).tiles == (128,)
  assert P((2, 3, 512), (1, 1, 512)).dims == (6, 512, 1)
  assert P((256, 4, 32), (128, 1, 1)).dims == (1, 256, 128)
  p = P((4, 64, 128), (4, 64, 1))
  assert p.dims == (1, 256, 128) and p.tiles == (256,) and p.reduce_axes == (0, 1) and p.inner_axes == (2,)
  assert P((128, 128), (8, 8)).kind == '5d'
  assert P((4, 64, 128), (4, 32, 1)).dims == (1, 4, 1, 64, 128)
  with pytest.raises(NotImplementedError):
    P((4, 4, 4, 4, 4, 4), (2, 1, 2, 1, 2, 1))


def test_get_how_to_quantize_matches_oracle():
  dn = (((2, 3), (0, 1)), ((), ()))
  for for_lhs in (True, False):
    a = dg.get_how_to_quantize(dimension_numbers=dn, ndims=(4, 3), for_lhs=for_lhs, qtype='int8', tile_size=32)
    b = O.dg_get_how_to_quantize(dimension_numbers=dn, ndims=(4, 3), for_lhs=for_lhs, qtype='int8', tile_size=32)
    assert dict(a.tiled_axes) == dict(b.tiled_axes) and list(a.channelwise_axes) == list(b.channelwise_axes)
    a = es.get_how_to_quantize(einsum_str='BTNH,NHO->BTO', ndims=(4, 3), for_lhs=for_lhs, qtype='int8', tile_size=32)
    b = O.einsum_get_how_to_quantize(einsum_str='BTNH,NHO->BTO', ndims=(4, 3), for_lhs=for_lhs, qtype='int8', tile_size=32)
    assert dict(a.tiled_axes) == dict(b.tiled_axes) and list(a.channelwise_axes) == list(b.channelwise_axes)
  h = dg.get_how_to_quantize(dimension_numbers=(((1,), (0,)), ((), ())), ndims=(2, 2), for_lhs=False, qtype='int4', tile_size={0: 128})
  assert dict(h.tiled_axes) == {0: 128} and list(h.channelwise_axes) == [1]


@pytest.mark.parametrize(
    's,ndims,batch,contract,nl,nr,no',
    [('abc,bcd->acd', None, ['c'], ['b'], 3, 3, 3), ('ab,bc->ac', None, [], ['b'], 2, 2, 2), ('bth,thk->btk', None, ['t'], ['h'], 3, 3, 3),
     (',i->i', None, [], [], 0, 1, 1), ('...a,ab->...b', (2, 2), [], ['a'], 2, 2, 2), ('ab,...b->...a', (2, 2), [], ['b'], 2, 2, 2),
     ('...a,...b->...', (2, 2), None, [], 2, 2, 1)],
)
def test_einsum_info_parse_table(s, ndims, batch, contract, nl, nr, no):
  """einsum_info_test.py:66-130 (subscript letters chosen for '...' may differ; structure may not)."""
  info = einsum_info.EinsumInfo.parse(s, ndims=ndims)
  assert (len(info.lhs), len(info.rhs), len(info.out)) == (nl, nr, no)
  if batch is not None:
    assert info.batch_chars == batch
  else:
    assert len(info.batch_chars) == 1
  assert info.contract_chars == contract
  o = O.EinsumInfo.parse(f'{info.lhs},{info.rhs}->{info.out}')
  assert info.dimension_numbers == o.dimension_numbers and info.output_perm == o.output_perm


def test_einsum_info_rejects_unsupported_strings():
  with pytest.raises(NotImplementedError):
    einsum_info.EinsumInfo.parse('ab,bc')
  with pytest.raises(NotImplementedError):
    einsum_info.EinsumInfo.parse('aab,bc->ac')


@pytest.mark.parametrize(
    'lhs,rhs,expect',
    [(torch.bfloat16, torch.float32, torch.float32), (torch.bfloat16, ('int8', torch.bfloat16), torch.bfloat16),
     (torch.bfloat16, ('int8', torch.float32), torch.float32), (('int4', torch.bfloat16), ('int8', torch.float32), torch.float32),
     (('float8_e4m3fn', torch.bfloat16), ('float8_e4m3fn', torch.float32), torch.float32), (torch.bool, ('int8', torch.bfloat16), torch.bfloat16)],
)
def test_result_dtype_table(lhs, rhs, expect):
  """dot_general_test.py:28-146, on CPU tensors (no kernels run)."""
  def mk(spec):
    if not isinstance(spec, tuple):
      return torch.ones(10, 10).to(spec)
    qt, st = spec
    if qt == 'int4':
      q = qarray.Int4Tensor(torch.zeros(10, 5, dtype=torch.uint8), (10, 10), 1)
    else:
      q = torch.ones(10, 10).to(numerics.storage_dtype(qt))
    return qarray.QArray(q, torch.ones(1, 1, dtype=st), None, qt)
  a, b = mk(lhs), mk(rhs)
  for pref in (None, torch.bfloat16, torch.float32):
    acc, res = qarray.get_accumulator_and_result_type(a, b, preferred_element_type=pref)
    assert res == (pref or expect)
  acc, _ = qarray.get_accumulator_and_result_type(mk(('int8', torch.bfloat16)), mk(('int4', torch.float32)), preferred_element_type=None)
  assert acc == torch.int32


def test_dispatcher_rule_and_validation():
  q = qarray.QArray(torch.zeros(256, 8, dtype=torch.int8), torch.ones(2, 8), None, 'int8')
  q64 = qarray.QArray(torch.zeros(256, 8, dtype=torch.int8), torch.ones(4, 8), None, 'int8')
  lq = qarray.QArray(torch.zeros(4, 256, dtype=torch.int8), torch.ones(4, 1), None, 'int8')
  dn = (((1,), (0,)), ((), ()))
  assert not dg._use_fast_path(torch.zeros(4, 256, dtype=torch.bfloat16), q, dn)
  assert dg._use_fast_path(torch.zeros(4, 256, dtype=torch.int8), q, dn)
  assert dg._use_fast_path(lq, q, dn) and not dg._use_fast_path(lq, q64, dn)
  with pytest.raises(ValueError, match='should be broadcastable'):
    qarray.validate_qarray(qarray.QArray(torch.ones(10, 10, dtype=torch.int8), torch.ones(10, 3)))
  assert qarray.get_tiled_axes(qarray.QArray(torch.ones(10, 256, 16, dtype=torch.int8), torch.ones(10, 8, 2))) == {1: 32, 2: 8}


def test_rule_lookup_first_full_match_wins_and_op_ids():
  rules = [qconfig.QuantizationRule(module_path='decoder/.*attn', weight_qtype='int4', tile_size=128),
           qconfig.QuantizationRule(module_path='.*', op_names=('einsum',), weight_qtype='float8_e4m3fn'),
           qconfig.QuantizationRule(module_path='.*', weight_qtype='int8', act_qtype='int8'),
           qconfig.QuantizationRule(module_path='never', weight_qtype='int8')]
  p = qconfig.QuantizationProvider(rules)
  with qconfig.module_scope('decoder'), qconfig.module_scope('self_attn'):
    r, op = p._get_current_rule_and_op_id('dot_general')
    assert r.weight_qtype == 'int4' and op == 'dot_general0'
    assert p._get_current_rule_and_op_id('dot_general')[1] == 'dot_general1'
  with qconfig.module_scope('mlp'):
    assert p._get_current_rule_and_op_id('einsum')[0].weight_qtype == 'float8_e4m3fn'
    assert p._get_current_rule_and_op_id('dot_general')[0].act_qtype == 'int8'
  assert qconfig.current_module_path() == ()
  with pytest.raises(ValueError, match='Quantization is not completed yet'):   # qconfig_test.py:97-115
    p.get_unused_rules()
  p._initial_run_complete = True   # what the model wrapper sets after the first run
  assert [r.module_path for r in p.get_unused_rules()] == ['never']
  # qconfig_test.py:117-127 and the defaults of qconfig.py:122-135
  with pytest.raises(ValueError, match='act_static_scale is set to True but act_qtype is None'):
    qconfig.QuantizationProvider([qconfig.QuantizationRule(weight_qtype='int8', act_static_scale=True)])
  filled = qconfig.QuantizationProvider([qconfig.QuantizationRule(weight_qtype='int8', act_qtype='int8')])._rules[0]
  assert filled.act_static_scale is False and filled.act_calibration_method == 'absmax'
  r = qconfig.QuantizationRule()
  assert (r.module_path, r.weight_qtype, r.act_qtype, r.tile_size, r.weight_calibration_method, tuple(r.act_batch_axes)) == ('.*', None, None, None, 'absmax', (0,))


def test_qarray_array_methods_follow_the_reference_table():
  """qarray_test.py:228-302: scale shapes under reshape / transpose / slicing of a (2, 2, 6) array quantized
  channelwise on axis 0 with tiles of 2 on axis 2 (scale (2, 1, 3))."""
  import torch
  from qwix_amd.core import qarray
  q = qarray.QArray(torch.arange(24, dtype=torch.int8).reshape(2, 2, 6),
                    torch.arange(1, 7, dtype=torch.float32).reshape(2, 1, 3), None, 'int8')
  assert q.shape == (2, 2, 6) and q.ndim == 3
  assert q.scale_tile_shape == (1, 2, 2) and q.zero_point_tile_shape is None
  r = q.reshape(4, 1, 3, 2)
  assert tuple(r.shape) == (4, 1, 3, 2) and tuple(r.scale.shape) == (2, 1, 3, 1)
  assert tuple(q.reshape(2, 1, 2, 6).scale.shape) == (2, 1, 1, 3)
  assert tuple(q.reshape(1, 4, 6).scale.shape) == (1, 2, 3)
  assert tuple(r.reshape(4, 6).scale.shape) == (2, 3)
  assert tuple(q.reshape((4, 6)).shape) == (4, 6) and tuple(q.reshape((4, 6)).scale.shape) == (2, 3)
  with pytest.raises(ValueError):  # (2, 2, 6) -> (12, 2) would merge the tiled axis
    q.reshape(12, 2)
  with pytest.raises(ValueError):
    q.reshape(5, 5)
  with pytest.raises(ValueError):  # the tiled axis cannot be merged with its neighbour
    qarray.QArray(torch.zeros(2, 2, 6, dtype=torch.int8), torch.ones(1, 2, 2), None, 'int8').reshape(4, 6)
  t = q.transpose(1, 2, 0)
  assert tuple(t.shape) == (2, 6, 2) and tuple(t.scale.shape) == (1, 3, 2)
  assert tuple(q.T.shape) == (6, 2, 2) and tuple(q.T.scale.shape) == (3, 1, 2)
  assert tuple(q.mT.shape) == (2, 6, 2) and tuple(q.mT.scale.shape) == (2, 3, 1)
  s = q[..., 1]
  assert tuple(s.shape) == (2, 2) and tuple(s.scale.shape) == (2, 1)
  assert torch.equal(s.qvalue, q.qvalue[..., 1]) and torch.equal(s.scale, q.scale[..., 0])
  assert tuple(q[0:1, 1:2, 4].scale.shape) == (1, 1) and q[0:1, 1:2, 4].scale.item() == 3.0
  assert tuple(q[0].scale.shape) == (1, 3)
  assert tuple(q[..., None].scale.shape) == (2, 1, 3, 1)
  assert tuple(q[None].scale.shape) == (1, 2, 1, 3)
  with pytest.raises(ValueError, match='Unsupported indexing'):
    q[:, :, 1:3]
  sw = q.swapaxes(1, 2)
  assert tuple(sw.shape) == (2, 6, 2) and tuple(sw.scale.shape) == (2, 3, 1)
  assert q.astype(torch.bfloat16).scale.dtype == torch.bfloat16
  with pytest.raises(ValueError):
    qarray.validate_qarray(qarray.QArray(torch.ones(10, 10, dtype=torch.int8), torch.ones(10, 3), None, 'int8'))
  assert qarray.get_tiled_axes(qarray.QArray(torch.ones(10, 256, 16, dtype=torch.int8), torch.ones(10, 8, 2))) == {1: 32, 2: 8}


def test_simple_moving_average_statistics():
  """averaging.py:38-99: float32 sums whatever the calibration dtype, plain average, the default calibration
  while no more than bootstrap_steps samples have been seen."""
  import torch
  from qwix_amd import averaging
  agg = averaging.SimpleMovingAverage()
  cal = {'min': torch.tensor([[-1.0]], dtype=torch.bfloat16), 'max': torch.tensor([[3.0]], dtype=torch.bfloat16)}
  stat = agg.init(cal)
  assert stat['count'].dtype == torch.int32 and int(stat['count']) == 0
  assert stat['sum_of_min'].dtype == torch.float32 and stat['sum_of_max'].shape == (1, 1)
  stat = agg.update(stat, cal)
  stat = agg.update(stat, {'min': torch.tensor([[-3.0]], dtype=torch.bfloat16), 'max': torch.tensor([[4.0]], dtype=torch.bfloat16)})
  got = agg.get_calibration(stat)
  assert int(stat['count']) == 2 and got['min'].item() == -2.0 and got['max'].item() == 3.5
  with pytest.raises(ValueError, match='Shape mismatch'):
    agg.update(stat, {'min': torch.zeros(2, 1), 'max': torch.zeros(2, 1)})
  boot = averaging.SimpleMovingAverage(bootstrap_steps=2)
  assert boot.get_calibration(stat, cal)['max'].item() == 3.0            # 2 samples: still the default
  stat = agg.update(stat, cal)
  out = boot.get_calibration(stat, cal)
  assert out['max'].dtype == torch.bfloat16 and abs(out['max'].item() - 10.0 / 3) < 0.02


def test_provider_pass_through_honours_batch_axes():
  """An op that no rule covers (or whose rule has no weight_qtype) is the float lax.dot_general, batch axes
  included (boxed_param.py:119-127): (2,3,4) x (2,5,4) over batch 0 gives (2,3,5), not (2,3,2,5)."""
  from qwix_amd.providers import ptq
  g = torch.Generator().manual_seed(0)
  a, b = torch.randn(2, 3, 4, generator=g), torch.randn(2, 5, 4, generator=g)
  dn = (((2,), (2,)), ((0,), (0,)))
  want = torch.einsum('bik,bjk->bij', a, b)
  out = ptq.PtqProvider([]).dot_general(a, b, dn)
  assert out.shape == (2, 3, 5) and torch.allclose(out, want, atol=1e-6)
  # a rule exists but does not match this module path; and a rule that matches but quantizes nothing
  for rules in ([qconfig.QuantizationRule(module_path='elsewhere', weight_qtype='int8')],
                [qconfig.QuantizationRule(module_path='.*', weight_qtype=None)]):
    with qconfig.module_scope('attn'):
      out = ptq.PtqProvider(rules).dot_general(a, b, dn, preferred_element_type=torch.bfloat16)
    assert out.dtype == torch.bfloat16 and out.shape == (2, 3, 5)
    assert torch.allclose(out.float(), want, atol=2e-2, rtol=2e-2)
  # several batch axes, batch axes not leading, two contracting axes: layout (batch..., lhs free..., rhs free...)
  a, b = torch.randn(3, 2, 4, 5, generator=g), torch.randn(5, 4, 6, 2, 3, generator=g)
  dn = (((2, 3), (1, 0)), ((1, 0), (3, 4)))
  out = dg.float_dot_general(a, b, dn)
  assert torch.allclose(out, torch.einsum('cbkl,lknbc->bcn', a, b), atol=1e-5)
  with pytest.raises(TypeError, match='differ'):
    dg.float_dot_general(torch.zeros(2, 3), torch.zeros(4, 3), (((0,), (0,)), ((), ())))


def test_own_kernel_size_limits_are_decided_in_python():
  """The routes onto this library's kernels are chosen from the kernels' own address limits, so that a call beyond
  them takes the dequantize + float GEMM route instead of raising from the C layer."""
  from qwix_amd.core import dot_general as dg
  # decode kernel: 31-bit lane offsets over 32 activation rows, 64 weight rows and all scales
  assert dg._decode_kernel_limits_ok(4096, 4096, 14336, 4096, 128, False, 4)
  assert dg._decode_kernel_limits_ok(4096, 2048, 14336, 4096, 128, True, 4)
  assert not dg._decode_kernel_limits_ok(1 << 25, 4096, 14336, 4096, 128, False, 4)        # activation pitch
  assert not dg._decode_kernel_limits_ok(1 << 25, 1 << 25, 64, 1 << 25, 128, False, 4)     # weight rows
  assert not dg._decode_kernel_limits_ok(8192, 8192, 1 << 24, 8192, 128, False, 4)         # scale array
  # bf16 tile GEMMs: each operand inside 2 GiB (a language-model head: vocabulary 131072 x K 8192 bf16 is exactly 2 GiB)
  assert dg._bf16_gemm_limits_ok(2048, 4096, 14336, 8192)
  assert not dg._bf16_gemm_limits_ok(512, 8192, 131072, 2 * 8192)
  assert not dg._bf16_gemm_limits_ok(1 << 20, 4096, 4096, 8192)
  # an activation view that starts inside a 16-byte unit or has a ragged pitch is copied, others pass through
  x = torch.zeros(4, 264, dtype=torch.bfloat16)
  assert dg._aligned_rows(x) is x
  assert dg._aligned_rows(x[:, 8:]) is not None and dg._aligned_rows(x[:, 8:]).data_ptr() == x[:, 8:].data_ptr()
  y = dg._aligned_rows(x[:, 3:259])
  assert y.data_ptr() % 16 == 0 and y.is_contiguous() and y.shape == (4, 256)


def test_weight_signature_sees_in_place_updates():
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  q = torch.zeros(8, 4, dtype=torch.int8)
  s = torch.ones(1, 4)
  z = torch.zeros(1, 4, dtype=torch.int8)
  w = qarray.QArray(q, s, z, 'int8')
  a = dg._weight_signature(w)
  assert a == dg._weight_signature(w)
  q.add_(1)
  b = dg._weight_signature(w)
  assert b != a
  s.mul_(2.0)
  c = dg._weight_signature(w)
  assert c != b
  z.add_(1)
  assert dg._weight_signature(w) != c
  p = qarray.Int4Tensor(torch.zeros(8, 2, dtype=torch.uint8), (8, 4), 1)
  w4 = qarray.QArray(p, s, None, 'int4')
  a4 = dg._weight_signature(w4)
  p.data.add_(1)
  assert dg._weight_signature(w4) != a4
