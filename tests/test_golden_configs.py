"""The five benchmark configurations at reduced shapes against the committed vectors in
tests/golden/config_vectors.npz (written by tests/golden/make_fixtures.py from the CPU oracle).

CPU: the oracle still reproduces the file.  GPU: the HIP path reproduces it -- quantized values,
scales and int32 accumulators bit for bit; int8 outputs bit for bit; fp8 and rotated outputs within the
tolerances stated in the tests."""
import os

import numpy as np
import pytest

from oracle import qwix_oracle as O
from tests.golden import make_fixtures as mf

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'config_vectors.npz')
DN = (((1,), (0,)), ((), ()))


@pytest.fixture(scope='module')
def vec():
  return dict(np.load(PATH))


def test_oracle_reproduces_committed_vectors(vec):
  now = mf.oracle_vectors()
  assert sorted(now) == sorted(vec)
  for k, v in now.items():
    assert np.array_equal(np.asarray(v), vec[k]), k


def _check_q(qa, vec, prefix):
  from tests import util
  assert np.array_equal(util.qvalues_np(qa), vec[prefix + '_q']), prefix + ' qvalues'
  assert np.array_equal(util.f32np(qa.scale), vec[prefix + '_s']), prefix + ' scales'


@pytest.mark.gpu
def test_c1_mlp_int8(vec):
  import torch
  from tests import util
  from qwix_amd.core import dot_general as dg, qarray
  i = mf.config_inputs('c1')
  wh = qarray.HowToQuantize(qtype='int8', channelwise_axes=[1])
  ah = qarray.HowToQuantize(qtype='int8', channelwise_axes=[0])
  w1, w2 = qarray.quantize(util.to_gpu(i['w1'], O.F32), wh), qarray.quantize(util.to_gpu(i['w2'], O.F32), wh)
  xq = qarray.quantize(util.to_gpu(i['x'], O.F32), ah)
  h, acc1 = dg._fast_dot_general(xq, w1, DN, return_accumulators=True)
  hq = qarray.quantize(torch.relu(h), ah)
  y, acc2 = dg._fast_dot_general(hq, w2, DN, return_accumulators=True)
  _check_q(w1, vec, 'c1_w1'); _check_q(w2, vec, 'c1_w2'); _check_q(xq, vec, 'c1_x'); _check_q(hq, vec, 'c1_h')
  assert np.array_equal(acc1.cpu().numpy(), vec['c1_acc1']) and np.array_equal(acc2.cpu().numpy(), vec['c1_acc2'])
  assert np.array_equal(util.f32np(y), vec['c1_out'])


@pytest.mark.gpu
def test_c2_weight_only_int4(vec):
  import torch
  from tests import util
  from qwix_amd.core import dot_general as dg, qarray
  i = mf.config_inputs('c2')
  wq = qarray.quantize_api(util.to_gpu(i['w'], O.BF16), 'int4', channelwise_axes=[1], tiled_axes={0: 128},
                           scale_dtype=torch.float32)
  _check_q(wq, vec, 'c2_w')
  out = dg.dot_general(util.to_gpu(i['x'], O.BF16), wq, DN, preferred_element_type=torch.bfloat16)
  # the reference dequantizes the weight to f32 and rounds the dot once; the kernel scales each
  # group's exact partial sum instead: equal up to bf16 output rounding (rtol 1e-2 of the north star)
  want = vec['c2_out']
  assert np.allclose(util.f32np(out), want, rtol=1e-2, atol=1e-2 * np.abs(want).mean())


@pytest.mark.gpu
@pytest.mark.parametrize('name,qt', [('c3', 'int8'), ('c4', 'float8_e4m3fn')])
def test_c3_c4_dynamic_range_w8a8(vec, name, qt):
  from tests import util
  from qwix_amd.core import dot_general as dg, qarray
  i = mf.config_inputs(name)
  xq = qarray.quantize(util.to_gpu(i['x'], O.BF16), qarray.HowToQuantize(qtype=qt, channelwise_axes=[0]))
  wq = qarray.quantize(util.to_gpu(i['w'], O.BF16), qarray.HowToQuantize(qtype=qt, channelwise_axes=[1]))
  _check_q(xq, vec, name + '_x'); _check_q(wq, vec, name + '_w')
  if qt == 'int8':
    out, acc = dg._fast_dot_general(xq, wq, DN, return_accumulators=True)
    assert np.array_equal(acc.cpu().numpy(), vec['c3_acc'])
    assert np.array_equal(util.f32np(out), vec['c3_out'])
  else:
    out = dg.dot_general(xq, wq, DN)
    want = vec['c4_out']   # f32 accumulation order differs from the exact sum: bf16 tolerance
    assert np.allclose(util.f32np(out), want, rtol=1e-2, atol=1e-2 * np.abs(want).mean())


@pytest.mark.gpu
def test_c5_hadamard_a8w4(vec):
  import torch
  from tests import util
  from qwix_amd.contrib import hadamard_rot as hr
  from qwix_amd.core import dot_general as dg, qarray
  i = mf.config_inputs('c5')
  x, w = util.to_gpu(i['x'], O.BF16), util.to_gpu(i['w'], O.BF16)
  signs = torch.from_numpy(i['signs']).to(torch.bfloat16).to(util.DEV)
  xr = hr.fwht(x, 1, signs, None, 1.0)            # what hadamard_rotate_inputs does with row signs `signs`
  wr = hr.fwht(w, 0, signs, None, 1.0 / 256)
  # the transform sums in f32 in butterfly order, the oracle exactly: equal up to one bf16 rounding
  for got, want in ((xr, vec['c5_xrot']), (wr, vec['c5_wrot'])):
    assert np.allclose(util.f32np(got), want, rtol=2.0 ** -7, atol=2.0 ** -7 * np.abs(want).max())
  # downstream stages on the oracle's rotated arrays: exact again
  xq = qarray.quantize(util.to_gpu(vec['c5_xrot'], O.BF16), qarray.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  wq = qarray.quantize(util.to_gpu(vec['c5_wrot'], O.BF16),
                       qarray.HowToQuantize(qtype='int4', channelwise_axes=[1], tiled_axes={0: 128}))
  _check_q(xq, vec, 'c5_x'); _check_q(wq, vec, 'c5_w')
  out, acc = dg._fast_dot_general(xq, wq, DN, exact=True, return_accumulators=True)
  assert np.array_equal(acc.cpu().numpy(), vec['c5_acc'])
  assert np.array_equal(util.f32np(out), vec['c5_out'])
  # the kernel dot_general runs by default (and bench.py times): the same int32 partials bit for bit, its
  # f32 sum of the scaled partials within the north-star tolerance of the reference's bf16-rounded sum
  out, acc = dg._fast_dot_general(xq, wq, DN, exact=False, return_accumulators=True)
  assert np.array_equal(acc.cpu().numpy(), vec['c5_acc'])
  want = vec['c5_out']
  owq = O.QArray(vec['c5_w_q'], O.FArr(vec['c5_w_s'], O.BF16), None, 'int4')
  oxq = O.QArray(vec['c5_x_q'], O.FArr(vec['c5_x_s'], O.BF16), None, 'int8')
  env = util.partials_envelope(vec['c5_acc'], oxq, owq)
  for got in (out, dg.dot_general(xq, wq, DN)):   # the run that dumped, and the plain run that bench.py times
    assert np.all(np.abs(util.f32np(got) - want) <= 1e-2 * np.abs(want) + env)
