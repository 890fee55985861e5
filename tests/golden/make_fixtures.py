"""Writes tests/golden/config_vectors.npz: the oracle's results for the five benchmark configurations at
reduced shapes.

  python tests/golden/make_fixtures.py          (from the repository root, CPU only)

Inputs are not stored: they come from numpy.random.Generator(PCG64(seed)) through tests/util.make_np, and
the tests regenerate them.  Stored are the quantized values, scales, int32 accumulators and outputs that
the CPU restatement of the reference produces, so that (a) a change of the oracle shows up as a diff of
this file and (b) the GPU tests have fixed vectors to hit besides the oracle itself.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import qwix_oracle as O  # noqa: E402
from tests import util  # noqa: E402

DN = (((1,), (0,)), ((), ()))


def config_inputs(name):
  """Seeded inputs of the reduced configurations (shared with tests/test_golden_configs.py)."""
  if name == 'c1':   # PTQ MLP, f32, int8 weights and activations
    return dict(x=util.make_np((16, 64), O.F32, 1001, dist='uniform'), w1=util.make_np((64, 128), O.F32, 1002, 0.02),
                w2=util.make_np((128, 32), O.F32, 1003, 0.02))
  if name == 'c2':   # weight-only int4 g128 GEMV, bf16 activations, f32 scales
    return dict(x=util.make_np((8, 256), O.BF16, 2001), w=util.make_np((256, 128), O.BF16, 2002, 0.02))
  if name in ('c3', 'c4'):   # dynamic-range w8a8, int8 / fp8
    base = 3000 if name == 'c3' else 4000
    return dict(x=util.make_np((64, 256), O.BF16, base + 1), w=util.make_np((256, 128), O.BF16, base + 2, 0.02))
  if name == 'c5':   # Hadamard-rotated a8w4 g128 with 1 % outlier channels
    x = util.make_np((32, 256), O.BF16, 5001)
    idx = util.rng(5003).choice(256, 3, replace=False)
    x[:, idx] *= 50.0
    x = O.round_to_bf16(x)
    signs = util.rng(5004).choice([-1.0, 1.0], 256).astype(np.float32)
    return dict(x=x, w=util.make_np((256, 128), O.BF16, 5002, 0.02), signs=signs)
  raise KeyError(name)


def _q(out, prefix, qa):
  out[prefix + '_q'] = np.asarray(qa.qvalue)
  out[prefix + '_s'] = np.asarray(qa.scale.v, np.float32)


def oracle_vectors():
  out = {}
  # C1
  i = config_inputs('c1')
  wh = O.HowToQuantize(qtype='int8', channelwise_axes=[1])
  ah = O.HowToQuantize(qtype='int8', channelwise_axes=[0])
  w1, w2 = O.quantize(O.FArr(i['w1'], O.F32), wh), O.quantize(O.FArr(i['w2'], O.F32), wh)
  xq = O.quantize(O.FArr(i['x'], O.F32), ah)
  h, acc1 = O.fast_dot_general(xq, w1, DN, return_acc=True)
  hr = O.FArr(np.maximum(h.v, 0.0).astype(np.float32), O.F32)
  hq = O.quantize(hr, ah)
  y, acc2 = O.fast_dot_general(hq, w2, DN, return_acc=True)
  _q(out, 'c1_w1', w1); _q(out, 'c1_w2', w2); _q(out, 'c1_x', xq); _q(out, 'c1_h', hq)
  out['c1_acc1'], out['c1_acc2'], out['c1_out'] = acc1, acc2, y.v
  # C2
  i = config_inputs('c2')
  wq = O.quantize_api(O.FArr(i['w'], O.BF16), 'int4', channelwise_axes=[1], tiled_axes={0: 128}, scale_dtype=O.F32)
  _q(out, 'c2_w', wq)
  out['c2_out'] = O.dot_general(O.FArr(i['x'], O.BF16), wq, DN, O.BF16).v
  # C3 / C4
  for name, qt in (('c3', 'int8'), ('c4', 'float8_e4m3fn')):
    i = config_inputs(name)
    xq = O.quantize(O.FArr(i['x'], O.BF16), O.HowToQuantize(qtype=qt, channelwise_axes=[0]))
    wq = O.quantize(O.FArr(i['w'], O.BF16), O.HowToQuantize(qtype=qt, channelwise_axes=[1]))
    _q(out, name + '_x', xq); _q(out, name + '_w', wq)
    if qt == 'int8':
      y, acc = O.fast_dot_general(xq, wq, DN, return_acc=True)
      out[name + '_acc'] = acc
    else:
      y = O.dot_general(xq, wq, DN)
    out[name + '_out'] = y.v
  # C5
  i = config_inputs('c5')
  xr, wr = O.hadamard_rotate_inputs(O.FArr(i["x"], O.BF16), O.FArr(i["w"], O.BF16), i["signs"], None,
                                      lhs_reduction_dim=1, rhs_reduction_dim=0)
  out['c5_xrot'], out['c5_wrot'] = xr.v, wr.v
  xq = O.quantize(xr, O.HowToQuantize(qtype='int8', channelwise_axes=[0]))
  wq = O.quantize(wr, O.HowToQuantize(qtype='int4', channelwise_axes=[1], tiled_axes={0: 128}))
  _q(out, 'c5_x', xq); _q(out, 'c5_w', wq)
  y, acc = O.fast_dot_general(xq, wq, DN, return_acc=True)
  out['c5_acc'], out['c5_out'] = acc, y.v
  return out


if __name__ == '__main__':
  path = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'config_vectors.npz')
  vec = oracle_vectors()
  np.savez_compressed(path, **vec)
  print(f'wrote {path}: {len(vec)} arrays, {os.path.getsize(path)} bytes')
