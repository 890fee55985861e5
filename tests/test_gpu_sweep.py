"""GPU parity: seeded random sweeps of the Python surface against the CPU oracle.

Each sweep draws shapes, dtypes, qtypes and scale layouts from a PCG64 stream, runs the product path and the oracle on
the same inputs and holds the result to the bar of its kind: bit for bit where the arithmetic is integer sums followed
by an elementwise epilogue, the stated tolerance where a float accumulation order is free (fp8 dots, the
dequantize-first path, f32 sums of per-group partials).  Where the oracle raises, the product has to raise the same
type.  A failing case prints its parameters; all failures of a sweep are reported together."""
import numpy as np
import pytest
import torch

from oracle import qwix_oracle as O
from tests import util

pytestmark = pytest.mark.gpu
DN = (((1,), (0,)), ((), ()))
TD = {O.F32: torch.float32, O.BF16: torch.bfloat16}


def _rel(got, want):
  return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-9))


def _exact(got, want):
  assert got.shape == want.shape, (got.shape, want.shape)
  bad = np.flatnonzero(got.ravel() != want.ravel())
  assert bad.size == 0, f'{bad.size} of {got.size} differ (max rel {_rel(got, want):.3g}): {got.ravel()[bad[:4]]} vs {want.ravel()[bad[:4]]}'


def _run(cases):
  """cases: iterable of (description, thunk).  Runs all, reports every failure."""
  failures = []
  n = 0
  for what, thunk in cases:
    n += 1
    print('case', what, flush=True)
    try:
      thunk()
      torch.cuda.synchronize()
    except Exception as e:  # noqa: BLE001 -- collected and re-raised below
      failures.append(f'{what}: {type(e).__name__}: {str(e)[:300]}')
  assert n > 0
  assert not failures, f'{len(failures)} of {n} cases failed:\n' + '\n'.join(failures)


def _same_outcome(oracle_fn, product_fn):
  """Both succeed (returns the two results) or both raise the same exception type (returns None)."""
  try:
    want, oerr = oracle_fn(), None
  except Exception as e:  # noqa: BLE001
    want, oerr = None, e
  try:
    got, err = product_fn(), None
  except Exception as e:  # noqa: BLE001
    got, err = None, e
  if oerr is not None or err is not None:
    assert type(oerr) is type(err), f'oracle raised {oerr!r}, product raised {err!r}'
    return None
  return got, want


# ---------------------------------------------------------------------------------------------------------------
# quantize / dequantize patterns (qarray.py:470-708)
# ---------------------------------------------------------------------------------------------------------------


def _quantize_cases(seed, count):
  from qwix_amd.core import qarray
  r = util.rng(seed)
  for c in range(count):
    nd = int(r.choice([1, 2, 2, 3, 4]))
    shape = tuple(int(r.choice([1, 2, 3, 5, 8, 16, 24, 48, 64, 96, 128, 200, 256])) for _ in range(nd))
    dt = O.BF16 if r.random() < 0.6 else O.F32
    qt = str(r.choice(['int8', 'int4', O.E4M3]))
    cw = [a for a in range(nd) if r.random() < 0.4]
    tiled = {}
    for a in range(nd):
      if a not in cw and r.random() < 0.3:
        tiled[a] = int(r.choice([d for d in (1, 2, 4, 8, 16, 32, 64, 128) if shape[a] % d == 0]))
    calib = str(r.choice(['absmax', 'absmax', 'minmax', 'absmax,0.9'])) if qt != O.E4M3 else 'absmax'
    if np.prod(shape) > 4_000_000 or (qt == 'int4' and all(d % 2 for d in shape)):
      continue  # packed int4 storage pairs the elements of an axis of even length

    def thunk(shape=shape, dt=dt, qt=qt, cw=cw, tiled=tiled, calib=calib, c=c):
      x_np, x_t = util.make(shape, dt, seed=100 + c)
      if calib == 'minmax':
        x_np = O.rnd(x_np + 0.4, dt)
        x_t = util.to_gpu(x_np, dt)
      how = dict(qtype=qt, channelwise_axes=cw, tiled_axes=tiled, calibration_method=calib)
      res = _same_outcome(lambda: O.quantize(O.FArr(x_np, dt), O.HowToQuantize(**how)),
                          lambda: qarray.quantize(x_t, qarray.HowToQuantize(**how)))
      if res is None:
        return
      q, oq = res
      util.assert_qarray_equal(q, oq, 'q')
      assert np.array_equal(util.f32np(qarray.dequantize(q)), O.dequantize(oq).v), 'dequantize differs'

    yield f'quantize shape={shape} {dt} {qt} cw={cw} tiled={tiled} {calib}', thunk


@pytest.mark.parametrize('seed', [3, 5, 9])
def test_sweep_quantize_patterns(seed):
  _run(_quantize_cases(seed, 200))


def _static_cases(seed, count):
  from qwix_amd.core import qarray
  r = util.rng(seed)
  for c in range(count):
    nd = int(r.choice([2, 3]))
    shape = tuple(int(r.choice([2, 8, 16, 64, 128, 256])) for _ in range(nd))
    qt = str(r.choice(['int8', 'int4', O.E4M3]))
    sshape = tuple(int(r.choice([d for d in (1, 2, 4, s) if s % d == 0])) for s in shape)
    asym = qt != O.E4M3 and r.random() < 0.4
    dt = O.BF16 if r.random() < 0.7 else O.F32
    if qt == 'int4' and (np.prod(shape) // np.prod(sshape)) % 2:
      continue  # one int4 value per scale

    def thunk(shape=shape, sshape=sshape, qt=qt, asym=asym, dt=dt, c=c):
      x_np, x_t = util.make(shape, dt, seed=c)
      s_np = (np.abs(util.make_np(sshape, dt, seed=c + 5)) * 0.02 + 0.005).astype(np.float32)
      if dt == O.BF16:
        s_np = O.round_to_bf16(s_np)
      z_np = util.rng(c).integers(-20, 20, sshape).astype(np.int8) if asym else None
      z_t = None if z_np is None else torch.from_numpy(z_np).to(util.DEV)
      res = _same_outcome(lambda: O.quantize_with_scale_zero_point(O.FArr(x_np, dt), qt, O.FArr(s_np, dt), z_np),
                          lambda: qarray.quantize_with_scale_zero_point(x_t, qt, util.to_gpu(s_np, dt), z_t))
      if res is None:
        return
      q, oq = res
      util.assert_qarray_equal(q, oq, 'static')
      assert np.array_equal(util.f32np(qarray.dequantize(q)), O.dequantize(oq).v), 'dequantize differs'
      nd_ = len(shape)
      how = dict(qtype=qt, channelwise_axes=[a for a in range(nd_) if sshape[a] == shape[a]],
                 tiled_axes={a: shape[a] // sshape[a] for a in range(nd_) if 1 < sshape[a] < shape[a]},
                 calibration_method='minmax' if asym else 'absmax')
      got, want = qarray.calibrate(x_t, qarray.HowToQuantize(**how)), O.calibrate(O.FArr(x_np, dt), O.HowToQuantize(**how))
      for k in want:
        assert np.array_equal(util.f32np(got[k]), want[k].v), 'calibrate ' + k

    yield f'static shape={shape} scales={sshape} {qt} asym={asym} {dt}', thunk


def test_sweep_static_scales_and_calibrate():
  _run(_static_cases(13, 120))


# ---------------------------------------------------------------------------------------------------------------
# dot_general on 2-D operands (dot_general.py:135-275, 407-491)
# ---------------------------------------------------------------------------------------------------------------


def _dot_cases(seed, count):
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  r = util.rng(seed)
  for c in range(count):
    kind = str(r.choice(['pc', 'pc', 'tiled', 'w4', 'asym', 'f8', 'wo']))
    M = int(r.choice([1, 3, 8, 16, 17, 31, 33, 64, 100, 128, 200, 256, 300, 513]))
    kq = int(r.choice([1, 2, 3, 4, 5, 8, 9, 16]))
    kb = int(r.choice([16, 32, 64, 128, 128, 256]))
    K = kq * kb
    N = int(r.choice([8, 16, 24, 40, 64, 72, 128, 136, 256, 264, 520, 1024]))
    dt = O.BF16 if r.random() < 0.7 else O.F32
    tile, aq, wqt, calib_a, calib_w = None, 'int8', 'int8', 'absmax', 'absmax'
    if kind == 'tiled':
      tile = kb
    elif kind == 'w4':
      wqt = 'int4'
      tile = kb if r.random() < 0.6 else None
    elif kind == 'asym':
      calib_a = 'minmax' if r.random() < 0.5 else 'absmax'
      calib_w = 'absmax' if calib_a == 'minmax' else 'minmax'
      tile = kb if r.random() < 0.3 else None
    elif kind == 'f8':
      aq = wqt = O.E4M3
    elif kind == 'wo':
      wqt = str(r.choice(['int8', 'int4']))
      tile = kb if r.random() < 0.7 else None

    def thunk(kind=kind, M=M, K=K, N=N, dt=dt, tile=tile, aq=aq, wqt=wqt, calib_a=calib_a, calib_w=calib_w, c=c):
      x_np, x_t = util.make((M, K), dt, seed=1000 + c)
      w_np, w_t = util.make((K, N), dt, seed=5000 + c, scale=0.05)
      if calib_a == 'minmax':
        x_np = O.rnd(x_np + 0.7, dt)
        x_t = util.to_gpu(x_np, dt)
      hw = dict(qtype=wqt, channelwise_axes=[1], tiled_axes={0: tile} if tile else {}, calibration_method=calib_w)
      ha = dict(qtype=aq, channelwise_axes=[0], tiled_axes={1: tile} if tile else {}, calibration_method=calib_a)
      wq, owq = qarray.quantize(w_t, qarray.HowToQuantize(**hw)), O.quantize(O.FArr(w_np, dt), O.HowToQuantize(**hw))
      util.assert_qarray_equal(wq, owq, 'rhs')
      loose = 2e-2 if dt == O.BF16 else 1e-4
      if kind == 'wo':
        got = util.f32np(dg.dot_general(x_t, wq, DN))
        assert _rel(got, O.dot_general(O.FArr(x_np, dt), owq, DN).v) < loose
        return
      xq, oxq = qarray.quantize(x_t, qarray.HowToQuantize(**ha)), O.quantize(O.FArr(x_np, dt), O.HowToQuantize(**ha))
      util.assert_qarray_equal(xq, oxq, 'lhs')
      got, want = util.f32np(dg.dot_general(xq, wq, DN)), O.dot_general(oxq, owq, DN).v
      if kind == 'f8':
        assert _rel(got, want) < loose
      elif tile and K // tile > 1:
        # several groups: f32 sums of partials (default mode keeps them unrounded), or the float path below 128
        assert _rel(got, want) < (2e-2 if dt == O.BF16 else 1e-5)
      else:
        _exact(got, want)

    yield f'dot {kind} M={M} K={K} N={N} tile={tile} {dt} a={aq}/{calib_a} w={wqt}/{calib_w}', thunk


@pytest.mark.parametrize('seed', [7, 11])
def test_sweep_dot_general_2d(seed):
  _run(_dot_cases(seed, 150))


def _combo_cases(seed, count):
  """tile_size through get_how_to_quantize, scale_dtype, preferred_element_type, int4 on either side; exact mode."""
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  r = util.rng(seed)
  for c in range(count):
    dt = O.BF16 if r.random() < 0.7 else O.F32
    M = int(r.choice([1, 4, 16, 33, 100, 256, 384]))
    K = int(r.choice([64, 128, 256, 512, 1024, 384]))
    N = int(r.choice([16, 72, 128, 256, 520]))
    lq = str(r.choice(['int8', 'int8', 'int4', O.E4M3]))
    rq = lq if lq == O.E4M3 else str(r.choice(['int8', 'int4']))
    tile = r.choice([None, None, 128, 64, 256, 32])
    tile = None if tile is None or K % int(tile) else int(tile)
    sdt = r.choice([None, None, O.F32, O.BF16])
    pet = r.choice([None, None, O.F32, O.BF16])

    def thunk(dt=dt, M=M, K=K, N=N, lq=lq, rq=rq, tile=tile, sdt=sdt, pet=pet, c=c):
      x_np, x_t = util.make((M, K), dt, seed=c)
      w_np, w_t = util.make((K, N), dt, seed=c + 999, scale=0.05)
      kw = dict(dimension_numbers=DN, ndims=(2, 2), tile_size=tile)

      def both(t, n, for_lhs, qtype):
        h = dg.get_how_to_quantize(for_lhs=for_lhs, qtype=qtype, **kw)
        oh = O.dg_get_how_to_quantize(for_lhs=for_lhs, qtype=qtype, **kw)
        q = qarray.quantize_api(t, h.qtype, channelwise_axes=h.channelwise_axes, tiled_axes=h.tiled_axes,
                                scale_dtype=None if sdt is None else TD[sdt])
        oq = O.quantize_api(O.FArr(n, dt), oh.qtype, channelwise_axes=oh.channelwise_axes, tiled_axes=oh.tiled_axes,
                            scale_dtype=sdt)
        util.assert_qarray_equal(q, oq, 'operand')
        return q, oq

      xq, oxq = both(x_t, x_np, True, lq)
      wq, owq = both(w_t, w_np, False, rq)
      out = dg.dot_general(xq, wq, DN, preferred_element_type=None if pet is None else TD[pet], exact=True)
      want = O.dot_general(oxq, owq, DN, preferred_element_type=pet)
      assert out.dtype == TD[want.dtype], (out.dtype, want.dtype)
      got = util.f32np(out)
      if lq == O.E4M3:
        assert _rel(got, want.v) < (2e-2 if out.dtype == torch.bfloat16 else 2e-3)
      elif tile and tile < 128 and K // tile > 1:
        # the dequantize-first path: a float dot whose accumulation order is free
        assert _rel(got, want.v) < (4e-3 if out.dtype == torch.bfloat16 else 1e-5)
      elif tile and K // tile > 1 and want.dtype == O.F32:
        assert _rel(got, want.v) < 1e-5  # f32 sum of the per-group partials: order free
      else:
        _exact(got, want.v)

    yield f'combo M={M} K={K} N={N} {lq}x{rq} tile={tile} {dt} scale_dtype={sdt} pet={pet}', thunk


@pytest.mark.parametrize('seed', [3, 4])
def test_sweep_dot_general_types_and_tiles(seed):
  _run(_combo_cases(seed, 150))


# ---------------------------------------------------------------------------------------------------------------
# weight-only: float activations against a quantized weight, the dequantize-first path (dot_general.py:264-275)
# ---------------------------------------------------------------------------------------------------------------


def _weight_only_cases(seed, count):
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  r = util.rng(seed)
  for c in range(count):
    dt = O.BF16 if r.random() < 0.85 else O.F32
    lead = [int(r.choice([1, 2, 3, 5, 8, 17, 33, 40, 50, 64, 100, 130, 300])) for _ in range(int(r.choice([1, 1, 2])))]
    if int(np.prod(lead)) > 700:
      lead = lead[:1]
    K = int(r.choice([256, 512, 1024, 2048, 3072, 4096, 6144]))
    N = int(r.choice([48, 64, 136, 520, 1024, 2048]))
    wt = str(r.choice(['int4', 'int8', O.E4M3]))
    g = int(r.choice([0, 64, 128, 256, 512, 1024]))
    g = 0 if g and K % g else g
    asym = wt != O.E4M3 and r.random() < 0.3
    sdt, pet = r.choice([None, O.F32, O.BF16]), r.choice([None, O.F32, O.BF16])

    def thunk(lead=lead, K=K, N=N, wt=wt, g=g, asym=asym, dt=dt, sdt=sdt, pet=pet, c=c):
      x_np, x_t = util.make(tuple(lead) + (K,), dt, seed=c)
      w_np, w_t = util.make((K, N), dt, seed=c + 999, scale=0.05)
      if asym:
        w_np = O.rnd(w_np + 0.02, dt)
        w_t = util.to_gpu(w_np, dt)
      dn = (((len(lead),), (0,)), ((), ()))
      kw = dict(channelwise_axes=[1], tiled_axes={0: g} if g else {})
      if asym:
        kw['calibration_method'] = 'minmax'
      wq = qarray.quantize_api(w_t, wt, scale_dtype=None if sdt is None else TD[sdt], **kw)
      owq = O.quantize_api(O.FArr(w_np, dt), wt, scale_dtype=sdt, **kw)
      util.assert_qarray_equal(wq, owq, 'weight')
      out = dg.dot_general(x_t, wq, dn, preferred_element_type=None if pet is None else TD[pet])
      want = O.dot_general(O.FArr(x_np, dt), owq, dn, preferred_element_type=pet)
      assert out.dtype == TD[want.dtype], (out.dtype, want.dtype)
      got = util.f32np(out)
      assert got.shape == want.v.shape, (got.shape, want.v.shape)
      # the decode kernel, the dequantizing tile GEMM (with and without K ranges) or dequantize + GEMM, by the shape:
      # bf16 operands on the matrix cores with f32 sums in the kernel's order.  A weight with f32 scales is rounded to
      # bf16 once more there (2^-9 relative; with one scale per column the same few roundings all along K, so the
      # deviations add up in step: up to 1.2e-2 of the mean magnitude at 300 x 512 x 1024 by construction)
      mag = np.abs(want.v).mean()
      assert np.allclose(got, want.v, rtol=1e-2, atol=2e-2 * mag), np.abs(got - want.v).max() / mag

    yield f'weight-only {lead} K={K} N={N} {wt} group={g} asym={asym} {dt} scale={sdt} result={pet}', thunk


@pytest.mark.parametrize('seed', [11, 12])
def test_sweep_weight_only(seed):
  _run(_weight_only_cases(seed, 80))


# ---------------------------------------------------------------------------------------------------------------
# general dimension numbers: batch axes, several contracting axes, any axis order (dot_general.py:79-132)
# ---------------------------------------------------------------------------------------------------------------


def _dimension_number_cases(seed, count):
  from qwix_amd.core import dot_general as dg
  from qwix_amd.core import qarray
  r = util.rng(seed)
  for c in range(count):
    nb, nc = int(r.choice([0, 0, 1, 2])), int(r.choice([1, 1, 2]))
    nlf, nrf = int(r.choice([0, 1, 1, 2])), int(r.choice([0, 1, 1, 2]))
    bs = [int(r.choice([1, 2, 3])) for _ in range(nb)]
    cs = [int(r.choice([16, 32, 64, 128, 256])) for _ in range(nc)]
    lf = [int(r.choice([1, 5, 16, 40])) for _ in range(nlf)]
    rf = [int(r.choice([2, 8, 24, 64])) for _ in range(nrf)]
    l_axes = [('b', i) for i in range(nb)] + [('c', i) for i in range(nc)] + [('f', i) for i in range(nlf)]
    r_axes = [('b', i) for i in range(nb)] + [('c', i) for i in range(nc)] + [('f', i) for i in range(nrf)]
    l_axes = [l_axes[i] for i in r.permutation(len(l_axes))]
    r_axes = [r_axes[i] for i in r.permutation(len(r_axes))]
    size = lambda kind, i, free: {'b': bs, 'c': cs, 'f': free}[kind][i]
    lshape = tuple(size(k, i, lf) for k, i in l_axes)
    rshape = tuple(size(k, i, rf) for k, i in r_axes)
    dn = ((tuple(l_axes.index(('c', i)) for i in range(nc)), tuple(r_axes.index(('c', i)) for i in range(nc))),
          (tuple(l_axes.index(('b', i)) for i in range(nb)), tuple(r_axes.index(('b', i)) for i in range(nb))))
    dt = O.BF16 if r.random() < 0.7 else O.F32
    lq = str(r.choice(['int8', 'int8', 'int4', O.E4M3]))
    rq = lq if lq == O.E4M3 else str(r.choice(['int8', 'int8', 'int4']))
    tile = int(r.choice([0, 0, 16, 64, 128]))
    if tile and cs[-1] % tile:
      tile = 0
    asym = lq != O.E4M3 and r.random() < 0.2
    if (lq == 'int4' and all(d % 2 for d in lshape)) or (rq == 'int4' and all(d % 2 for d in rshape)):
      continue  # packed int4 storage pairs the elements of an axis of even length

    def thunk(lshape=lshape, rshape=rshape, dn=dn, dt=dt, lq=lq, rq=rq, tile=tile, asym=asym, last_k=cs[-1], c=c):
      x_np, x_t = util.make(lshape, dt, seed=c)
      w_np, w_t = util.make(rshape, dt, seed=c + 999, scale=0.05)
      if asym:
        x_np = O.rnd(x_np + 0.5, dt)
        x_t = util.to_gpu(x_np, dt)
      kw = dict(dimension_numbers=dn, ndims=(len(lshape), len(rshape)), tile_size=tile or None)
      cm = 'minmax' if asym else 'absmax'
      xq = qarray.quantize(x_t, dg.get_how_to_quantize(for_lhs=True, qtype=lq, calibration_method=cm, **kw))
      wq = qarray.quantize(w_t, dg.get_how_to_quantize(for_lhs=False, qtype=rq, **kw))
      oxq = O.quantize(O.FArr(x_np, dt), O.dg_get_how_to_quantize(for_lhs=True, qtype=lq, calibration_method=cm, **kw))
      owq = O.quantize(O.FArr(w_np, dt), O.dg_get_how_to_quantize(for_lhs=False, qtype=rq, **kw))
      util.assert_qarray_equal(xq, oxq, 'lhs')
      util.assert_qarray_equal(wq, owq, 'rhs')
      got, want = util.f32np(dg.dot_general(xq, wq, dn, exact=True)), O.dot_general(oxq, owq, dn).v
      assert got.shape == want.shape, (got.shape, want.shape)
      groups = last_k // tile if tile else 1
      if lq == O.E4M3 or (tile and tile < 128 and groups > 1):
        assert _rel(got, want) < (2e-2 if dt == O.BF16 else 2e-3)
      elif groups > 1 and dt == O.F32:
        assert _rel(got, want) < 1e-5
      else:
        _exact(got, want)

    yield f'dimension numbers {lshape} x {rshape} {dn} {dt} {lq}x{rq} tile={tile} asym={asym}', thunk


@pytest.mark.parametrize('seed', [3, 17])
def test_sweep_dimension_numbers(seed):
  _run(_dimension_number_cases(seed, 250))


# ---------------------------------------------------------------------------------------------------------------
# einsum, ragged_dot
# ---------------------------------------------------------------------------------------------------------------

_SIZES = {'b': [1, 2, 3], 'h': [1, 2, 4], 'q': [1, 5, 16, 40, 130], 'k': [1, 8, 24, 136], 'd': [16, 32, 64, 128, 256, 80],
          'e': [2, 4, 8], 'n': [8, 24, 64, 200]}
_TEMPLATES = ['bqd,bkd->bqk', 'bhqd,bhkd->bhqk', 'bqd,dn->bqn', 'bqed,edn->bqn', 'qd,dn->nq', 'dq,dn->qn', 'bqd,bdn->bnq',
              'bhqd,hdn->bqn', 'bqhd,hdn->bqhn', 'qd,nd->qn', 'bqd,bkd->bkq']


def _einsum_cases(seed, count):
  from qwix_amd.core import einsum as es
  from qwix_amd.core import qarray
  r = util.rng(seed)
  for c in range(count):
    t = str(r.choice(_TEMPLATES))
    sz = {ch: int(r.choice(v)) for ch, v in _SIZES.items()}
    ls, rs = t.split('->')[0].split(',')
    lshape, rshape = tuple(sz[ch] for ch in ls), tuple(sz[ch] for ch in rs)
    qt = str(r.choice(['int8', 'int8', O.E4M3]))
    dt = O.BF16 if r.random() < 0.7 else O.F32

    def thunk(t=t, lshape=lshape, rshape=rshape, qt=qt, dt=dt, c=c):
      x_np, x_t = util.make(lshape, dt, seed=c)
      w_np, w_t = util.make(rshape, dt, seed=c + 999, scale=0.05)
      kw = dict(einsum_str=t, ndims=(len(lshape), len(rshape)), tile_size=None, qtype=qt)
      xq = qarray.quantize(x_t, es.get_how_to_quantize(for_lhs=True, **kw))
      wq = qarray.quantize(w_t, es.get_how_to_quantize(for_lhs=False, **kw))
      oxq = O.quantize(O.FArr(x_np, dt), O.einsum_get_how_to_quantize(for_lhs=True, **kw))
      owq = O.quantize(O.FArr(w_np, dt), O.einsum_get_how_to_quantize(for_lhs=False, **kw))
      util.assert_qarray_equal(xq, oxq, 'lhs')
      util.assert_qarray_equal(wq, owq, 'rhs')
      got, want = util.f32np(es.einsum(t, xq, wq)), O.einsum(t, oxq, owq).v
      if qt == 'int8':
        _exact(got, want)
      else:
        assert got.shape == want.shape and _rel(got, want) < (2e-2 if dt == O.BF16 else 1e-3)

    yield f'einsum {t} {lshape} {rshape} {dt} {qt}', thunk


def test_sweep_einsum():
  _run(_einsum_cases(8, 150))


def _ragged_cases(seed, count):
  from qwix_amd.core import qarray
  from qwix_amd.core import ragged_dot as rd
  r = util.rng(seed)
  for c in range(count):
    dt = O.BF16 if r.random() < 0.7 else O.F32
    G = int(r.choice([1, 2, 3, 5, 8, 16]))
    K = int(r.choice([16, 48, 128, 256, 384, 512]))
    N = int(r.choice([8, 24, 72, 128, 256, 260]))
    sizes = [int(r.choice([0, 1, 3, 16, 17, 40, 64, 130, 300])) for _ in range(G)]
    M = sum(sizes) + int(r.choice([0, 0, 5]))
    qt = str(r.choice(['int8', 'int8', O.E4M3]))
    lcw = [(), (0,)][int(r.integers(2))]
    rcw = [(), (0,), (2,), (0, 2)][int(r.integers(4))]
    rt = [None, None, {1: 128}, {1: 128, 2: 128}][int(r.integers(4))]
    if rt and (K % 128 or (2 in rt and N % 128)):
      rt = None
    if rt and 2 in rt:
      rcw = tuple(a for a in rcw if a != 2)
    lt = {1: 128} if (rt and r.random() < 0.4) else None
    lhs_float = r.random() < 0.15
    calib = 'minmax' if (qt == 'int8' and r.random() < 0.15) else 'absmax'
    if M == 0:
      continue

    def thunk(dt=dt, G=G, K=K, N=N, sizes=sizes, M=M, qt=qt, lcw=lcw, rcw=rcw, rt=rt, lt=lt, lhs_float=lhs_float,
              calib=calib, c=c):
      x_np, x_t = util.make((M, K), dt, seed=c)
      w_np, w_t = util.make((G, K, N), dt, seed=c + 999, scale=0.05)
      ha = dict(qtype=qt, channelwise_axes=list(lcw), tiled_axes=lt or {})
      hw = dict(qtype=qt, channelwise_axes=list(rcw), tiled_axes=rt or {}, calibration_method=calib)
      wq, owq = qarray.quantize(w_t, qarray.HowToQuantize(**hw)), O.quantize(O.FArr(w_np, dt), O.HowToQuantize(**hw))
      util.assert_qarray_equal(wq, owq, 'rhs')
      if lhs_float:
        xq, oxq = x_t, O.FArr(x_np, dt)
      else:
        xq, oxq = qarray.quantize(x_t, qarray.HowToQuantize(**ha)), O.quantize(O.FArr(x_np, dt), O.HowToQuantize(**ha))
      gs = torch.tensor(sizes, dtype=torch.int32, device=util.DEV)
      got = util.f32np(rd.ragged_dot(xq, wq, gs))
      want = O.ragged_dot(oxq, owq, np.array(sizes, dtype=np.int32)).v
      if qt == 'int8' and not lhs_float and calib == 'absmax' and not (rt and 1 in rt and K > 128):
        _exact(got, want)
      else:
        assert got.shape == want.shape and _rel(got, want) < (2e-2 if dt == O.BF16 else 2e-3)

    yield (f'ragged M={M} K={K} G={G} N={N} sizes={sizes} {dt} {qt} lcw={lcw} rcw={rcw} rhs tiles={rt} lhs tiles={lt} '
           f'float lhs={lhs_float} {calib}'), thunk


def test_sweep_ragged_dot():
  _run(_ragged_cases(3, 150))
