"""qwix_hip_quantize_static (the entry point that allocates nothing: its calibration scratch is a
file-scope device array) against qwix_hip_quantize with a caller workspace, through the C ABI.

Bit-exact on qvalues, scales and zero points; two calls in a row on the same GPU, the second on a
smaller input, so that what the first call left in the shared array would show.
"""
import pytest
import torch

from qwix_amd import _lib

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


def _quantize(entry, x, outer, reduce, inner, tile, qtype, cal, layout):
  """Calls `entry` ('qwix_hip_quantize' or 'qwix_hip_quantize_static') on the 3-D view of x."""
  lib = _lib.load()
  n = outer * reduce * inner
  nscale = outer * (reduce // tile) * inner
  q = torch.full((n if qtype != _lib.INT4 else n // 2,), 0x55, dtype=torch.uint8, device=DEV)
  scale = torch.full((nscale,), -1.0, dtype=x.dtype, device=DEV)
  zp = torch.full((nscale,), 77, dtype=torch.int8, device=DEV) if cal == _lib.MINMAX else None
  tag = _lib.float_tag(x.dtype)
  st = _lib.stream_of(x)
  if entry == 'qwix_hip_quantize':
    need = lib.qwix_hip_quantize_workspace_bytes(outer, reduce, inner, tile, cal)
    assert need > 0, 'the case must be one whose kernels use scratch memory'
    ws = torch.full((need,), 0xAB, dtype=torch.uint8, device=DEV)
    _lib.call(entry, x.data_ptr(), tag, outer, reduce, inner, tile, qtype, cal, 0.0, layout, q.data_ptr(),
              scale.data_ptr(), _lib.ptr(zp), ws.data_ptr(), need, st)
  else:
    _lib.call(entry, x.data_ptr(), tag, outer, reduce, inner, tile, qtype, cal, 0.0, layout, q.data_ptr(),
              scale.data_ptr(), _lib.ptr(zp), st)
  torch.cuda.synchronize()
  return q, scale, zp


def _same(a, b, what):
  for got, want, name in zip(a, b, ('qvalue', 'scale', 'zero_point')):
    if want is None:
      assert got is None
      continue
    g, w = got.view(torch.uint8).cpu(), want.view(torch.uint8).cpu()
    assert torch.equal(g, w), f'{what}: {name} differs in {(g != w).sum().item()} bytes'


# (outer, reduce, inner, tile, dtype, qtype, calibration, layout): per-channel weights whose scale groups
# span several workgroups (atomic partials in the scratch array), and per-tensor scales over long rows
# (piecewise partials in the scratch array).
CASES = [
    ((1, 2048, 1024, 2048, torch.bfloat16, _lib.INT8, _lib.ABSMAX, _lib.LAYOUT_REDUCE_MINOR),
     (1, 512, 256, 512, torch.bfloat16, _lib.INT8, _lib.ABSMAX, _lib.LAYOUT_REDUCE_MINOR)),
    ((2, 1024, 512, 512, torch.float32, _lib.INT4, _lib.MINMAX, _lib.LAYOUT_NATURAL),
     (1, 256, 64, 256, torch.float32, _lib.INT4, _lib.MINMAX, _lib.LAYOUT_NATURAL)),
    ((1, 4096, 2048, 4096, torch.bfloat16, _lib.E4M3, _lib.ABSMAX, _lib.LAYOUT_REDUCE_MINOR),
     (1, 384, 128, 384, torch.bfloat16, _lib.E4M3, _lib.ABSMAX, _lib.LAYOUT_REDUCE_MINOR)),
    ((4, 65536, 1, 65536, torch.bfloat16, _lib.INT8, _lib.MINMAX, _lib.LAYOUT_NATURAL),
     (2, 32768, 1, 32768, torch.bfloat16, _lib.INT8, _lib.MINMAX, _lib.LAYOUT_NATURAL)),
]


@pytest.mark.parametrize('first,second', CASES)
def test_static_scratch_quantize_matches_workspace_quantize_twice_in_a_row(first, second):
  for i, (outer, reduce, inner, tile, dtype, qtype, cal, layout) in enumerate((first, second)):
    g = torch.Generator(device='cpu').manual_seed(100 + i)
    # the second input is much larger in magnitude... and the first leaves large partials behind
    mag = 50.0 if i == 0 else 0.01
    x = (torch.randn(outer * reduce * inner, generator=g) * mag).to(dtype).to(DEV)
    want = _quantize('qwix_hip_quantize', x, outer, reduce, inner, tile, qtype, cal, layout)
    got = _quantize('qwix_hip_quantize_static', x, outer, reduce, inner, tile, qtype, cal, layout)
    _same(got, want, f'call {i} {(outer, reduce, inner, tile)}')


def test_static_scratch_limit_is_enforced_on_the_host():
  lib = _lib.load()
  limit = lib.qwix_hip_quantize_static_max_bytes()
  assert limit == 1 << 20
  inner = limit // 4 + 8  # one u32 partial per column: just past the limit
  assert lib.qwix_hip_quantize_workspace_bytes(1, 256, inner, 256, _lib.ABSMAX) > limit
  x = torch.zeros(8, dtype=torch.bfloat16, device=DEV)  # never read: the call must be refused first
  with pytest.raises(NotImplementedError, match='static buffer holds'):
    _lib.call('qwix_hip_quantize_static', x.data_ptr(), _lib.BF16, 1, 256, inner, 256, _lib.INT8, _lib.ABSMAX, 0.0,
              _lib.LAYOUT_NATURAL, x.data_ptr(), x.data_ptr(), None, _lib.stream_of(x))


def test_static_scratch_quantize_allocates_no_device_memory():
  """What the entry point exists for: free device memory, as the driver reports it, is the same before and after a
  series of calls (after one warm-up call, which may load the code object and resolve the array's address)."""
  outer, reduce, inner, tile = 1, 2048, 1024, 2048
  x = torch.randn(outer * reduce * inner, dtype=torch.float32).to(torch.bfloat16).to(DEV)
  q = torch.empty(outer * reduce * inner, dtype=torch.uint8, device=DEV)
  scale = torch.empty(inner, dtype=torch.bfloat16, device=DEV)
  st = _lib.stream_of(x)
  args = (x.data_ptr(), _lib.BF16, outer, reduce, inner, tile, _lib.INT8, _lib.ABSMAX, 0.0, _lib.LAYOUT_REDUCE_MINOR,
          q.data_ptr(), scale.data_ptr(), None, st)
  _lib.call('qwix_hip_quantize_static', *args)
  torch.cuda.synchronize()
  free_before = torch.cuda.mem_get_info()[0]
  reserved_before = torch.cuda.memory_reserved()
  for _ in range(8):
    _lib.call('qwix_hip_quantize_static', *args)
  torch.cuda.synchronize()
  assert torch.cuda.mem_get_info()[0] == free_before
  assert torch.cuda.memory_reserved() == reserved_before
