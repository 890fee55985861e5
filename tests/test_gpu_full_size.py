"""GPU: size-independent properties at the full benchmark shapes, where the oracle would take minutes.

Operands are small integers, so that every product and every partial sum is an exact integer in f32 whatever
the accumulation order: sampled output rows must equal an int64 product computed on the host, and the sum of
all outputs must equal (column sums of a) . (row sums of b), a checksum of checksums."""
import numpy as np
import pytest
import torch

from tests import util

pytestmark = pytest.mark.gpu


def _small_ints(shape, lo, hi, seed, dtype):
  g = torch.Generator(device='cpu').manual_seed(seed)
  return torch.randint(lo, hi + 1, shape, generator=g, dtype=torch.int8).to(util.DEV).to(dtype)


def _check_rows_and_checksum(out, a_int, b_nk_int, rows):
  """out (M, N) float/int tensor on the GPU; a_int (M, K), b_nk_int (N, K) int8 tensors on the GPU."""
  want = a_int[rows].cpu().numpy().astype(np.int64) @ b_nk_int.cpu().numpy().astype(np.int64).T
  assert np.array_equal(out[rows].cpu().to(torch.float64).numpy(), want.astype(np.float64))
  total = out.to(torch.float64).sum().item()
  want_total = float(a_int.to(torch.float64).sum(0).cpu().numpy() @ b_nk_int.to(torch.float64).sum(0).cpu().numpy())
  assert total == want_total


def test_fp8_gemm_at_the_ffn_shape():
  """(8192, 8192) x (8192, 28672) e4m3, f32 out, no scales: values in -2..2 are exact in e4m3, sums stay below 2^24."""
  from qwix_amd import _lib
  M, K, N = 8192, 8192, 28672
  a_i = _small_ints((M, K), -2, 2, 1, torch.int8)
  b_i = _small_ints((N, K), -2, 2, 2, torch.int8)
  a, b = a_i.to(torch.float32).to(torch.float8_e4m3fn), b_i.to(torch.float32).to(torch.float8_e4m3fn)
  out = torch.empty(M, N, dtype=torch.float32, device=util.DEV)
  print('case fp8 full size', M, K, N, flush=True)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), K, b.data_ptr(), K, _lib.E4M3, M, N, K, None, 0, None, 0, _lib.F32,
            out.data_ptr(), _lib.F32, N, _lib.stream_of(a))
  torch.cuda.synchronize()
  rows = util.rng(3).choice(M, 8, replace=False)
  _check_rows_and_checksum(out, a_i, b_i, rows)


def test_int8_gemm_bf16_epilogue_at_8192():
  """8192^3 int8 through the scaled epilogue (power-of-two scales keep every value exact in bf16)."""
  from qwix_amd import _lib
  M = N = K = 8192
  a = _small_ints((M, K), -1, 1, 5, torch.int8)
  b = _small_ints((N, K), -1, 1, 6, torch.int8)
  # |sum| <= 8192 -> needs 14 bits: keep it exact in bf16 by making operands sparse enough: |sum| < 256
  a = a * (torch.rand(M, K, device=util.DEV) < 0.01).to(torch.int8)
  sa = torch.full((M,), 0.5, dtype=torch.bfloat16, device=util.DEV)
  sb = torch.full((N,), 4.0, dtype=torch.bfloat16, device=util.DEV)
  out = torch.empty(M, N, dtype=torch.bfloat16, device=util.DEV)
  print('case int8 full size', M, K, N, flush=True)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), K, b.data_ptr(), K, _lib.INT8, M, N, K, sa.data_ptr(), _lib.BF16,
            sb.data_ptr(), _lib.BF16, 0, out.data_ptr(), _lib.BF16, N, _lib.stream_of(a))
  torch.cuda.synchronize()
  rows = util.rng(4).choice(M, 8, replace=False)
  want = a[rows].cpu().numpy().astype(np.int64) @ b.cpu().numpy().astype(np.int64).T
  assert np.abs(want).max() < 256
  assert np.array_equal(out[rows].float().cpu().numpy(), want.astype(np.float32) * 2.0)


def test_grouped_a8w4_gemm_at_the_hadamard_shape():
  """(2048, 8192) int8 x (8192, 8192) int4, groups of 128, unit scales: the f32 sum of the int32 partials is exact."""
  from qwix_amd import _lib
  from qwix_amd.core.qarray import Int4Tensor
  M, K, N, G = 2048, 8192, 8192, 128
  a = _small_ints((M, K), -127, 127, 7, torch.int8)
  b_i = _small_ints((N, K), -8, 7, 8, torch.int8)           # (N, K) K-contiguous logical values
  packed = Int4Tensor.pack(b_i).data if hasattr(Int4Tensor, 'pack') else None
  if packed is None:
    u = (b_i.to(torch.int16) & 0xF).to(torch.uint8)
    packed = (u[:, 0::2] | (u[:, 1::2] << 4)).contiguous()
  sb = torch.ones(K // G, N, dtype=torch.float32, device=util.DEV)
  out = torch.empty(M, N, dtype=torch.float32, device=util.DEV)
  print('case grouped full size', M, K, N, flush=True)
  _lib.call('qwix_hip_qgemm_grouped', a.data_ptr(), K, packed.data_ptr(), K // 2, _lib.INT4, M, N, K, G, None, 0, 1,
            sb.data_ptr(), _lib.F32, out.data_ptr(), _lib.F32, N, 0, None, _lib.stream_of(a))
  torch.cuda.synchronize()
  rows = util.rng(5).choice(M, 8, replace=False)
  _check_rows_and_checksum(out, a, b_i, rows)


def test_ragged_gemm_at_the_moe_shape():
  """8192 tokens, 8 experts, K 4096, N 14336: every row against its own expert, leftover rows zero."""
  from qwix_amd import _lib
  M, K, N, G = 8192, 4096, 14336, 8
  a = _small_ints((M, K), -15, 15, 9, torch.int8)
  b = _small_ints((G, N, K), -15, 15, 10, torch.int8)
  sizes_host = [1000, 1100, 900, 1024, 1500, 600, 1000, 1000]   # 8124 rows: the last 68 belong to no expert
  sizes = torch.tensor(sizes_host, dtype=torch.int32, device=util.DEV)
  out = torch.full((M, N), 7.0, dtype=torch.float32, device=util.DEV)
  print('case ragged full size', M, K, N, G, flush=True)
  _lib.call('qwix_hip_qgemm_ragged', a.data_ptr(), K, b.data_ptr(), K, N * K, _lib.INT8, M, N, K, sizes.data_ptr(), G,
            None, 0, None, 0, 0, 0, out.data_ptr(), _lib.F32, N, _lib.stream_of(a))
  torch.cuda.synchronize()
  starts = np.concatenate([[0], np.cumsum(sizes_host)])
  rows = np.array([0, 999, 1000, 2099, 2100, 4023, 4024, 8123])
  for r in rows:
    g = int(np.searchsorted(starts, r, side='right') - 1)
    want = a[r].cpu().numpy().astype(np.int64) @ b[g].cpu().numpy().astype(np.int64).T
    assert np.array_equal(out[r].cpu().numpy().astype(np.int64), want), (r, g)
  assert torch.count_nonzero(out[starts[-1]:]).item() == 0
  # checksum per expert: sum of its rows' outputs == (column sums of its rows) . (row sums of its weight)
  for g in range(G):
    blk = out[starts[g]:starts[g + 1]].to(torch.float64).sum().item()
    want = float(a[starts[g]:starts[g + 1]].to(torch.float64).sum(0).cpu().numpy() @ b[g].to(torch.float64).sum(0).cpu().numpy())
    assert blk == want, g


def test_activation_quantize_at_8192_square():
  """Per-token int8 / e4m3 quantize of (8192, 8192) bf16, checked by torch arithmetic as an independent hand:
  scale = bf16(absmax / qmax) per row, and every value lies within half a step (one bf16 rounding of the
  quotient included) of its reconstruction."""
  from qwix_amd.core import qarray
  g = torch.Generator(device='cpu').manual_seed(11)
  x = torch.randn(8192, 8192, generator=g, dtype=torch.float32).to(torch.bfloat16).to(util.DEV)
  for qtype, qmax in (('int8', 127.5), ('float8_e4m3fn', 448.0)):
    q = qarray.quantize(x, qarray.HowToQuantize(qtype=qtype, channelwise_axes=[0]))
    absmax = x.abs().amax(dim=1, keepdim=True)
    want_scale = (absmax.float() / qmax).to(torch.bfloat16)
    assert torch.equal(q.scale, want_scale), qtype
    quot = (x.float() / q.scale.float()).to(torch.bfloat16).float()
    if qtype == 'int8':
      assert torch.equal(q.qvalue.float(), torch.clamp(torch.round(quot), -128, 127))
    else:
      assert torch.equal(q.qvalue.float(), torch.clamp(quot, -448, 448).to(torch.float8_e4m3fn).float())


def test_weight_quantize_at_ffn_size_in_column_strips():
  """Per-channel (reduction along the strided axis) e4m3 / int8 quantize of an (8192, 28672) bf16 weight, which
  is larger than the memory-side cache and therefore taken in strips of columns; checked by torch arithmetic."""
  from qwix_amd.core import qarray
  g = torch.Generator(device='cpu').manual_seed(12)
  w = (torch.randn(8192, 28672, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(util.DEV)
  w *= torch.linspace(0.5, 2.0, 28672, device=util.DEV).to(torch.bfloat16)  # a scale in the wrong column shows
  for qtype, qmax, layout in (('float8_e4m3fn', 448.0, None), ('int8', 127.5, 'natural')):
    q = qarray.quantize(w, qarray.HowToQuantize(qtype=qtype, channelwise_axes=[1]), layout=layout)
    want_scale = (w.abs().amax(dim=0, keepdim=True).float() / qmax).to(torch.bfloat16)
    assert torch.equal(q.scale, want_scale), qtype
    quot = (w.float() / q.scale.float()).to(torch.bfloat16).float()
    if qtype == 'int8':
      assert torch.equal(q.qvalue.float(), torch.clamp(torch.round(quot), -128, 127))
    else:
      assert torch.equal(q.qvalue.float(), torch.clamp(quot, -448, 448).to(torch.float8_e4m3fn).float())
    del q, quot


def test_block_quantize_at_ffn_size():
  """One e4m3 scale per 128 x 128 block of a (4096, 14336) bf16 weight, checked by torch arithmetic."""
  from qwix_amd.core import qarray
  g = torch.Generator(device='cpu').manual_seed(13)
  w = (torch.randn(4096, 14336, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(util.DEV)
  w *= torch.linspace(0.5, 2.0, 14336, device=util.DEV).to(torch.bfloat16)
  q = qarray.quantize(w, qarray.HowToQuantize(qtype='float8_e4m3fn', tiled_axes={0: 128, 1: 128}))
  blocks = w.reshape(32, 128, 112, 128)
  want_scale = (blocks.abs().amax(dim=(1, 3)).float() / 448.0).to(torch.bfloat16)
  assert torch.equal(q.scale, want_scale)
  s = q.scale.float().repeat_interleave(128, 0).repeat_interleave(128, 1)
  quot = (w.float() / s).to(torch.bfloat16).float()
  assert torch.equal(q.qvalue.float(), torch.clamp(quot, -448, 448).to(torch.float8_e4m3fn).float())


def test_zero_point_gemm_at_4096():
  """4096^3 int8 with the zero-point correction in the epilogue of the large-tile kernel, f32 out, no scales:
  out = a.b^T - zu (x) zv exactly."""
  from qwix_amd import _lib
  M = N = K = 4096
  a = _small_ints((M, K), -3, 3, 21, torch.int8)
  b = _small_ints((N, K), -3, 3, 22, torch.int8)
  g = torch.Generator(device='cpu').manual_seed(23)
  zu = torch.randint(-128, 128, (M,), generator=g, dtype=torch.int32).to(util.DEV)
  zv = torch.empty(N, dtype=torch.int32, device=util.DEV)
  _lib.call('qwix_hip_ksum_i8', b.data_ptr(), K, N, K, zv.data_ptr(), _lib.stream_of(b))
  assert torch.equal(zv, b.to(torch.int32).sum(1, dtype=torch.int32))
  out = torch.empty(M, N, dtype=torch.float32, device=util.DEV)
  print('case zero point full size', M, K, N, flush=True)
  _lib.call('qwix_hip_qgemm_zp', a.data_ptr(), K, b.data_ptr(), K, M, N, K, None, 0, None, 0, zu.data_ptr(),
            zv.data_ptr(), out.data_ptr(), _lib.F32, N, _lib.stream_of(a))
  torch.cuda.synchronize()
  rows = util.rng(24).choice(M, 8, replace=False)
  want = a[rows].cpu().numpy().astype(np.int64) @ b.cpu().numpy().astype(np.int64).T
  want = want - zu[rows].cpu().numpy().astype(np.int64)[:, None] * zv.cpu().numpy().astype(np.int64)[None, :]
  assert np.abs(want).max() < 2 ** 24
  assert np.array_equal(out[rows].cpu().to(torch.float64).numpy(), want.astype(np.float64))


@pytest.mark.parametrize('n_extra', [0, 100])
def test_int8_gemm_with_a_short_last_round(n_extra):
  """2048 x 10240 x 512: 320 tiles of 256 x 256 are one full round of the chip plus a quarter (and, with 100
  more columns, a ragged last tile column).  Scales differ per column, so a misplaced column shows; the
  zero-point variant runs over the same shape."""
  from qwix_amd import _lib
  M, K, N = 2048, 512, 10240 + n_extra
  a = _small_ints((M, K), -3, 3, 31, torch.int8)
  b = _small_ints((N, K), -3, 3, 32, torch.int8)
  sb = (2.0 ** torch.randint(-2, 3, (N,), generator=torch.Generator().manual_seed(33)).float()).to(util.DEV)
  out = torch.empty(M, N, dtype=torch.float32, device=util.DEV)
  print('case short last round', M, K, N, flush=True)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), K, b.data_ptr(), K, _lib.INT8, M, N, K, None, 0, sb.data_ptr(), _lib.F32, 0,
            out.data_ptr(), _lib.F32, N, _lib.stream_of(a))
  torch.cuda.synchronize()
  rows = util.rng(34).choice(M, 8, replace=False)
  want = a[rows].cpu().numpy().astype(np.int64) @ b.cpu().numpy().astype(np.int64).T
  assert np.array_equal(out[rows].cpu().numpy().astype(np.float64), want * sb.cpu().numpy().astype(np.float64)[None, :])
  total = (out.to(torch.float64) / sb.to(torch.float64)).sum().item()
  assert total == float(a.to(torch.float64).sum(0).cpu().numpy() @ b.to(torch.float64).sum(0).cpu().numpy())
  # zero-point correction across the same split
  zu = torch.randint(-128, 128, (M,), generator=torch.Generator().manual_seed(35), dtype=torch.int32).to(util.DEV)
  zv = b.to(torch.int32).sum(1, dtype=torch.int32)
  _lib.call('qwix_hip_qgemm_zp', a.data_ptr(), K, b.data_ptr(), K, M, N, K, None, 0, sb.data_ptr(), _lib.F32, zu.data_ptr(),
            zv.data_ptr(), out.data_ptr(), _lib.F32, N, _lib.stream_of(a))
  torch.cuda.synchronize()
  want = want - zu[rows].cpu().numpy().astype(np.int64)[:, None] * zv.cpu().numpy().astype(np.int64)[None, :]
  assert np.array_equal(out[rows].cpu().numpy().astype(np.float64), want * sb.cpu().numpy().astype(np.float64)[None, :])


def test_one_row_against_a_large_vocabulary_projection():
  """1 x 4096 x 65536 int8 (256 MB of weights: the small-workgroup shape of the weight-streaming kernel), f32 out
  with per-column power-of-two scales: every output is an exact integer times its scale."""
  from qwix_amd import _lib
  M, K, N = 3, 4096, 65536
  a = _small_ints((M, K), -3, 3, 41, torch.int8)
  b = _small_ints((N, K), -3, 3, 42, torch.int8)
  sb = (2.0 ** torch.randint(-2, 3, (N,), generator=torch.Generator().manual_seed(43)).float()).to(util.DEV)
  out = torch.empty(M, N, dtype=torch.float32, device=util.DEV)
  print('case large vocabulary', M, K, N, flush=True)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), K, b.data_ptr(), K, _lib.INT8, M, N, K, None, 0, sb.data_ptr(), _lib.F32, 0,
            out.data_ptr(), _lib.F32, N, _lib.stream_of(a))
  torch.cuda.synchronize()
  want = a.cpu().numpy().astype(np.int64) @ b.cpu().numpy().astype(np.int64).T
  assert np.array_equal(out.cpu().numpy().astype(np.float64), want * sb.cpu().numpy().astype(np.float64)[None, :])


@pytest.mark.parametrize('M,K,N', [(64, 4096, 14336), (33, 2048, 8200), (20, 8192, 28672), (48, 128, 66000), (64, 384, 22016),
                                   (32, 4096, 14336), (24, 8192, 8192), (17, 2048, 28700), (64, 4096, 28672),
                                   (128, 4096, 14336), (100, 2048, 8200), (65, 512, 16384), (128, 1024, 28672),
                                   (64, 4096, 4096), (24, 2048, 6100), (20, 1152, 8100), (50, 1024, 8190),
                                   (256, 4096, 4096), (200, 2048, 8192), (130, 1280, 8000), (16, 4096, 28672), (3, 8192, 14000)])
def test_decode_batch_against_a_wide_weight(M, K, N):
  """17 to 256 rows against megabytes of weights (fewer rows too from about 100 MB of weights on) (the deep-prefetch tile): int8 with per-row and per-column
  power-of-two scales, f32 out; every output is an exact integer times two exact scales.  K of one, three
  and many 128-wide slabs exercise the start and the end of the prefetch pipeline; N = 8200 a ragged last tile.
  The shapes cover the 32-, 64- and 128-row tiles (also two 128-row tiles one above the other), and workgroups of 32, 64 and 128 columns; up to N 8192 the
  wavefronts of a workgroup split K instead (9 slabs over 4 wavefronts: uneven shares; 8: fewer than the pipeline is deep)."""
  from qwix_amd import _lib
  a = _small_ints((M, K), -127, 127, 51, torch.int8)
  b = _small_ints((N, K), -127, 127, 52, torch.int8)
  g = torch.Generator().manual_seed(53)
  sa = (2.0 ** torch.randint(-3, 3, (M,), generator=g).float()).to(util.DEV)
  sb = (2.0 ** torch.randint(-3, 3, (N,), generator=g).float()).to(util.DEV)
  out = torch.full((M, N), float('nan'), dtype=torch.float32, device=util.DEV)
  print('case decode batch', M, K, N, flush=True)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), K, b.data_ptr(), K, _lib.INT8, M, N, K, sa.data_ptr(), _lib.F32, sb.data_ptr(),
            _lib.F32, 0, out.data_ptr(), _lib.F32, N, _lib.stream_of(a))
  torch.cuda.synchronize()
  want = (a.double() @ b.double().T) * sa.double()[:, None] * sb.double()[None, :]
  assert torch.equal(out.double(), want)
  # bf16 out through bf16 scales: the rounding flags of the run-time epilogue
  outb = torch.empty(M, N, dtype=torch.bfloat16, device=util.DEV)
  sab, sbb = sa.to(torch.bfloat16), sb.to(torch.bfloat16)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), K, b.data_ptr(), K, _lib.INT8, M, N, K, sab.data_ptr(), _lib.BF16,
            sbb.data_ptr(), _lib.BF16, 0, outb.data_ptr(), _lib.BF16, N, _lib.stream_of(a))
  accb = (a.double() @ b.double().T).float().to(torch.bfloat16)
  wantb = (accb * sab[:, None]) * sbb[None, :]
  assert torch.equal(outb, wantb)


@pytest.mark.parametrize('M,K,N', [(64, 4096, 14336), (32, 8192, 8192), (40, 2048, 28700), (128, 4096, 8192), (48, 4096, 4096), (40, 2304, 4000), (30, 8192, 2048), (250, 2048, 4096)])
def test_fp8_decode_batch_against_a_wide_weight(M, K, N):
  """The same tile with e4m3 operands: values in -2..2 are exact in e4m3 and every sum stays below 2^24, so the
  f32 output must equal the integer product; power-of-two scales keep the bf16 epilogue exact as well."""
  from qwix_amd import _lib
  a_i = _small_ints((M, K), -2, 2, 61, torch.int8)
  b_i = _small_ints((N, K), -2, 2, 62, torch.int8)
  a, b = a_i.to(torch.float32).to(torch.float8_e4m3fn), b_i.to(torch.float32).to(torch.float8_e4m3fn)
  g = torch.Generator().manual_seed(63)
  sa = (2.0 ** torch.randint(-3, 3, (M,), generator=g).float()).to(util.DEV)
  sb = (2.0 ** torch.randint(-3, 3, (N,), generator=g).float()).to(util.DEV)
  out = torch.full((M, N), float('nan'), dtype=torch.float32, device=util.DEV)
  print('case fp8 decode batch', M, K, N, flush=True)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), K, b.data_ptr(), K, _lib.E4M3, M, N, K, sa.data_ptr(), _lib.F32, sb.data_ptr(),
            _lib.F32, _lib.F32, out.data_ptr(), _lib.F32, N, _lib.stream_of(a))
  torch.cuda.synchronize()
  want = (a_i.double() @ b_i.double().T) * sa.double()[:, None] * sb.double()[None, :]
  assert torch.equal(out.double(), want)


def test_weight_only_int4_prefill_at_the_gemv_weight_shape():
  """(2048, 4096) bf16 x (4096, 14336) int4 in groups of 128 with power-of-two scales, through reduce-minor
  dequantize + the bf16 MFMA GEMM: the dequantized weights are small multiples of the scales, exact in bf16, and
  every partial sum is exact in f32."""
  from qwix_amd import _lib
  M, K, N, G = 2048, 4096, 14336, 128
  x_i = _small_ints((M, K), -3, 3, 11, torch.int8)
  b_i = _small_ints((N, K), -8, 7, 12, torch.int8)
  u = (b_i.to(torch.int16) & 0xF).to(torch.uint8)
  packed = (u[:, 0::2] | (u[:, 1::2] << 4)).contiguous()
  # scale 2^(g mod 3 - 1) per group, the same for every column: out = sum_g 2^e_g * (x_g . b_g)
  e = (torch.arange(K // G, device=util.DEV) % 3 - 1).to(torch.float32)
  sb = torch.pow(2.0, e)[:, None].expand(K // G, N).contiguous()
  x = x_i.to(torch.bfloat16)
  w = torch.empty(N, K, dtype=torch.bfloat16, device=util.DEV)
  out = torch.empty(M, N, dtype=torch.float32, device=util.DEV)
  print('case weight-only prefill full size', M, K, N, flush=True)
  st = _lib.stream_of(x)
  _lib.call('qwix_hip_dequantize_rm', packed.data_ptr(), _lib.INT4, 1, K, N, G, sb.data_ptr(), None, _lib.F32, w.data_ptr(),
            _lib.BF16, st)
  _lib.call('qwix_hip_gemm_bf16', x.data_ptr(), K, w.data_ptr(), K, M, N, K, out.data_ptr(), _lib.F32, N, st)
  torch.cuda.synchronize()
  # the weights in units of 1/2: exact integers
  w2 = (b_i.to(torch.int32).reshape(N, K // G, G) * torch.pow(2.0, e + 1).to(torch.int32)[None, :, None]).reshape(N, K)
  assert torch.equal((w.to(torch.float32) * 2).to(torch.int32), w2)
  rows = util.rng(13).choice(M, 8, replace=False)
  want = x_i[rows].cpu().numpy().astype(np.int64) @ w2.cpu().numpy().astype(np.int64).T
  assert np.abs(want).max() < 2 ** 24
  assert np.array_equal(out[rows].cpu().to(torch.float64).numpy() * 2, want.astype(np.float64))
  total = out.to(torch.float64).sum().item() * 2
  assert total == float(x_i.to(torch.float64).sum(0).cpu().numpy() @ w2.to(torch.float64).sum(0).cpu().numpy())


def test_quantize_of_more_than_2_31_elements():
  """70000 x 32768 bf16 (2.29e9 elements, 4.6 GB): element indices pass 2^31 in every quantize layout.  Sampled rows
  and columns are compared with the oracle bit for bit (the oracle on the whole array would take minutes)."""
  from oracle import qwix_oracle as O
  from qwix_amd.core import qarray
  M, K = 70000, 32768
  x = torch.randn(M, K, device=util.DEV, dtype=torch.bfloat16)
  rows = [0, 1, 12345, 65535, 65536, M - 1]
  xs = x[rows].float().cpu().numpy()
  for qt in ('int8', 'int4', O.E4M3):
    print('case big per-token', qt, flush=True)
    q = qarray.quantize(x, qarray.HowToQuantize(qtype=qt, channelwise_axes=[0]))
    oq = O.quantize(O.FArr(xs, O.BF16), O.HowToQuantize(qtype=qt, channelwise_axes=[0]))
    vals = q.qvalue.unpack()[rows] if qt == 'int4' else q.qvalue[rows]
    got = vals.view(torch.uint8).cpu().numpy() if qt == O.E4M3 else vals.cpu().numpy()
    assert np.array_equal(got, oq.qvalue), qt
    assert np.array_equal(util.f32np(q.scale[rows]), oq.scale.v), qt
    del q, vals
  print('case big groups of 128', flush=True)
  how = dict(qtype='int8', channelwise_axes=[0], tiled_axes={1: 128})
  q = qarray.quantize(x, qarray.HowToQuantize(**how))
  oq = O.quantize(O.FArr(xs, O.BF16), O.HowToQuantize(**how))
  assert np.array_equal(q.qvalue[rows].cpu().numpy(), oq.qvalue) and np.array_equal(util.f32np(q.scale[rows]), oq.scale.v)
  del q
  print('case big per-channel', flush=True)
  cols = [0, 7, 8, 1000, K - 1]
  q = qarray.quantize(x, qarray.HowToQuantize(qtype='int8', channelwise_axes=[1]))
  oq = O.quantize(O.FArr(x[:, cols].float().cpu().numpy(), O.BF16), O.HowToQuantize(qtype='int8', channelwise_axes=[1]))
  assert np.array_equal(util.f32np(q.scale[:, cols]), oq.scale.v)
  assert np.array_equal(q.qvalue[:, cols].cpu().numpy(), oq.qvalue)
  d = qarray.dequantize(q)
  assert np.array_equal(util.f32np(d[:, cols]), O.dequantize(oq).v)


@pytest.mark.parametrize('M,K,N', [(50000, 49152, 256), (300, 98304, 50000)])
def test_int8_gemm_with_an_operand_of_more_than_2_31_bytes(M, K, N):
  """Byte offsets into one operand pass 2^31 (2.46 GB of activations / 4.9 GB of weights): sampled outputs against the
  exact integer product and the bf16 epilogue chain."""
  from qwix_amd import _lib
  print('case big gemm', M, K, N, flush=True)
  a = torch.randint(-128, 128, (M, K), dtype=torch.int8, device=util.DEV)
  b = torch.randint(-128, 128, (N, K), dtype=torch.int8, device=util.DEV)
  acc = torch.empty(M, N, dtype=torch.int32, device=util.DEV)
  st = _lib.stream_of(a)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), K, b.data_ptr(), K, _lib.INT8, M, N, K, None, 0, None, 0, 0, acc.data_ptr(),
            _lib.I32, N, st)
  rows, cols = [0, 1, M // 2 + 3, M - 1], [0, 5, N // 2, N - 1]
  want = a[rows].double() @ b[cols].double().T            # |sums| < 2^53: exact
  assert torch.equal(acc[rows][:, cols].double(), want)
  sa = (torch.rand(M, device=util.DEV) * 0.01 + 0.001).to(torch.bfloat16)
  sb = (torch.rand(N, device=util.DEV) * 0.01 + 0.001).to(torch.bfloat16)
  out = torch.empty(M, N, dtype=torch.bfloat16, device=util.DEV)
  _lib.call('qwix_hip_qgemm', a.data_ptr(), K, b.data_ptr(), K, _lib.INT8, M, N, K, sa.data_ptr(), _lib.BF16,
            sb.data_ptr(), _lib.BF16, 0, out.data_ptr(), _lib.BF16, N, st)
  w = acc[rows][:, cols].float().bfloat16()
  w = (w.float() * sa[rows].float()[:, None]).bfloat16()
  w = (w.float() * sb[cols].float()[None, :]).bfloat16()
  assert torch.equal(out[rows][:, cols], w)
