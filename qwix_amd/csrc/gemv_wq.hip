// Weight-only skinny GEMM (decode): bf16 activations x int4 / int8 / e4m3 group-quantized weights.
//
//   out[m,n] = sum_g s[g,n] * sum_{k in g} x[m,k] * q[n,k]         M small (16 rows per pass)
//
// HBM-bound: the weight bytes are read exactly once, the activations stay in L2.  Even at M = 16
// the multiply-adds exceed what the vector ALUs can do in the time the weights stream in, so the
// products run on v_mfma_f32_16x16x32_bf16 with the weights converted to bf16 in registers, in
// offset binary so that the conversion is one or two bit-ops per pair of weights:
//   int4: (nibble ^ 8) lands in the mantissa of bf16 128.0, giving 128 + (q + 8) exactly;
//   int8: (byte ^ 0x80) is converted with v_cvt_f32_ubyte and truncated to bf16 (exact below 256);
//   e4m3: v_cvt_pk_f32_fp8, truncated to bf16 (exact: four significant bits), no offset.
// The offset is removed by seeding each accumulator with -offset * rowsum(x), which four MFMAs against
// a constant operand produce in the accumulator's own layout.
// A workgroup is 16 wavefronts that split K; each handles NT tiles of 16 output columns with two K
// blocks of loads in flight (int4 weights by way of a wavefront-private LDS panel, in whole 128-byte lines), and
// the partial sums meet in LDS.
#include "common.h"

namespace qwix {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));


struct GemvArgs {
  const uint16_t* x; int64_t ldx;
  const uint8_t* q; int64_t ldb;
  int M, N, K;
  int bpg;         // 128-wide K blocks per scale group
  uint64_t magic;  // ceil(2^32 / bpg): kb / bpg == (kb * magic) >> 32 while kb * bpg < 2^32
  const void* s; int s_dtype;
  const int8_t* zp;  // zero points (K / group, N) like the scales, or null (symmetric weights)
  void* out; int out_dtype; int64_t ldo;
};

__device__ __forceinline__ bf16x8 as_bf16x8(v4u v) { return __builtin_bit_cast(bf16x8, v); }

// Everything one wavefront needs for one 128-wide K block: its 4 activation fragments, and per
// column tile the packed weights and the scale.
template <int BQT, int NT, int RT>
struct Block {
  v4u xf[RT][4];  // RT tiles of 16 rows of x
  v4u wq[NT][BQT == QWIX_INT4 ? 1 : 2];
  unsigned sraw[NT];  // scale bits as loaded: bf16 in the low half, or f32
  unsigned zraw[NT];  // zero point as loaded (one byte, zero-extended); only with asymmetric weights
};

// Every load is a buffer load: a wave-uniform descriptor (the operand's first byte for this workgroup) plus a
// per-lane unsigned 32-bit byte offset that is fixed for the whole kernel, plus a wave-uniform offset that
// moves along K, so that a load costs no vector arithmetic and an address no second register.  Columns
// beyond N are clamped to the last valid one instead of being predicated: an output element depends only on its
// own row of x and its own column of the weights, and the clamped ones are never stored.
template <int NT>
struct LaneOff {
  unsigned x;      // bytes from the first row of this workgroup's rows of x
  unsigned w[NT];  // bytes from row n_base of the weights
  unsigned s[NT];  // bytes from column n_base of the scales
  // int4 weights, two K blocks at a time, go through LDS (see load_blocks):
  unsigned f[2];       // bytes from the start of a 16-row tile in the wavefront's LDS panel, per K block
  uint8_t* panel;      // the wavefront's LDS panel: 16 * NT rows of 128 bytes
  const void *bx, *bw, *bs;  // wave-uniform: x from row row0, weights from row n_base, scales from column n_base
  const void* bz;            // zero points from column n_base (asymmetric weights)
};

// How the weight bytes are requested decides the speed of this kernel.  The memory side works in 128-byte lines;
// the 64 bytes that the four lanes of a column need from a weight row per K block are half a line, and reading the
// 4096 x 14336 int4 weight as 16 rows x 64 bytes per instruction takes 7.9 us (halves requested far apart) or
// 6.4 us (halves in consecutive instructions), against 6.1 us for 8 rows x 128 bytes per instruction, which is
// what a plain copy kernel reaches.  So two K blocks of int4 weights (one whole line per row) are fetched as whole
// lines, by direct-to-LDS loads into a panel private to the wavefront (one instruction = 8 rows x 128 bytes =
// 1 KiB of LDS), and the MFMA fragments are read back from there: nothing but the wavefront's own wait stands
// between the two.  Inside a row the eight 16-byte chunks sit at position chunk ^ ((row >> 1) & 7), chosen
// by having each lane fetch the matching global chunk, so that the fragment reads of 16 consecutive rows fall
// into 16 different 16-byte bank groups.  A last, single K block and int8 weights (whose lanes read 32
// consecutive bytes, a whole line per row and instruction pair) are loaded straight into registers.
//
// Direct-to-LDS loads of K blocks kb and kb + 1 (int4).  Load i fetches rows 8 i .. 8 i + 7 of the panel; its
// address needs the lane's row in that group of eight and one of two chunk offsets, nothing else, so the first
// of these loads can leave a few dozen instructions into the kernel.
template <int T0, int T1>
__device__ __forceinline__ void fetch_panel(const GemvArgs& p, const void* bw, uint8_t* panel, unsigned grow,
                                            const unsigned (&gchunk)[2], int n_base, int kb) {
  const auto rw = buffer_from(bw);
  const unsigned last_row = static_cast<unsigned>(p.N - 1 - n_base), pitch = static_cast<unsigned>(p.ldb);
#pragma unroll
  for (int i = 2 * T0; i < 2 * T1; ++i)  // column tiles T0 .. T1 - 1: 16 rows each
    buffer_to_lds16(rw, panel + i * 1024, min(i * 8 + grow, last_row) * pitch + gchunk[i & 1], kb * 64);
}

// Activations and scales of one or two consecutive K blocks, and (WEIGHTS) the weights straight into registers.
template <int BQT, int NT, bool SBF, int RT, bool TWO, bool WEIGHTS, bool ZP>
__device__ __forceinline__ void load_blocks(const GemvArgs& p, const LaneOff<NT>& a, const bool (&xrow)[RT], int kb,
                                            Block<BQT, NT, RT>* b0, Block<BQT, NT, RT>* b1) {
  constexpr bool W4 = (BQT == QWIX_INT4);
  constexpr int NB = TWO ? 2 : 1;
  Block<BQT, NT, RT>* const b[2] = {b0, b1};
  const auto rx = buffer_from(a.bx), rw = buffer_from(a.bw), rs = buffer_from(a.bs);
  // every vector load occupies the texture path for as long as its active lanes need, also when they
  // repeat an address: lanes whose row of x does not exist stay idle and feed zeros to the MFMA
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const unsigned xr = a.x + static_cast<unsigned>(rt) * 32u * static_cast<unsigned>(p.ldx);  // 16 rows of bf16 further down
#pragma unroll
    for (int h = 0; h < NB; ++h)
#pragma unroll
      for (int j = 0; j < 4; ++j) b[h]->xf[rt][j] = v4u{0, 0, 0, 0};
    if (xrow[rt]) {
#pragma unroll
      for (int h = 0; h < NB; ++h)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          b[h]->xf[rt][j] = __builtin_amdgcn_raw_buffer_load_b128(rx, xr + h * 256 + j * 16, kb * 256, 0);
    }
  }
#pragma unroll
  for (int h = 0; h < NB; ++h) {
    const int sg = static_cast<int>((static_cast<uint64_t>(static_cast<unsigned>(kb + h)) * p.magic) >> 32);
    const int s0 = sg * p.N * (SBF ? 2 : 4);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if constexpr (SBF)
        b[h]->sraw[t] = __builtin_amdgcn_raw_buffer_load_b16(rs, a.s[t], s0, 0);
      else
        b[h]->sraw[t] = __builtin_amdgcn_raw_buffer_load_b32(rs, a.s[t], s0, 0);
    }
    if constexpr (ZP) {
      const auto rz = buffer_from(a.bz);
#pragma unroll
      for (int t = 0; t < NT; ++t) b[h]->zraw[t] = __builtin_amdgcn_raw_buffer_load_b8(rz, a.s[t] / (SBF ? 2u : 4u), sg * p.N, 0);
    }
  }
  if constexpr (WEIGHTS) {
    const int wk = kb * (W4 ? 64 : 128);
    // the scheduler may not pull the two halves of a line apart
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int h = 0; h < NB; ++h) {
        b[h]->wq[t][0] = __builtin_amdgcn_raw_buffer_load_b128(rw, a.w[t] + h * (W4 ? 64 : 128), wk, 0);
        if constexpr (!W4) b[h]->wq[t][1] = __builtin_amdgcn_raw_buffer_load_b128(rw, a.w[t] + h * 128 + 16, wk, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// Weights enter the MFMA in offset binary (int4: 128 + (q + 8), int8: q + 128, both exact in bf16);
// the offset times the row sum of x is taken out by four MFMAs against the constant -offset, whose
// result seeds the accumulator of every column tile.  A widened weight fragment serves all RT row tiles; every
// output element sees the same operations in the same order whatever RT is.
// ZP (asymmetric weights): the row sums of x themselves are kept as well (four MFMAs against the constant 1); the
// zero point of a column and group times that sum is what its partial carries too much.
template <int BQT, int NT, int RT, bool ZP>
__device__ __forceinline__ void prepare_x(Block<BQT, NT, RT>& b, v4f (&base)[RT], v4f (&sumx)[RT]) {
  constexpr bool W4 = (BQT == QWIX_INT4);
  constexpr unsigned kNegOff = W4 ? 0xC308C308u : 0xC300C300u;  // bf16 -136 / -128, twice
  const v4u negoff = {kNegOff, kNegOff, kNegOff, kNegOff};
  v4u (&xf)[RT][4] = b.xf;
  if constexpr (W4) {  // element order (k0,k4,k1,k5,k2,k6,k3,k7): what the nibble widening yields (in place)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const v4u d = xf[rt][j];
        xf[rt][j][0] = __builtin_amdgcn_perm(d[2], d[0], 0x05040100);
        xf[rt][j][1] = __builtin_amdgcn_perm(d[2], d[0], 0x07060302);
        xf[rt][j][2] = __builtin_amdgcn_perm(d[3], d[1], 0x05040100);
        xf[rt][j][3] = __builtin_amdgcn_perm(d[3], d[1], 0x07060302);
      }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    base[rt] = v4f{0.f, 0.f, 0.f, 0.f};
    if constexpr (BQT != QWIX_E4M3) {  // float weights carry no offset
#pragma unroll
      for (int j = 0; j < 4; ++j)
        base[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xf[rt][j]), as_bf16x8(negoff), base[rt], 0, 0, 0);
    }
    if constexpr (ZP) {
      const v4u ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
      sumx[rt] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j)
        sumx[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xf[rt][j]), as_bf16x8(ones), sumx[rt], 0, 0, 0);
    }
  }
}

// Column tile t of one K block, after prepare_x: widen, multiply, scale, add.
template <int BQT, int NT, bool SBF, int RT, bool ZP>
__device__ __forceinline__ void compute_tile(const Block<BQT, NT, RT>& b, const v4f (&base)[RT], const v4f (&sumx)[RT], int t,
                                             v4f (&outacc)[RT][NT]) {
  constexpr bool W4 = (BQT == QWIX_INT4);
  v4f acc[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) acc[rt] = base[rt];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    v4u w;
    if constexpr (W4) {
      // (u & 0x000F000F) ^ 0x43084308: flips the nibble's sign bit and drops it into the mantissa of
      // bf16 128.0, one three-input bit-op per pair of weights
      const unsigned u = b.wq[t][0][j];
      w[0] = (u & 0x000F000Fu) ^ 0x43084308u;          // (k0, k4)
      w[1] = ((u >> 4) & 0x000F000Fu) ^ 0x43084308u;   // (k1, k5)
      w[2] = ((u >> 8) & 0x000F000Fu) ^ 0x43084308u;   // (k2, k6)
      w[3] = ((u >> 12) & 0x000F000Fu) ^ 0x43084308u;  // (k3, k7)
    } else if constexpr (BQT == QWIX_E4M3) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        // an e4m3 value has 4 significant bits: the upper half of its f32 is its bf16
        const int u = static_cast<int>(b.wq[t][j >> 1][2 * (j & 1) + h]);
        const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(u, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8(u, true);
        w[2 * h] = __builtin_amdgcn_perm(__float_as_uint(lo[1]), __float_as_uint(lo[0]), 0x07060302);
        w[2 * h + 1] = __builtin_amdgcn_perm(__float_as_uint(hi[1]), __float_as_uint(hi[0]), 0x07060302);
      }
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const unsigned u = b.wq[t][j >> 1][2 * (j & 1) + h] ^ 0x80808080u;
        // integers up to 255 have 8 significant bits: the upper half of their f32 is their bf16
        const unsigned f0 = __float_as_uint(static_cast<float>(u & 0xFFu));
        const unsigned f1 = __float_as_uint(static_cast<float>((u >> 8) & 0xFFu));
        const unsigned f2 = __float_as_uint(static_cast<float>((u >> 16) & 0xFFu));
        const unsigned f3 = __float_as_uint(static_cast<float>(u >> 24));
        w[2 * h] = __builtin_amdgcn_perm(f1, f0, 0x07060302);
        w[2 * h + 1] = __builtin_amdgcn_perm(f3, f2, 0x07060302);
      }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
      acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(b.xf[rt][j]), as_bf16x8(w), acc[rt], 0, 0, 0);
  }
  const float sc = __uint_as_float(SBF ? b.sraw[t] << 16 : b.sraw[t]);
  if constexpr (ZP) {  // sum x (q - z) = sum x q - z sum x
    const float z = static_cast<float>(static_cast<int>(b.zraw[t] << 24) >> 24);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[rt][r] = fmaf(-z, sumx[rt][r], acc[rt][r]);
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int r = 0; r < 4; ++r) outacc[rt][t][r] = fmaf(acc[rt][r], sc, outacc[rt][t][r]);
}

template <int BQT, int NT, bool SBF, int RT, bool ZP>
__device__ __forceinline__ void compute_block(Block<BQT, NT, RT>& b, v4f (&outacc)[RT][NT]) {
  v4f base[RT], sumx[RT];
  prepare_x<BQT, NT, RT, ZP>(b, base, sumx);
#pragma unroll
  for (int t = 0; t < NT; ++t) compute_tile<BQT, NT, SBF, RT, ZP>(b, base, sumx, t, outacc);
}

// Tiles T .. NT - 1 of a pair of K blocks whose int4 weights come through the LDS panel: the fragments of a tile are
// read once its two direct-to-LDS loads have landed (the tiles from H on are the newest 2 (NT - H) vector memory
// operations in flight: all but the newest 2 (NT - 1 - T) of them must be back; vmcnt only, the other counters
// stay open), and both blocks' products of that tile follow at once, so that the arithmetic of the early tiles
// runs while the late ones are still on their way.  Per output element the order of operations is that of
// compute_block on the first block, then on the second.
template <int T, int H, int NT, bool SBF, int RT, bool ZP>
__device__ __forceinline__ void consume_panel(const LaneOff<NT>& a, Block<QWIX_INT4, NT, RT>& b0, Block<QWIX_INT4, NT, RT>& b1,
                                              const v4f (&base0)[RT], const v4f (&base1)[RT], const v4f (&sumx0)[RT],
                                              const v4f (&sumx1)[RT], v4f (&outacc)[RT][NT]) {
  if constexpr (T >= H) {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * (NT - 1 - T)));
  }
  __builtin_amdgcn_sched_barrier(0);
  b0.wq[T][0] = *reinterpret_cast<const v4u*>(a.panel + T * 2048 + a.f[0]);
  b1.wq[T][0] = *reinterpret_cast<const v4u*>(a.panel + T * 2048 + a.f[1]);
  __builtin_amdgcn_sched_barrier(0);
  compute_tile<QWIX_INT4, NT, SBF, RT, ZP>(b0, base0, sumx0, T, outacc);
  compute_tile<QWIX_INT4, NT, SBF, RT, ZP>(b1, base1, sumx1, T, outacc);
  if constexpr (T + 1 < NT) consume_panel<T + 1, H, NT, SBF, RT, ZP>(a, b0, b1, base0, base1, sumx0, sumx1, outacc);
}

// NWAVE wavefronts per workgroup, each owning a slice of K; NT tiles of 16 output columns, RT tiles of 16 rows
// (the weights are read, and widened, once per workgroup whatever RT is).
template <int BQT, int NWAVE, int NT, bool SBF, int RT = 1, bool ZP = false>
__global__ void __launch_bounds__(NWAVE * 64) gemv_wq_kernel(GemvArgs p) {
  extern __shared__ float red_raw[];
  float (*red)[RT * NT][4][64] = reinterpret_cast<float (*)[RT * NT][4][64]>(red_raw);  // [NWAVE]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int n_base = blockIdx.x * (16 * NT);
  const int nblk = p.K / 128;
  // K is dealt out in pairs of blocks, so that a wavefront's slice starts on an even block
  const int per_wave = 2 * ((nblk + 2 * NWAVE - 1) / (2 * NWAVE));
  const int kb0 = min(nblk, wave * per_wave), kb1 = min(nblk, kb0 + per_wave);

  const int row0 = blockIdx.y * (16 * RT);
  LaneOff<NT> a;
  a.bw = p.q + static_cast<int64_t>(n_base) * p.ldb;
  a.panel = reinterpret_cast<uint8_t*>(red_raw) + wave * (NT * 2048);
  // int4: the first pair of K blocks is on its way to LDS before anything else is worked out.  The key of panel
  // row 8 i + r is (4 i + (r >> 1)) & 7: it alternates between two values per lane.
  // Column tiles whose weights are requested before the activations and scales: one (M = 1, K 4096, N 14336 by the
  // number of early tiles out of four: one 8.44 us, two 8.82 us, three 9.00 us; with one the first products start
  // when a quarter of the wavefront's bytes are there).
  constexpr int H = 1;
  const unsigned grow = lane >> 3;
  unsigned gchunk[2];
  if constexpr (BQT == QWIX_INT4) {
#pragma unroll
    for (int odd = 0; odd < 2; ++odd) gchunk[odd] = static_cast<unsigned>((lane & 7) ^ ((4 * odd + (lane >> 4)) & 7)) * 16u;
    if (kb0 + 1 < kb1) fetch_panel<0, H>(p, a.bw, a.panel, grow, gchunk, n_base, kb0);
    __builtin_amdgcn_sched_barrier(0);
  }

  bool xrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) xrow[rt] = row0 + rt * 16 + col < p.M;
  a.x = static_cast<unsigned>(col) * static_cast<unsigned>(p.ldx) * 2u + kq * 64u;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const unsigned n = static_cast<unsigned>(min(t * 16 + col, p.N - 1 - n_base));
    a.s[t] = n * (SBF ? 2u : 4u);
    a.w[t] = n * static_cast<unsigned>(p.ldb) + kq * (BQT == QWIX_INT4 ? 16u : 32u);
  }
  a.bx = p.x + static_cast<int64_t>(row0) * p.ldx;
  a.bs = static_cast<const char*>(p.s) + static_cast<int64_t>(n_base) * (SBF ? 2 : 4);
  a.bz = ZP ? p.zp + n_base : nullptr;
  // fragment of K block h: chunk 4 h + kq of panel row col (the key of row 16 t + col does not depend on t)
#pragma unroll
  for (int h = 0; h < 2; ++h) a.f[h] = col * 128u + static_cast<unsigned>((h * 4 + kq) ^ ((col >> 1) & 7)) * 16u;

  v4f outacc[RT][NT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int t = 0; t < NT; ++t) outacc[rt][t] = v4f{0.f, 0.f, 0.f, 0.f};

  // Two K blocks per trip, all their loads issued before the first is consumed.  With int4 weights the first
  // column tile is requested first of all (for the first trip: before the address arithmetic of
  // everything else), then activations and scales, then the other tiles; the fences keep the scheduler from
  // moving anything across the hand-counted waits.
  int kb = kb0;
  for (; kb + 1 < kb1; kb += 2) {
    Block<BQT, NT, RT> b0, b1;
    if constexpr (BQT == QWIX_INT4) {
      load_blocks<BQT, NT, SBF, RT, true, false, ZP>(p, a, xrow, kb, &b0, &b1);
      __builtin_amdgcn_sched_barrier(0);
      fetch_panel<H, NT>(p, a.bw, a.panel, grow, gchunk, n_base, kb);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * (NT - H)));  // vmcnt: activations, scales and the first H tiles are here
      __builtin_amdgcn_sched_barrier(0);
      v4f base0[RT], base1[RT], sumx0[RT], sumx1[RT];
      prepare_x<BQT, NT, RT, ZP>(b0, base0, sumx0);
      prepare_x<BQT, NT, RT, ZP>(b1, base1, sumx1);
      consume_panel<0, H, NT, SBF, RT, ZP>(a, b0, b1, base0, base1, sumx0, sumx1, outacc);
      __builtin_amdgcn_sched_barrier(0);
      if (kb + 3 < kb1) fetch_panel<0, H>(p, a.bw, a.panel, grow, gchunk, n_base, kb + 2);
      __builtin_amdgcn_sched_barrier(0);
    } else {
      load_blocks<BQT, NT, SBF, RT, true, true, ZP>(p, a, xrow, kb, &b0, &b1);
      compute_block<BQT, NT, SBF, RT, ZP>(b0, outacc);
      compute_block<BQT, NT, SBF, RT, ZP>(b1, outacc);
    }
  }
  if (kb < kb1) {  // a last, single block
    Block<BQT, NT, RT> b0;
    load_blocks<BQT, NT, SBF, RT, false, true, ZP>(p, a, xrow, kb, &b0, &b0);
    compute_block<BQT, NT, SBF, RT, ZP>(b0, outacc);
  }

  if constexpr (BQT == QWIX_INT4) __syncthreads();  // the partial sums take the place of the weight panels
  // result lane layout: column n = lane % 16, row m = 4 * (lane / 16) + r; rows past M are neither written nor summed
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (row0 + rt * 16 + 4 * kq + r < p.M) {
#pragma unroll
        for (int t = 0; t < NT; ++t) red[wave][rt * NT + t][r][lane] = outacc[rt][t][r];
      }
  __syncthreads();
  for (int idx = tid; idx < RT * NT * 256; idx += NWAVE * 64) {
    const int t2 = idx >> 8, r = (idx >> 6) & 3, l = idx & 63;
    const int rt = t2 / NT, t = t2 % NT;
    const int mo = row0 + rt * 16 + 4 * (l >> 4) + r, n = n_base + t * 16 + (l & 15);
    if (mo < p.M && n < p.N) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < NWAVE; ++w) v += red[w][t2][r][l];
      if (p.out_dtype == QWIX_BF16)
        reinterpret_cast<uint16_t*>(p.out)[static_cast<int64_t>(mo) * p.ldo + n] = f32_to_bf16_bits(v);
      else
        reinterpret_cast<float*>(p.out)[static_cast<int64_t>(mo) * p.ldo + n] = v;
    }
  }
}

}  // namespace
}  // namespace qwix

using namespace qwix;

static int gemv_wq_impl(const void* x, int64_t ldx, const void* q, int64_t ldb_bytes, int b_qtype, int64_t M, int64_t N,
                        int64_t K, int64_t group, const void* s, int s_dtype, const int8_t* zp, void* out, int out_dtype,
                        int64_t ldo, void* stream) {
  if (!x || !q || !s || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null argument");
  if (M <= 0 || N <= 0 || K <= 0 || N > INT32_MAX || K > INT32_MAX || M > 65535 * 16)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (b_qtype != QWIX_INT4 && b_qtype != QWIX_INT8 && b_qtype != QWIX_E4M3)
    return fail(QWIX_ERR_UNSUPPORTED, "weight-only kernel takes int4, int8 or e4m3 weights (got qtype %d)", b_qtype);
  if (b_qtype == QWIX_E4M3 && zp) return fail(QWIX_ERR_INVALID_ARGUMENT, "float weights have no zero point");
  if (K % 128 || group <= 0 || group % 128 || K % group)
    return fail(QWIX_ERR_UNSUPPORTED, "K=%lld and group=%lld must be multiples of 128 with group | K", (long long)K,
                (long long)group);
  const int64_t brow = b_qtype == QWIX_INT4 ? K / 2 : K;
  if (ldx % 8 || ldx < K || ldb_bytes % 16 || ldb_bytes < brow || !aligned16(x) || !aligned16(q))
    return fail(QWIX_ERR_UNSUPPORTED, "x rows and weight rows must be 16-byte aligned");
  auto ok = [](int d) { return d == QWIX_F32 || d == QWIX_BF16; };
  if (!ok(s_dtype) || !ok(out_dtype) || ldo < N) return fail(QWIX_ERR_INVALID_ARGUMENT, "bad scale/output description");
  // per-lane offsets and the offsets that move along K are 31-bit: 32 rows of x, 64 rows of weights, all scale rows
  const int64_t es = s_dtype == QWIX_BF16 ? 2 : 4;
  if (32 * ldx * 2 + K * 2 > INT32_MAX || 64 * ldb_bytes + brow > INT32_MAX || (K / group) * N * es > INT32_MAX)
    return fail(QWIX_ERR_UNSUPPORTED, "row strides too large for 32-bit lane offsets");
  GemvArgs p;
  p.x = static_cast<const uint16_t*>(x); p.ldx = ldx;
  p.q = static_cast<const uint8_t*>(q); p.ldb = ldb_bytes;
  p.M = static_cast<int>(M); p.N = static_cast<int>(N); p.K = static_cast<int>(K);
  p.bpg = static_cast<int>(group / 128);
  p.magic = (0x100000000ull + p.bpg - 1) / p.bpg;
  p.s = s; p.s_dtype = s_dtype;
  p.zp = zp;
  p.out = out; p.out_dtype = out_dtype; p.ldo = ldo;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Byte weights of 32 MB and more stream faster through the smallest workgroups (4 wavefronts, two row tiles, several
  // workgroups per CU) whatever the rows, even when the second row tile is empty: K 4096, N 14336, int8, 1 / 16 / 32
  // rows 25.5 / 26.9 / 21.9 -> 16.2 / 17.5 / 21.0 us (8 wavefronts: 16.5 / 18.2), e4m3 21.9 / 23.8 -> 15.5 / 17.8;
  // K = N = 8192: 20.0 / 24.4 / 29.4 -> 17.8 / 20.0 / 26.9; at 16 MB (K = N = 4096) 9.3 against 10.2 us the other way
  // round, and int4 gains nothing at any size.
  const bool small_groups = b_qtype != QWIX_INT4 && N * K >= (int64_t{32} << 20);
#define QWIX_GEMV_KERNEL(KERN, NW, NTT, RTT)                                                                \
  do {                                                                                                     \
    /* the partial sums of all wavefronts; before them, in the same memory, the int4 weight panels */      \
    constexpr size_t smem = NW * NTT * (RTT * 1024 > 2048 ? RTT * 1024 : 2048);                            \
    static LdsGrant granted;                                                                               \
    if (smem >= 65536) if (int e_ = grant_lds(reinterpret_cast<const void*>(KERN), smem, granted)) return e_;\
    KERN<<<grid, NW * 64, smem, st>>>(p);                                                                  \
  } while (0)
#define QWIX_GEMV_LAUNCH_ZP(NW, NTT, RTT, ZPP)                                                             \
  do {                                                                                                     \
    const dim3 grid(static_cast<unsigned>((N + 16 * NTT - 1) / (16 * NTT)),                                \
                    static_cast<unsigned>((M + 16 * RTT - 1) / (16 * RTT)));                               \
    if (b_qtype == QWIX_INT4 && s_dtype == QWIX_BF16)                                                      \
      QWIX_GEMV_KERNEL((gemv_wq_kernel<QWIX_INT4, NW, NTT, true, RTT, ZPP>), NW, NTT, RTT);                \
    else if (b_qtype == QWIX_INT4)                                                                         \
      QWIX_GEMV_KERNEL((gemv_wq_kernel<QWIX_INT4, NW, NTT, false, RTT, ZPP>), NW, NTT, RTT);               \
    else if (b_qtype == QWIX_E4M3 && s_dtype == QWIX_BF16)                                                 \
      QWIX_GEMV_KERNEL((gemv_wq_kernel<QWIX_E4M3, NW, NTT, true, RTT, false>), NW, NTT, RTT);              \
    else if (b_qtype == QWIX_E4M3)                                                                         \
      QWIX_GEMV_KERNEL((gemv_wq_kernel<QWIX_E4M3, NW, NTT, false, RTT, false>), NW, NTT, RTT);             \
    else if (s_dtype == QWIX_BF16)                                                                         \
      QWIX_GEMV_KERNEL((gemv_wq_kernel<QWIX_INT8, NW, NTT, true, RTT, ZPP>), NW, NTT, RTT);                \
    else                                                                                                   \
      QWIX_GEMV_KERNEL((gemv_wq_kernel<QWIX_INT8, NW, NTT, false, RTT, ZPP>), NW, NTT, RTT);               \
  } while (0)
#define QWIX_GEMV_LAUNCH_RT(NW, NTT, RTT)                                                                  \
  do {                                                                                                     \
    if (zp) QWIX_GEMV_LAUNCH_ZP(NW, NTT, RTT, true); else QWIX_GEMV_LAUNCH_ZP(NW, NTT, RTT, false);        \
  } while (0)
#define QWIX_GEMV_LAUNCH(NW, NTT)                                                                          \
  do {                                                                                                     \
    if (M <= 16 && !small_groups) QWIX_GEMV_LAUNCH_RT(NW, NTT, 1);                                         \
    else if (M <= 32 && !small_groups) QWIX_GEMV_LAUNCH_RT(8, NTT, 2);                                     \
    else QWIX_GEMV_LAUNCH_RT(4, NTT, 2); /* several passes side by side: smaller workgroups, two per CU */  \
  } while (0)
  // Wider column tiles reuse each activation fragment more often; narrower ones keep every CU busy
  // when the weight matrix has few columns.
  if (N >= 192 * 64)
    QWIX_GEMV_LAUNCH(16, 4);
  else if (N >= 192 * 32)
    QWIX_GEMV_LAUNCH(16, 2);
  else
    QWIX_GEMV_LAUNCH(16, 1);
#undef QWIX_GEMV_LAUNCH
#undef QWIX_GEMV_LAUNCH_RT
#undef QWIX_GEMV_LAUNCH_ZP
#undef QWIX_GEMV_KERNEL
  return check_launch("gemv_wq");
}

extern "C" int qwix_hip_gemv_wq(const void* x, int64_t ldx, const void* q, int64_t ldb_bytes, int b_qtype, int64_t M,
                                int64_t N, int64_t K, int64_t group, const void* s, int s_dtype, void* out,
                                int out_dtype, int64_t ldo, void* stream) {
  return gemv_wq_impl(x, ldx, q, ldb_bytes, b_qtype, M, N, K, group, s, s_dtype, nullptr, out, out_dtype, ldo, stream);
}

extern "C" int qwix_hip_gemv_wq_zp(const void* x, int64_t ldx, const void* q, int64_t ldb_bytes, int b_qtype, int64_t M,
                                   int64_t N, int64_t K, int64_t group, const void* s, int s_dtype, const int8_t* zp,
                                   void* out, int out_dtype, int64_t ldo, void* stream) {
  if (!zp) return fail(QWIX_ERR_INVALID_ARGUMENT, "null zero points");
  return gemv_wq_impl(x, ldx, q, ldb_bytes, b_qtype, M, N, K, group, s, s_dtype, zp, out, out_dtype, ldo, stream);
}
