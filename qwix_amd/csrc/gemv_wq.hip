// Weight-only skinny GEMM (decode): bf16 activations x int4/int8 group-quantized weights.
//
//   out[m,n] = sum_g s[g,n] * sum_{k in g} x[m,k] * q[n,k]         M small (16 rows per pass)
//
// HBM-bound: the weight bytes are read exactly once, the activations stay in L2.  Even at M = 16
// the multiply-adds exceed what the vector ALUs can do in the time the weights stream in, so the
// products run on v_mfma_f32_16x16x32_bf16 with the weights converted to bf16 in registers, in
// offset binary so that the conversion is one or two bit-ops per pair of weights:
//   int4: (nibble ^ 8) lands in the mantissa of bf16 128.0, giving 128 + (q + 8) exactly;
//   int8: (byte ^ 0x80) is converted with v_cvt_f32_ubyte and truncated to bf16 (exact below 256).
// The offset is removed by seeding each accumulator with -offset * rowsum(x), which four MFMAs against
// a constant operand produce in the accumulator's own layout.
// A workgroup is 16 wavefronts that split K; each handles NT tiles of 16 output columns with two K
// blocks of loads in flight, and the partial sums meet in LDS.
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
};

// Addresses are a wave-uniform 64-bit base plus a per-lane unsigned 32-bit byte offset that is fixed
// for the whole kernel, so that a load costs no vector arithmetic.  Columns beyond N are clamped to
// the last valid one instead of being predicated: an output element depends only on its own row of
// x and its own column of the weights, and the clamped ones are never stored.
template <int NT>
struct LaneOff {
  unsigned x;      // bytes from the first row of this workgroup's 16 rows of x
  unsigned w[NT];  // bytes from row n_base of the weights
  unsigned s[NT];  // elements from column n_base of the scales
};

template <int BQT, int NT, bool SBF, int RT>
__device__ __forceinline__ void load_block(const GemvArgs& p, const LaneOff<NT>& a, const bool (&xrow)[RT], int row0,
                                           int n_base, int kb, Block<BQT, NT, RT>* b) {
  constexpr bool W4 = (BQT == QWIX_INT4);
  const char* xb = reinterpret_cast<const char*>(p.x + static_cast<int64_t>(row0) * p.ldx + kb * 128);
  // every vector load occupies the texture path for as long as its active lanes need, also when they
  // repeat an address: lanes whose row of x does not exist stay idle and feed zeros to the MFMA
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const char* xr = xb + static_cast<int64_t>(rt) * 32 * p.ldx;  // 16 rows of bf16 further down
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      b->xf[rt][j] = v4u{0, 0, 0, 0};
      if (xrow[rt]) b->xf[rt][j] = *reinterpret_cast<const v4u*>(xr + a.x + j * 16);
    }
  }
  const int sg = static_cast<int>((static_cast<uint64_t>(static_cast<unsigned>(kb)) * p.magic) >> 32);
  const int64_t s0 = static_cast<int64_t>(sg) * p.N + n_base;
  const uint8_t* wb = p.q + static_cast<int64_t>(n_base) * p.ldb + kb * (W4 ? 64 : 128);
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    b->wq[t][0] = *reinterpret_cast<const v4u*>(wb + a.w[t]);
    if constexpr (!W4) b->wq[t][1] = *reinterpret_cast<const v4u*>(wb + a.w[t] + 16);
    if constexpr (SBF)
      b->sraw[t] = (reinterpret_cast<const uint16_t*>(p.s) + s0)[a.s[t]];
    else
      b->sraw[t] = (reinterpret_cast<const unsigned*>(p.s) + s0)[a.s[t]];
  }
}

// Weights enter the MFMA in offset binary (int4: 128 + (q + 8), int8: q + 128, both exact in bf16);
// the offset times the row sum of x is taken out by four MFMAs against the constant -offset, whose
// result seeds the accumulator of every column tile.  A widened weight fragment serves all RT row tiles; every
// output element sees the same operations in the same order whatever RT is.
template <int BQT, int NT, bool SBF, int RT>
__device__ __forceinline__ void compute_block(Block<BQT, NT, RT>& b, v4f (&outacc)[RT][NT]) {
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
  v4f base[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    base[rt] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j)
      base[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xf[rt][j]), as_bf16x8(negoff), base[rt], 0, 0, 0);
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) {
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
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xf[rt][j]), as_bf16x8(w), acc[rt], 0, 0, 0);
    }
    const float sc = __uint_as_float(SBF ? b.sraw[t] << 16 : b.sraw[t]);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int r = 0; r < 4; ++r) outacc[rt][t][r] = fmaf(acc[rt][r], sc, outacc[rt][t][r]);
  }
}

// NWAVE wavefronts per workgroup, each owning a slice of K; NT tiles of 16 output columns, RT tiles of 16 rows
// (the weights are read, and widened, once per workgroup whatever RT is).
template <int BQT, int NWAVE, int NT, bool SBF, int RT = 1>
__global__ void __launch_bounds__(NWAVE * 64) gemv_wq_kernel(GemvArgs p) {
  extern __shared__ float red_raw[];
  float (*red)[RT * NT][4][64] = reinterpret_cast<float (*)[RT * NT][4][64]>(red_raw);  // [NWAVE]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int n_base = blockIdx.x * (16 * NT);
  const int nblk = p.K / 128;
  const int per_wave = (nblk + NWAVE - 1) / NWAVE;
  const int kb0 = wave * per_wave, kb1 = min(nblk, kb0 + per_wave);

  const int row0 = blockIdx.y * (16 * RT);
  LaneOff<NT> a;
  bool xrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) xrow[rt] = row0 + rt * 16 + col < p.M;
  a.x = static_cast<unsigned>(col) * static_cast<unsigned>(p.ldx) * 2u + kq * 64u;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    a.s[t] = static_cast<unsigned>(min(t * 16 + col, p.N - 1 - n_base));
    a.w[t] = a.s[t] * static_cast<unsigned>(p.ldb) + kq * (BQT == QWIX_INT4 ? 16u : 32u);
  }

  v4f outacc[RT][NT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int t = 0; t < NT; ++t) outacc[rt][t] = v4f{0.f, 0.f, 0.f, 0.f};

  // Two K blocks per trip, all their loads issued before the first is consumed.  Nothing loaded is
  // carried from one trip to the next; the other wavefronts of the SIMD cover the gap.
  for (int kb = kb0; kb < kb1; kb += 2) {
    Block<BQT, NT, RT> b0, b1;
    const bool two = kb + 1 < kb1;
    load_block<BQT, NT, SBF, RT>(p, a, xrow, row0, n_base, kb, &b0);
    if (two) load_block<BQT, NT, SBF, RT>(p, a, xrow, row0, n_base, kb + 1, &b1);
    compute_block<BQT, NT, SBF, RT>(b0, outacc);
    if (two) compute_block<BQT, NT, SBF, RT>(b1, outacc);
  }

#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][rt * NT + t][r][lane] = outacc[rt][t][r];
  __syncthreads();
  // result lane layout: column n = lane % 16, row m = 4 * (lane / 16) + r
  for (int idx = tid; idx < RT * NT * 256; idx += NWAVE * 64) {
    const int t2 = idx >> 8, r = (idx >> 6) & 3, l = idx & 63;
    const int rt = t2 / NT, t = t2 % NT;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < NWAVE; ++w) v += red[w][t2][r][l];
    const int mo = row0 + rt * 16 + 4 * (l >> 4) + r, n = n_base + t * 16 + (l & 15);
    if (mo < p.M && n < p.N) {
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

extern "C" int qwix_hip_gemv_wq(const void* x, int64_t ldx, const void* q, int64_t ldb_bytes, int b_qtype, int64_t M,
                                int64_t N, int64_t K, int64_t group, const void* s, int s_dtype, void* out,
                                int out_dtype, int64_t ldo, void* stream) {
  if (!x || !q || !s || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null argument");
  if (M <= 0 || N <= 0 || K <= 0 || N > INT32_MAX || K > INT32_MAX || M > 65535 * 16)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (b_qtype != QWIX_INT4 && b_qtype != QWIX_INT8)
    return fail(QWIX_ERR_UNSUPPORTED, "weight-only kernel takes int4 or int8 weights (got qtype %d)", b_qtype);
  if (K % 128 || group <= 0 || group % 128 || K % group)
    return fail(QWIX_ERR_UNSUPPORTED, "K=%lld and group=%lld must be multiples of 128 with group | K", (long long)K,
                (long long)group);
  const int64_t brow = b_qtype == QWIX_INT4 ? K / 2 : K;
  if (ldx % 8 || ldx < K || ldb_bytes % 16 || ldb_bytes < brow || !aligned16(x) || !aligned16(q))
    return fail(QWIX_ERR_UNSUPPORTED, "x rows and weight rows must be 16-byte aligned");
  auto ok = [](int d) { return d == QWIX_F32 || d == QWIX_BF16; };
  if (!ok(s_dtype) || !ok(out_dtype) || ldo < N) return fail(QWIX_ERR_INVALID_ARGUMENT, "bad scale/output description");
  if (16 * ldx * 2 > INT32_MAX || 64 * ldb_bytes > INT32_MAX)
    return fail(QWIX_ERR_UNSUPPORTED, "row strides too large for 32-bit lane offsets");
  GemvArgs p;
  p.x = static_cast<const uint16_t*>(x); p.ldx = ldx;
  p.q = static_cast<const uint8_t*>(q); p.ldb = ldb_bytes;
  p.M = static_cast<int>(M); p.N = static_cast<int>(N); p.K = static_cast<int>(K);
  p.bpg = static_cast<int>(group / 128);
  p.magic = (0x100000000ull + p.bpg - 1) / p.bpg;
  p.s = s; p.s_dtype = s_dtype;
  p.out = out; p.out_dtype = out_dtype; p.ldo = ldo;
  hipStream_t st = static_cast<hipStream_t>(stream);
#define QWIX_GEMV_KERNEL(KERN, NW, NTT, RTT)                                                                \
  do {                                                                                                     \
    constexpr size_t smem = sizeof(float) * NW * RTT * NTT * 4 * 64;                                       \
    static LdsGrant granted;                                                                               \
    if (smem >= 65536) if (int e_ = grant_lds(reinterpret_cast<const void*>(KERN), smem, granted)) return e_;\
    KERN<<<grid, NW * 64, smem, st>>>(p);                                                                  \
  } while (0)
#define QWIX_GEMV_LAUNCH_RT(NW, NTT, RTT)                                                                  \
  do {                                                                                                     \
    const dim3 grid(static_cast<unsigned>((N + 16 * NTT - 1) / (16 * NTT)),                                \
                    static_cast<unsigned>((M + 16 * RTT - 1) / (16 * RTT)));                               \
    if (b_qtype == QWIX_INT4 && s_dtype == QWIX_BF16)                                                      \
      QWIX_GEMV_KERNEL((gemv_wq_kernel<QWIX_INT4, NW, NTT, true, RTT>), NW, NTT, RTT);                     \
    else if (b_qtype == QWIX_INT4)                                                                         \
      QWIX_GEMV_KERNEL((gemv_wq_kernel<QWIX_INT4, NW, NTT, false, RTT>), NW, NTT, RTT);                    \
    else if (s_dtype == QWIX_BF16)                                                                         \
      QWIX_GEMV_KERNEL((gemv_wq_kernel<QWIX_INT8, NW, NTT, true, RTT>), NW, NTT, RTT);                     \
    else                                                                                                   \
      QWIX_GEMV_KERNEL((gemv_wq_kernel<QWIX_INT8, NW, NTT, false, RTT>), NW, NTT, RTT);                    \
  } while (0)
#define QWIX_GEMV_LAUNCH(NW, NTT)                                                                          \
  do {                                                                                                     \
    if (M <= 16) QWIX_GEMV_LAUNCH_RT(NW, NTT, 1);                                                          \
    else if (M <= 32) QWIX_GEMV_LAUNCH_RT(8, NTT, 2);                                                      \
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
#undef QWIX_GEMV_KERNEL
  return check_launch("gemv_wq");
}
