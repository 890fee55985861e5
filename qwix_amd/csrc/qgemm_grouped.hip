// Sub-channel quantized GEMM: int8 activations x int8/int4 weights with one weight scale per
// group of `group` K-elements (and optionally per-group activation scales).
//
//   out[m,n] = cast( sum_g ((T(acc_g[m,n]) * sa[m,g']) * sb[g,n]) ),  acc_g = sum_{k in g} a[m,k] b[n,k]
//
// Same tiling as the per-channel kernel (128 x 128 output tile, 2 x 2 wavefronts, 128-byte K slabs
// through two LDS stages, v_mfma_i32_32x32x32_i8) with two differences:
//   * int4 weights travel packed through LDS and are widened in registers: every nibble becomes
//     the HIGH nibble of a byte (value x 16, sign kept), which costs three bit-ops per 8 values;
//     the activation fragment is byte-permuted to the same K order, and the factor 16 is folded
//     into the weight scale (exact: a power of two);
//   * at each group boundary the int32 partial is converted, scaled by sb[g, n] and added to an
//     f32 accumulator; the int32 accumulator restarts from zero.
// The lane that owns column n of the MFMA result owns it for all its registers, so one weight scale
// per 32x32 tile and group is enough.  The result leaves through LDS so that global stores are
// 16-byte and row-contiguous.
#include <type_traits>

#include "common.h"

namespace qwix {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
// LDS reads inside the main loops go through these, never through HIP's struct vectors (float4, int4): behind a
// struct-typed LDS access the compiler waits for every direct-to-LDS load in flight (vmcnt 0), the slabs requested
// ahead included.
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int BM = 128, BN = 128, BK = 128, TM = 2, TN = 2, kPad = 16;

struct GroupedArgs {
  const uint8_t* A; int64_t lda;
  const uint8_t* B; int64_t ldb;
  int M, N, K, group;
  const void* sa; int sa_dtype; int ga;
  const void* sb; int sb_dtype;
  int t_dtype;      // dtype of the scaled partials (promotion of the scale dtypes, and of acc_dtype for e4m3)
  int acc_dtype;    // e4m3 operands: the dtype each group's f32 dot is rounded to before it is scaled
  uint8_t* out; int out_dtype; int64_t ldo;
  int32_t* acc_out;
  // Zero-point correction of an asymmetric operand, per group: acc_g[m,n] -= zu[m,g] * zv[g,n].  One array
  // holds zero points, the other the per-group K-sums of the opposite operand; element strides, 0 along the
  // group axis for an array that is the same for all groups.  Both null: symmetric operands.
  const int32_t* zu; int64_t zu_sm, zu_sg;
  const int32_t* zv; int64_t zv_sn, zv_sg;
  // One group spans all of K (int4 weights with per-channel scales): the fast kernel then scales like the untiled
  // contraction, ((T(acc) * sx) * sy) with a rounding per step (dot_general.py:255-261), not like a sum of partials.
  int single;
  // K in ranges (0: none): workgroups with blockIdx.y = y contract elements [y ksplit, (y + 1) ksplit) -- whole groups --
  // and write the f32 sums of their scaled partials, without the activation scale and the final rounding, as the y-th
  // M x N array at `out` (the host passes f32, ldo = N, sa = null); grouped_reduce_kernel finishes.
  int ksplit;
};

__device__ __forceinline__ float ld_scale(const void* p, int dtype, int64_t i) {
  return dtype == QWIX_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i])
                            : reinterpret_cast<const float*>(p)[i];
}

template <int BQT, bool EXACT>
__global__ void __launch_bounds__(256) qgemm_grouped_kernel(GroupedArgs p) {
  constexpr bool W4 = (BQT == QWIX_INT4);
  constexpr bool F8 = (BQT == QWIX_E4M3);  // both operands e4m3, f32 partial per group (v_mfma_f32_32x32x64_f8f6f4)
  using AccV = typename std::conditional<F8, v16f, v16i>::type;
  constexpr int A_STRIDE = BK + kPad;
  constexpr int B_ROW = W4 ? BK / 2 : BK;
  constexpr int B_STRIDE = B_ROW + kPad;
  constexpr int STAGE = BM * A_STRIDE + BN * B_STRIDE;
  constexpr int A_CH = BK / 16, B_CH = B_ROW / 16;
  constexpr int A_LOADS = BM * A_CH / 256, B_LOADS = BN * B_CH / 256;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (p.N + BN - 1) / BN;
  int pid = blockIdx.x;
  if ((gridDim.x & 7) == 0) pid = (pid & 7) * (gridDim.x >> 3) + (pid >> 3);  // one XCD, one run of tiles
  const int m0 = (pid / tiles_n) * BM, n0 = (pid % tiles_n) * BN;

  AccV acc[TM][TN];
  float accf[TM][TN][16];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        acc[i][j][r] = 0;
        accf[i][j][r] = 0.f;
      }

  uint4 ra[A_LOADS], rb[B_LOADS];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int c = tid + i * 256, row = c / A_CH, kc = c % A_CH;
      const int m = m0 + row, k = k0 + kc * 16;
      ra[i] = (m < p.M && k < p.K) ? *reinterpret_cast<const uint4*>(p.A + static_cast<int64_t>(m) * p.lda + k)
                                   : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int c = tid + i * 256, row = c / B_CH, kc = c % B_CH;
      const int n = n0 + row, k = k0 + kc * (W4 ? 32 : 16);
      rb[i] = (n < p.N && k < p.K)
                  ? *reinterpret_cast<const uint4*>(p.B + static_cast<int64_t>(n) * p.ldb + (W4 ? k / 2 : k))
                  : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_lds = [&](int s) {
    uint8_t* base = smem + s * STAGE;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int c = tid + i * 256, row = c / A_CH, kc = c % A_CH;
      *reinterpret_cast<uint4*>(base + row * A_STRIDE + kc * 16) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
      const int c = tid + i * 256, row = c / B_CH, kc = c % B_CH;
      *reinterpret_cast<uint4*>(base + BM * A_STRIDE + row * B_STRIDE + kc * 16) = rb[i];
    }
  };
  auto compute = [&](int s) {
    const uint8_t* pa = smem + s * STAGE + (wm * (BM / 2) + (lane & 31)) * A_STRIDE;
    const uint8_t* pb = smem + s * STAGE + BM * A_STRIDE + (wn * (BN / 2) + (lane & 31)) * B_STRIDE;
    if constexpr (F8) {
      // a lane holds 32 consecutive bytes of its row per k-step of 64
#pragma unroll
      for (int ks = 0; ks < BK / 64; ++ks) {
        v8i fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const uint8_t* q = pa + i * 32 * A_STRIDE + ks * 64 + (lane >> 5) * 32;
          const v4i lo = *reinterpret_cast<const v4i*>(q), hi = *reinterpret_cast<const v4i*>(q + 16);
          fa[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const uint8_t* q = pb + j * 32 * B_STRIDE + ks * 64 + (lane >> 5) * 32;
          const v4i lo = *reinterpret_cast<const v4i*>(q), hi = *reinterpret_cast<const v4i*>(q + 16);
          fb[j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], 0, 0, 0, 0, 0, 0);
      }
      return;
    } else {
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      v4i fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const v4i t = *reinterpret_cast<const v4i*>(pa + i * 32 * A_STRIDE + ks * 32 + (lane >> 5) * 16);
        if constexpr (W4) {  // K order (0,2,4,6 | 1,3,5,7 | 8,10,12,14 | 9,11,13,15), as the widened nibbles
          fa[i][0] = __builtin_amdgcn_perm(t[1], t[0], 0x06040200);
          fa[i][1] = __builtin_amdgcn_perm(t[1], t[0], 0x07050301);
          fa[i][2] = __builtin_amdgcn_perm(t[3], t[2], 0x06040200);
          fa[i][3] = __builtin_amdgcn_perm(t[3], t[2], 0x07050301);
        } else {
          fa[i] = t;
        }
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if constexpr (W4) {
          const uint2 q = *reinterpret_cast<const uint2*>(pb + j * 32 * B_STRIDE + ks * 16 + (lane >> 5) * 8);
          fb[j][0] = static_cast<int>((q.x << 4) & 0xF0F0F0F0u);
          fb[j][1] = static_cast<int>(q.x & 0xF0F0F0F0u);
          fb[j][2] = static_cast<int>((q.y << 4) & 0xF0F0F0F0u);
          fb[j][3] = static_cast<int>(q.y & 0xF0F0F0F0u);
        } else {
          fb[j] = *reinterpret_cast<const v4i*>(pb + j * 32 * B_STRIDE + ks * 32 + (lane >> 5) * 16);
        }
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    }
  };

  // acc[i][j][r]: m = m0 + wm*64 + i*32 + 8*(r/4) + 4*(lane/32) + r%4,  n = n0 + wn*(BN/2) + j*32 + lane%32.
  auto row_of = [&](int i, int r) { return m0 + wm * (BM / 2) + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); };
  auto col_of = [&](int j) { return n0 + wn * (BN / 2) + j * 32 + (lane & 31); };

  auto flush = [&](int g) {
    float sbv[TN];
    int zvv[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = col_of(j);
      sbv[j] = n < p.N ? ld_scale(p.sb, p.sb_dtype, static_cast<int64_t>(g) * p.N + n) : 0.f;
      zvv[j] = (p.zu != nullptr && n < p.N) ? p.zv[n * p.zv_sn + g * p.zv_sg] : 0;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = row_of(i, r);
        float sav = 1.f;
        if (p.sa != nullptr && (EXACT || F8 || p.ga > 1) && m < p.M)
          sav = ld_scale(p.sa, p.sa_dtype, static_cast<int64_t>(m) * p.ga + (p.ga > 1 ? g : 0));
        const int zuv = (p.zu != nullptr && m < p.M) ? p.zu[m * p.zu_sm + g * p.zu_sg] : 0;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          if constexpr (F8) {
            // dot_general.py:214-260 for float operands: the group's dot is delivered in the accumulator dtype, then
            // scaled lhs first, every step in the promotion of the types met so far, one rounding per step
            float v = acc[i][j][r];
            bool bf = (p.acc_dtype == QWIX_BF16);
            if (bf) v = round_bf16(v);
            if (p.sa != nullptr) {
              bf = bf && p.sa_dtype == QWIX_BF16;
              v *= sav;
              if (bf) v = round_bf16(v);
            }
            bf = bf && p.sb_dtype == QWIX_BF16;
            v *= sbv[j];
            if (bf) v = round_bf16(v);
            accf[i][j][r] += v;
            acc[i][j][r] = 0;
            continue;
          } else {
          // int4 weights were widened to 16 x value: the partial is an exact multiple of 16
          const int raw = (W4 ? (acc[i][j][r] >> 4) : acc[i][j][r]) - zuv * zvv[j];
          if (p.acc_out != nullptr && m < p.M && col_of(j) < p.N)
            p.acc_out[(static_cast<int64_t>(g) * p.M + m) * p.N + col_of(j)] = raw;
          float v = static_cast<float>(raw);
          if constexpr (EXACT) {
            // (T(acc) * sa) * sb with one rounding per step, as the reference computes it.
            if (p.sa != nullptr) {
              if (p.sa_dtype == QWIX_BF16) v = round_bf16(round_bf16(v) * sav); else v = v * sav;
            }
            const bool tb = (p.t_dtype == QWIX_BF16);
            if (tb) v = round_bf16(round_bf16(v) * sbv[j]); else v = v * sbv[j];
            accf[i][j][r] += v;
          } else {
            accf[i][j][r] = __builtin_fmaf(v, (p.ga > 1 ? sav : 1.f) * sbv[j], accf[i][j][r]);
          }
          acc[i][j][r] = 0;
          }
        }
      }
  };

  const int KT = (p.K + BK - 1) / BK;
  const int tiles_per_group = p.group / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < KT) load_global((kt + 1) * BK);
    compute(cur);
    if ((kt + 1) % tiles_per_group == 0) flush(kt / tiles_per_group);
    if (kt + 1 < KT) store_lds(cur ^ 1);
    __syncthreads();
  }

  // Epilogue through LDS: each wavefront stages 32 rows x (BN/2) columns of f32 at a time.
  constexpr int WCOLS = BN / 2;
  constexpr int ROW_F = WCOLS + 4;  // floats per staged row (+ 4 padding)
  constexpr int CPR = WCOLS / 4;    // 16-byte chunks per staged row
  float* stage = reinterpret_cast<float*>(smem) + wave * (32 * ROW_F);
  const bool t_bf16 = (p.t_dtype == QWIX_BF16);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float v = accf[i][j][r];
        if (!EXACT && !F8 && p.sa != nullptr && p.ga == 1) {
          const int m = row_of(i, r);
          v *= (m < p.M) ? ld_scale(p.sa, p.sa_dtype, m) : 0.f;
        }
        if (t_bf16) v = round_bf16(v);  // the sum over groups is cast back to the partials' dtype
        stage[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * ROW_F + j * 32 + (lane & 31)] = v;
      }
#pragma unroll
    for (int c = 0; c < 32 * CPR / 64; ++c) {
      const int chunk = lane + 64 * c, row = chunk / CPR, cc = chunk % CPR;
      const int m = m0 + wm * (BM / 2) + i * 32 + row, n = n0 + wn * (BN / 2) + cc * 4;
      if (m >= p.M || n >= p.N) continue;
      const float4 v = *reinterpret_cast<const float4*>(stage + row * ROW_F + cc * 4);
      const float vv[4] = {v.x, v.y, v.z, v.w};
      if (p.out_dtype == QWIX_BF16) {
        uint16_t* o = reinterpret_cast<uint16_t*>(p.out) + static_cast<int64_t>(m) * p.ldo + n;
        if (n + 3 < p.N && (p.ldo & 3) == 0) {
          *reinterpret_cast<uint2*>(o) =
              make_uint2(f32_to_bf16_bits(vv[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(vv[1])) << 16),
                         f32_to_bf16_bits(vv[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(vv[3])) << 16));
        } else {
          _Pragma("unroll") for (int e = 0; e < 4; ++e)
            if (n + e < p.N) o[e] = f32_to_bf16_bits(vv[e]);
        }
      } else {
        float* o = reinterpret_cast<float*>(p.out) + static_cast<int64_t>(m) * p.ldo + n;
        if (n + 3 < p.N && (p.ldo & 3) == 0) {
          *reinterpret_cast<float4*>(o) = v;
        } else {
          _Pragma("unroll") for (int e = 0; e < 4; ++e)
            if (n + e < p.N) o[e] = vv[e];
        }
      }
    }
  }
}

template <int BQT, bool EXACT>
int launch_grouped(const GroupedArgs& p, hipStream_t st) {
  constexpr bool W4 = (BQT == QWIX_INT4);
  constexpr size_t stage = BM * (BK + kPad) + BN * ((W4 ? BK / 2 : BK) + kPad);
  constexpr size_t epi = 4 * 32 * (BN / 2 + 4) * sizeof(float);
  constexpr size_t smem = 2 * stage > epi ? 2 * stage : epi;
  auto kern = qgemm_grouped_kernel<BQT, EXACT>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  const int64_t tiles = static_cast<int64_t>((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  kern<<<dim3(static_cast<unsigned>(tiles)), 256, smem, st>>>(p);
  return check_launch("qgemm_grouped");
}


// ------------------------------------------------------------------------------------------------
// Fast path (no per-partial rounding, per-token or no activation scale, no accumulator dump).
//
// 128 x 256 output tile, 8 wavefronts side by side along N, each owning all 128 rows of 32 columns
// (4 MFMA tiles that share one weight fragment, so the int4 widening is paid once per 4 MFMAs).  The
// 128-wide K slabs travel global -> LDS directly in 1 KiB pieces, XOR-swizzled per 16-byte chunk so
// that the fragment reads are bank-conflict free:
//   A  (int8, 128 B per row):  8 rows per KiB, chunk c of row r sits at position c ^ ((r >> 1) & 7);
//   B  (int4,  64 B per row): 16 rows per KiB, chunk c of row r sits at position c ^ ((r >> 2) & 3).
// One 16-byte chunk of packed int4 holds 32 consecutive k; a lane consumes it over two k-steps, and
// the A fragments of those two k-steps are the two 16-byte chunks with the same 32 k.  The widened
// nibbles (x 16, sign kept) are byte-permuted into natural K order, so A goes to the MFMA untouched.
// The first k-step of a group starts from a zero accumulator operand; at the end of a group each
// int32 partial costs one convert and one FMA.  LDS then becomes staging space for row-contiguous
// 16-byte stores, where the per-token scale is applied once per row.
#define QWIX_GLDS16(gptr, lptr)                                                                       \
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gptr),             \
                                   (__attribute__((address_space(3))) void*)(lptr), 16, 0, 0)

struct Fast {
  static constexpr int kBM = 128, kBN = 256, kBK = 128, kNW = 8, kTM = 4;
};
// The same kernel with two wavefronts and 64 columns per workgroup: four times the workgroups, for problems whose
// 128 x 256 tiles would leave most of the chip idle (a few hundred rows, or decode batches, against a weight of a few
// thousand columns).
struct Narrow {
  static constexpr int kBM = 128, kBN = 64, kBK = 128, kNW = 2, kTM = 4;
};
// ... and with 64 or 32 rows for decode batches: a quarter of the MFMAs and folds per slab where the other rows of a
// 128-row tile would be padding.
struct Narrow64 {
  static constexpr int kBM = 64, kBN = 64, kBK = 128, kNW = 2, kTM = 2;
};
struct Narrow32 {
  static constexpr int kBM = 32, kBN = 64, kBK = 128, kNW = 2, kTM = 1;
};

// SAG: the activations carry one scale per row and group as well (both operands tiled along K): the
// tile's (groups x 128 rows) scales are converted to f32 and parked in LDS behind the slab stages; folding a
// group in then takes convert, multiply, FMA per accumulator instead of convert, FMA.
// AUX: the instantiation for asymmetric operands and for parity runs.  Loads, LDS layout, MFMA sequence and
// epilogue are the ones of the plain instantiation; only the fold of a finished group differs: the int32
// partial is taken as a plain integer (int4: shifted back by the factor 16 of the widening), corrected by
// zu[m,g] * zv[g,n] when an operand is asymmetric, written to acc_out when that is given, then scaled.
// MAGIC (groups of exactly 128, bf16 partials, per-token or no activation scale): the first MFMA of a group
// starts from the integer 0x4B400000 in every accumulator instead of 0.  The group's partial p satisfies
// |p| < 2^22, so the finished accumulator, read as a float, IS 1.5 * 2^23 + p exactly, and folding the group in
// is one FMA per accumulator (no integer-to-float conversion).  The constants C * sb[g,n] that this adds are
// tracked per lane (a lane owns one column) and taken out every fourth group, so the running sums stay within
// 4 * C * sb and the f32 rounding they pick up is about 2^-12 of a partial: far inside the 2^-9 the reference
// itself spends on rounding every scaled partial to bf16.
// ST: slab stages in LDS.  With 3, the loads of slab k+2 are issued at the start of slab k and get two slabs of
// time to land; the wait before the barrier that ends slab k leaves them in flight (vmcnt counts oldest first).
// ONE: every group is one slab (group == 128): the main loop then has a single straight-line body.
// DUMP (with AUX): the corrected partials are also written to acc_out (parity runs).
template <int BQT, bool SBF, bool SAG, bool AUX, bool MAGIC = false, int ST = 2, bool ONE = false, bool DUMP = false,
          typename G = Fast>
__global__ void __launch_bounds__(G::kNW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
    qgemm_grouped_dma_kernel(GroupedArgs p) {
  constexpr int BM = G::kBM, BN = G::kBN, BK = G::kBK, NW = G::kNW, TM = G::kTM;
  constexpr int WR = 1;  // every wavefront owns all rows of its 32 columns
  constexpr bool W4 = (BQT == QWIX_INT4);
  if (p.ksplit > 0) {  // this workgroup's range of K: every operand moves to its first element
    const int y = blockIdx.y, k0 = y * p.ksplit;
    p.A += k0;
    p.B += W4 ? k0 / 2 : k0;
    p.sb = static_cast<const uint8_t*>(p.sb) + static_cast<int64_t>(k0 / p.group) * p.N * (SBF ? 2 : 4);
    p.out += static_cast<int64_t>(y) * p.M * p.N * 4;
    p.K = p.ksplit;
  }
  // e4m3 x e4m3: bytes travel like int8; two 16-byte fragments of consecutive k-steps make one operand of
  // v_mfma_f32_32x32x64_f8f6f4 (both operands take the same 32 of the 64 k per lane half, so the dot is complete),
  // the group's partial is f32 already.  Never MAGIC, never AUX.
  constexpr bool F8 = (BQT == QWIX_E4M3);
  static_assert(!F8 || (!MAGIC && !AUX), "e4m3 operands have neither int32 partials nor zero points");
  using AccV = typename std::conditional<F8, v16f, v16i>::type;
  constexpr int B_ROWB = W4 ? 64 : 128;          // bytes of one B row in a slab
  constexpr int A_BYTES = BM * BK, B_BYTES = BN * B_ROWB, STAGE = A_BYTES + B_BYTES;
  constexpr int A_LOADS = A_BYTES / 1024 / NW;   // KiB pieces per wavefront and slab
  constexpr int B_LOADS = B_BYTES / 1024 / NW;
  constexpr int B_RPL = 1024 / B_ROWB;           // B rows per KiB piece
  constexpr int NK = BK / 32;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wc = wave % (NW / WR), wr = wave / (NW / WR);   // column group, row group of this wavefront
  constexpr int WROWS = BM / WR;                              // rows per wavefront
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  int tile_m, tile_n;
  {  // every XCD gets a contiguous run of tiles; tiles walk down 8 tile-rows before moving along N
    const int nb = gridDim.x;
    int pid = blockIdx.x;
    if ((nb & 7) == 0) pid = (pid & 7) * (nb >> 3) + (pid >> 3);
    constexpr int GM = 8;
    const int per_group = GM * tiles_n, grp = pid / per_group, first_m = grp * GM;
    const int gsz = min(tiles_m - first_m, GM);
    tile_m = first_m + (pid % per_group) % gsz;
    tile_n = (pid % per_group) / gsz;
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  float* sa_lds = reinterpret_cast<float*>(smem + ST * STAGE);  // [group][row of the tile]
  if constexpr (SAG) {
    const int ng = p.K / p.group;
    for (int idx = tid; idx < ng * BM; idx += NW * 64) {
      const int row = idx & (BM - 1), g = idx / BM;
      const int m = min(m0 + row, p.M - 1);
      sa_lds[idx] = ld_scale(p.sa, p.sa_dtype, static_cast<int64_t>(m) * p.ga + g);
    }
  }
  // zero-point side values of the tile's rows, [group or 0][row], behind the activation scales
  int* zu_lds = reinterpret_cast<int*>(smem + ST * STAGE) + (SAG ? (p.K / p.group) * BM : 0);
  if constexpr (AUX) {
    if (p.zu != nullptr) {
      const int gz = p.zu_sg != 0 ? p.K / p.group : 1;
      for (int idx = tid; idx < gz * BM; idx += NW * 64) {
        const int row = idx & (BM - 1), g = idx / BM;
        zu_lds[idx] = p.zu[static_cast<int64_t>(min(m0 + row, p.M - 1)) * p.zu_sm + g * p.zu_sg];
      }
    }
  }

  // ---- loader: wave-uniform 64-bit tile base + per-lane 32-bit offset, rows clamped to the last valid one
  const uint8_t* a_base = p.A + static_cast<int64_t>(m0) * p.lda;
  const uint8_t* b_base = p.B + static_cast<int64_t>(n0) * p.ldb;
  uint32_t a_off[A_LOADS], b_off[B_LOADS];
#pragma unroll
  for (int j = 0; j < A_LOADS; ++j) {
    const int row = (j * NW + wave) * 8 + (lane >> 3);
    a_off[j] = static_cast<uint32_t>(min(row, p.M - 1 - m0)) * static_cast<uint32_t>(p.lda) + (((lane & 7) ^ swz128(row)) << 4);
  }
#pragma unroll
  for (int j = 0; j < B_LOADS; ++j) {
    int row, chunk;
    if constexpr (W4) {
      row = (j * NW + wave) * 16 + (lane >> 2);
      chunk = (lane & 3) ^ ((lane >> 4) & 3);
    } else {
      row = (j * NW + wave) * 8 + (lane >> 3);
      chunk = (lane & 7) ^ swz128(row);
    }
    b_off[j] = static_cast<uint32_t>(min(row, p.N - 1 - n0)) * static_cast<uint32_t>(p.ldb) + (chunk << 4);
  }
  auto issue_loads = [&](int s, int kt) __attribute__((always_inline)) {
    const uint8_t* ga = a_base + kt * BK;
    const uint8_t* gb = b_base + kt * B_ROWB;
    uint8_t* ls = smem + s * STAGE;
    // The 32-bit lane offsets are made opaque here, inside the slab: widened to 64 bits once, ahead of the loop, each
    // would occupy two registers for the whole kernel and every load would need a 64-bit vector add; seen next to the
    // load, base + offset is a scalar base register plus a 32-bit vector offset.
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) {
      asm volatile("" : "+v"(a_off[j]));
      QWIX_GLDS16(ga + a_off[j], ls + (j * NW + wave) * 1024);
    }
#pragma unroll
    for (int j = 0; j < B_LOADS; ++j) {
      asm volatile("" : "+v"(b_off[j]));
      QWIX_GLDS16(gb + b_off[j], ls + A_BYTES + (j * NW + wave) * 1024);
    }
  };

  // ---- fragments
  const int frow = lane & 31, hx = lane >> 5;
  const int a_row = (wr * WROWS + frow) * BK, a_sw = swz128(wr * WROWS + frow);
  const int b_row = (wc * 32 + frow) * B_ROWB, b_sw = W4 ? ((frow >> 2) & 3) : swz128(wc * 32 + frow);
  v4i fa[2][TM];
  v4i fbr[2];  // int4: one chunk = two k-steps; int8: one chunk = one k-step
  // e4m3: an operand of the 64-wide MFMA is two such 16-byte pieces (k-steps 2 kp and 2 kp + 1 of pair kp), read
  // straight into the halves of an 8-register operand; buffer kp holds pair kp
  v8i fa8[2][TM];
  v8i fb8[2];
  auto read_pair_a = [&](int s, int kp, int i) __attribute__((always_inline)) {
    const int c0 = 4 * kp + hx, c1 = c0 + 2;
    const uint8_t* ab = smem + s * STAGE + a_row + i * 32 * BK;
    const v4i lo = *reinterpret_cast<const v4i*>(ab + ((c0 ^ a_sw) << 4));
    const v4i hi = *reinterpret_cast<const v4i*>(ab + ((c1 ^ a_sw) << 4));
    fa8[kp][i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  auto read_pair_b = [&](int s, int kp) __attribute__((always_inline)) {
    const int c0 = 4 * kp + hx, c1 = c0 + 2;
    const uint8_t* bb = smem + s * STAGE + A_BYTES + b_row;
    const v4i lo = *reinterpret_cast<const v4i*>(bb + ((c0 ^ b_sw) << 4));
    const v4i hi = *reinterpret_cast<const v4i*>(bb + ((c1 ^ b_sw) << 4));
    fb8[kp] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  auto read_pair = [&](int s, int kp) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < TM; ++i) read_pair_a(s, kp, i);
    read_pair_b(s, kp);
  };
  auto read_a = [&](int s, int ks, int buf) __attribute__((always_inline)) {
    const int chunk = W4 ? (4 * (ks >> 1) + 2 * hx + (ks & 1)) : (2 * ks + hx);
    const uint8_t* base = smem + s * STAGE + a_row + ((chunk ^ a_sw) << 4);
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[buf][i] = *reinterpret_cast<const v4i*>(base + i * 32 * BK);
  };
  auto read_b = [&](int s, int idx, int buf) __attribute__((always_inline)) {  // idx: pair of k-steps (int4) or k-step (int8)
    const int chunk = 2 * idx + hx;
    fbr[buf] = *reinterpret_cast<const v4i*>(smem + s * STAGE + A_BYTES + b_row + ((chunk ^ b_sw) << 4));
  };
  auto b_frag = [&](int ks) __attribute__((always_inline)) -> v4i {
    if constexpr (W4) {
      const v4i raw = fbr[(ks >> 1) & 1];
      v4i f;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const unsigned w = static_cast<unsigned>(raw[2 * (ks & 1) + h]);
        const unsigned ev = (w << 4) & 0xF0F0F0F0u, od = w & 0xF0F0F0F0u;  // nibbles 0,2,4,6 and 1,3,5,7, x 16
        f[2 * h] = static_cast<int>(__builtin_amdgcn_perm(od, ev, 0x05010400));
        f[2 * h + 1] = static_cast<int>(__builtin_amdgcn_perm(od, ev, 0x07030602));
      }
      return f;
    } else {
      return fbr[ks & 1];
    }
  };

  AccV acc[TM];
  float accf[TM][16];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[i][r] = 0;
      accf[i][r] = 0.f;
    }
  constexpr int kMagicBits = 0x4B400000;           // 1.5 * 2^23 as a float
  constexpr float kMagic = 12582912.0f;
  v16i magic;
  if constexpr (MAGIC) {
#pragma unroll
    for (int r = 0; r < 16; ++r) magic[r] = kMagicBits;
    // keep the sixteen copies in registers of their own: the MFMA reads its addend from consecutive registers
    asm volatile("" : "+v"(magic));
  }
  float corr = 0.f;  // MAGIC: sum of C * sb over the groups folded in since the constants were last taken out

  // acc[i][r]: m = m0 + wr*WROWS + i*32 + 8*(r/4) + 4*hx + r%4,  n = n0 + wc*32 + frow: one weight scale per lane and group
  const int ncl = min(n0 + wc * 32 + frow, p.N - 1);
  constexpr float kUnscale = W4 ? 0.0625f : 1.0f;
  auto load_sb = [&](int g) __attribute__((always_inline)) -> unsigned {
    const int64_t i = static_cast<int64_t>(g) * p.N + ncl;
    if constexpr (SBF) return reinterpret_cast<const uint16_t*>(p.sb)[i];
    return reinterpret_cast<const unsigned*>(p.sb)[i];
  };

  const int KT = p.K / BK;
  const int tpg = p.group / BK;
  // The same load, hidden from the compiler's own wait-count bookkeeping: at the loop's back edge it would
  // otherwise wait for every outstanding load (vmcnt 0), the slab loads issued two slabs ahead included.  The
  // result is valid once the explicit wait at the end of the slab has passed (the load is older than the slab
  // loads of its iteration, and loads complete in order); until then nothing may read or copy `dst`.
  auto load_sb_async = [&](int g, unsigned& dst) __attribute__((always_inline)) {
    const int64_t i = static_cast<int64_t>(g) * p.N + ncl;
    if constexpr (SBF) {
      const uint16_t* ptr = reinterpret_cast<const uint16_t*>(p.sb) + i;
      asm volatile("global_load_ushort %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory");
    } else {
      const unsigned* ptr = reinterpret_cast<const unsigned*>(p.sb) + i;
      asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(ptr) : "memory");
    }
  };
  unsigned sb_raw = load_sb(0);
  issue_loads(0, 0);
  if (ST == 3 && KT > 1) issue_loads(1, 1);
  __syncthreads();
  if constexpr (F8) {
    read_pair(0, 0);
  } else {
    read_a(0, 0, 0);
    read_b(0, 0, 0);
  }

  int cs = 0;  // stage that holds the current slab
  auto next_stage = [&](int s, int by) __attribute__((always_inline)) { return s + by >= ST ? s + by - ST : s + by; };
  // End of slab kt: every wavefront's loads of slab kt+1 have landed (what was issued during this slab may stay
  // in flight when there are three stages), all wavefronts are done reading slab kt; then the first fragments
  // of slab kt+1.
  auto end_slab = [&](int kt) __attribute__((always_inline)) {
    if constexpr (ST == 3) {
      __builtin_amdgcn_sched_barrier(0);
      if (kt + 2 < KT) __builtin_amdgcn_s_waitcnt(0x0F70 | (A_LOADS + B_LOADS)); else __builtin_amdgcn_s_waitcnt(0x0F70);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    } else {
      __syncthreads();
    }
    cs = next_stage(cs, 1);
    if (kt + 1 < KT) {
      if constexpr (F8) {
        read_pair(cs, 0);
      } else {
        read_a(cs, 0, 0);
        read_b(cs, 0, 0);
      }
    }
  };

  // Folding a finished group into the f32 sums, one 32 x 32 tile at a time: acc[i] of group g, weight scale sbg
  // (with the 1/16 of the int4 widening folded in).
  auto fold_tile = [&](int i, int g, float sbg, bool recentre) __attribute__((always_inline)) {
    if constexpr (SAG) {
      // rows of acc[i][4*qd .. 4*qd+3]: i*32 + 8*qd + 4*hx + 0..3, one 16-byte LDS read (a broadcast per half)
      const float* sg = sa_lds + g * BM + wr * WROWS + 4 * hx;
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const v4f sa4 = *reinterpret_cast<const v4f*>(sg + i * 32 + 8 * qd);
        const float sv[4] = {sa4[0], sa4[1], sa4[2], sa4[3]};
#pragma unroll
        for (int j = 0; j < 4; ++j)
          accf[i][4 * qd + j] = __builtin_fmaf(static_cast<float>(acc[i][4 * qd + j]) * sv[j], sbg, accf[i][4 * qd + j]);
      }
    } else if constexpr (MAGIC) {
      if (i == 0) corr = __builtin_fmaf(kMagic, sbg, corr);
#pragma unroll
      for (int r = 0; r < 16; ++r) accf[i][r] = __builtin_fmaf(__int_as_float(acc[i][r]), sbg, accf[i][r]);
      if (recentre) {
#pragma unroll
        for (int r = 0; r < 16; ++r) accf[i][r] -= corr;
        if (i == TM - 1) corr = 0.f;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) accf[i][r] = __builtin_fmaf(static_cast<float>(acc[i][r]), sbg, accf[i][r]);
    }
  };

  // A use of a tile's sums right behind its fold: without one the compiler moves the whole fold into the block
  // where the sums are next read (behind the slab's barrier), all scale reads of the four tiles are then in flight at
  // once and their registers push loop invariants into scratch memory.
  auto pin_sums = [&](int i) __attribute__((always_inline)) {
    asm volatile("" : "+v"(accf[i][0]), "+v"(accf[i][1]), "+v"(accf[i][2]), "+v"(accf[i][3]), "+v"(accf[i][4]),
                 "+v"(accf[i][5]), "+v"(accf[i][6]), "+v"(accf[i][7]), "+v"(accf[i][8]), "+v"(accf[i][9]),
                 "+v"(accf[i][10]), "+v"(accf[i][11]), "+v"(accf[i][12]), "+v"(accf[i][13]), "+v"(accf[i][14]),
                 "+v"(accf[i][15]));
  };

  // One slab.  FIRST: it opens a group (the accumulators restart from zero, or from the magic constant).
  // LAST: it closes one.  Then the last two k-steps run tile by tile instead of k-step by k-step, and the fold of
  // tile i sits behind the MFMAs of tile i+1: its sixteen accumulators are complete by then, and the vector work
  // runs while the matrix core multiplies the next tile; only the last tile's fold has nothing to hide behind.
  // (A wavefront issues in order: vector work placed after all MFMAs of a group would run with the matrix
  // core idle, and the other wavefront of the SIMD is at the same point of its own program.)
  auto slab = [&](int kt, auto first_tag, auto last_tag, int g, float sbg, bool recentre) __attribute__((always_inline)) {
    constexpr bool FIRST = decltype(first_tag)::value;
    constexpr bool LAST = decltype(last_tag)::value && !AUX;
    const int cur = cs;
    if (kt + ST - 1 < KT) issue_loads(next_stage(cs, ST - 1), kt + ST - 1);
    if constexpr (F8) {
      // pair 0 was read at the end of the slab before; pair 1 is read under the MFMAs of pair 0; when the slab closes
      // a group, the fold of tile i - 1 sits behind the last MFMA of tile i, as in the integer kernel
      // (a tile's half of pair 1 is requested behind that tile's MFMA of pair 0: its registers can be the ones that MFMA
      // has just read, and three MFMAs run before it is needed)
      read_pair_b(cur, 1);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        if constexpr (FIRST) {
          const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa8[0][i], fb8[0], zero, 0, 0, 0, 0, 0, 0);
        } else {
          acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa8[0][i], fb8[0], acc[i], 0, 0, 0, 0, 0, 0);
        }
        read_pair_a(cur, 1, i);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa8[1][i], fb8[1], acc[i], 0, 0, 0, 0, 0, 0);
        if constexpr (LAST) {
          if (i > 0) {
            fold_tile(i - 1, g, sbg, recentre);
            if constexpr (SAG) pin_sums(i - 1);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if constexpr (LAST) {
        fold_tile(TM - 1, g, sbg, recentre);
        if constexpr (SAG) pin_sums(TM - 1);
      }
      return;
    } else {
    auto read_next = [&](int ks) __attribute__((always_inline)) {  // fragments of k-step ks + 1
      if (ks + 1 < NK) {
        read_a(cur, ks + 1, (ks + 1) & 1);
        if constexpr (W4) {
          if ((ks & 1) == 1) read_b(cur, (ks + 1) >> 1, ((ks + 1) >> 1) & 1);
        } else {
          read_b(cur, ks + 1, (ks + 1) & 1);
        }
      }
    };
    auto mfma = [&](int ks, int i, const v4i& fb) __attribute__((always_inline)) {
      if (FIRST && ks == 0) {
        if constexpr (MAGIC) {
          acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks & 1][i], fb, magic, 0, 0, 0);
        } else {
          const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks & 1][i], fb, zero, 0, 0, 0);
        }
      } else {
        acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks & 1][i], fb, acc[i], 0, 0, 0);
      }
    };
    constexpr int NKM = LAST ? NK - 2 : NK;  // k-steps that run k-step by k-step
#pragma unroll
    for (int ks = 0; ks < NKM; ++ks) {
      read_next(ks);
      const v4i fb = b_frag(ks);
#pragma unroll
      for (int i = 0; i < TM; ++i) mfma(ks, i, fb);
    }
    if constexpr (LAST) {
      read_next(NK - 2);
      const v4i fb2 = b_frag(NK - 2), fb3 = b_frag(NK - 1);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        mfma(NK - 2, i, fb2);
        mfma(NK - 1, i, fb3);
        if (i > 0) fold_tile(i - 1, g, sbg, recentre);
        __builtin_amdgcn_sched_barrier(0);
      }
      fold_tile(TM - 1, g, sbg, recentre);
    }
    }
  };

  // The scale of the next group is fetched at the start of a group, together with the slab loads:
  // a load issued just before the barrier would make the barrier's wait for the slab wait for it too.
  auto to_scale = [&](unsigned raw) __attribute__((always_inline)) {
    if (p.single) return AUX ? 1.0f : kUnscale;  // the sums hold the plain integer; the epilogue scales it
    return __uint_as_float(SBF ? raw << 16 : raw) * (AUX ? 1.0f : kUnscale);
  };
  unsigned sb_cur = sb_raw, sb_next = 0;
  using T = std::true_type;
  using F = std::false_type;
  if constexpr (ONE && !AUX) {
    // every slab is a group of its own (always so for the conversion-free fold): one loop body
    for (int kt = 0; kt < KT; ++kt) {
      if (kt + 1 < KT) load_sb_async(kt + 1, sb_next);
      slab(kt, T{}, T{}, kt, to_scale(sb_cur), (kt & 3) == 3 || kt == KT - 1);
      end_slab(kt);  // its wait covers the scale load above
      asm volatile("" : "+v"(sb_next));
      sb_cur = sb_next;
    }
  } else
  for (int kt = 0; kt < KT; ++kt) {
    const int in_group = kt % tpg;
    const int g = kt / tpg;
    const float sbg = to_scale(sb_cur);
    const bool recentre = false;
    const bool first = in_group == 0, last = in_group == tpg - 1;
    if (first && kt + tpg < KT) sb_next = load_sb(g + 1);
    // (groups of several slabs: two loop bodies, the fold after the group's last MFMA)
    if (first) slab(kt, T{}, F{}, g, sbg, recentre);
    else slab(kt, F{}, F{}, g, sbg, recentre);
    if (last) {
      if constexpr (!AUX) {
#pragma unroll
        for (int i = 0; i < TM; ++i) fold_tile(i, g, sbg, false);
      }
      if constexpr (AUX) {
        // Asymmetric operands and parity runs: the partials as plain integers, folded at the end of the group.
        // acc[i][4*qd + j]: row i*32 + 8*qd + 4*hx + j of the wavefront's rows, column ncol
        const int ncol = n0 + wc * 32 + frow;
        const bool zp = p.zu != nullptr;
        const int zvl = zp ? p.zv[ncl * p.zv_sn + g * p.zv_sg] : 0;
        const int* zrow = zu_lds + (p.zu_sg != 0 ? g * BM : 0) + wr * WROWS + 4 * hx;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int qd = 0; qd < 4; ++qd) {
            v4i z4 = {0, 0, 0, 0};
            if (zp) z4 = *reinterpret_cast<const v4i*>(zrow + i * 32 + 8 * qd);  // a broadcast per wavefront half
            const int zz[4] = {z4[0], z4[1], z4[2], z4[3]};
            float sv[4] = {1.f, 1.f, 1.f, 1.f};
            if constexpr (SAG) {
              const v4f s4 = *reinterpret_cast<const v4f*>(sa_lds + g * BM + wr * WROWS + 4 * hx + i * 32 + 8 * qd);
              sv[0] = s4[0]; sv[1] = s4[1]; sv[2] = s4[2]; sv[3] = s4[3];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int r = 4 * qd + j;
              // the widened weights carry a factor 16, exactly
              const int val = (W4 ? (acc[i][r] >> 4) : acc[i][r]) - zz[j] * zvl;
              if constexpr (DUMP) {
                const int m = m0 + wr * WROWS + i * 32 + 8 * qd + 4 * hx + j;
                if (m < p.M && ncol < p.N) p.acc_out[(static_cast<int64_t>(g) * p.M + m) * p.N + ncol] = val;
              }
              float f = static_cast<float>(val);
              if constexpr (SAG) f *= sv[j];
              accf[i][r] = __builtin_fmaf(f, sbg, accf[i][r]);
            }
          }
      }
      sb_cur = sb_next;
    }
    end_slab(kt);
  }
  if constexpr (ST == 3) __syncthreads();  // before LDS turns into staging space for the output

  // ---- epilogue: 32 rows x 32 columns of f32 per wavefront and pass through LDS
  constexpr int ROW_F = 36;  // floats per staged row (32 + padding)
  float* stg = reinterpret_cast<float*>(smem) + wave * (32 * ROW_F);
  const bool t_bf16 = (p.t_dtype == QWIX_BF16) && p.ksplit == 0;  // a range's sums stay f32: the reduction rounds
  const bool vec_ok = (p.ldo % 8 == 0) && (p.N % 4 == 0);
  // chunk c = lane + 64*q of the 32 x 8 grid of 16-byte pieces: row c/8, columns 4*(c%8) .. +3
  float sav[TM][4];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = m0 + wr * WROWS + i * 32 + (lane + 64 * q) / 8;
      sav[i][q] = (!SAG && p.sa != nullptr && m < p.M) ? ld_scale(p.sa, p.sa_dtype, m) : 1.f;
    }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int r = 0; r < 16; ++r) stg[(8 * (r >> 2) + 4 * hx + (r & 3)) * ROW_F + frow] = accf[i][r];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int c = lane + 64 * q, row = c >> 3, cc = c & 7;
      const float4 v4 = *reinterpret_cast<const float4*>(stg + row * ROW_F + cc * 4);
      float v[4] = {v4.x, v4.y, v4.z, v4.w};
      const int m = m0 + wr * WROWS + i * 32 + row, n = n0 + wc * 32 + cc * 4;
      if (p.single) {
        // the untiled chain: the integer takes the first scale's dtype, every product the promotion of its factors
        const bool a_bf = p.sa == nullptr || p.sa_dtype == QWIX_BF16;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float t = v[e];
          if (p.sa != nullptr) {
            if (a_bf) t = round_bf16(t);
            t *= sav[i][q];
            if (a_bf) t = round_bf16(t);
          } else if (t_bf16) {
            t = round_bf16(t);
          }
          t *= (n + e < p.N) ? ld_scale(p.sb, p.sb_dtype, n + e) : 0.f;
          if (t_bf16) t = round_bf16(t);
          v[e] = t;
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] *= sav[i][q];
          if (t_bf16) v[e] = round_bf16(v[e]);
        }
      }
      if (m >= p.M || n >= p.N) continue;
      if (p.out_dtype == QWIX_BF16) {
        uint16_t* o = reinterpret_cast<uint16_t*>(p.out) + static_cast<int64_t>(m) * p.ldo + n;
        if (vec_ok) {
          nt_store8(reinterpret_cast<uint2*>(o),
                    make_uint2(f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16),
                               f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16)));
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < p.N) o[e] = f32_to_bf16_bits(v[e]);
        }
      } else {
        float* o = reinterpret_cast<float*>(p.out) + static_cast<int64_t>(m) * p.ldo + n;
        if (vec_ok) {
          nt_store16(reinterpret_cast<uint4*>(o), make_uint4(__float_as_uint(v[0]), __float_as_uint(v[1]),
                                                             __float_as_uint(v[2]), __float_as_uint(v[3])));
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < p.N) o[e] = v[e];
        }
      }
    }
  }
}

// LDS of the fast kernel: `st` slab stages, plus the f32 activation scales of the tile when they are per group.
template <int BQT, typename G = Fast>
size_t grouped_dma_lds(bool sag, int64_t K, int64_t group, int st, int64_t zu_groups = 0) {
  const size_t stages = st * (G::kBM * G::kBK + G::kBN * (BQT == QWIX_INT4 ? 64 : 128));
  return stages + (sag ? static_cast<size_t>(K / group) * G::kBM * sizeof(float) : 0) +
         static_cast<size_t>(zu_groups) * G::kBM * sizeof(int);
}
// rows of zero-point side values that ride along in LDS: one per group, one in all, or none
inline int64_t zu_groups_of(const GroupedArgs& p) { return p.zu == nullptr ? 0 : (p.zu_sg != 0 ? p.K / p.group : 1); }
constexpr size_t kLdsMax = 160 * 1024;
// Up to this many 128 x 256 tiles the narrow geometries run instead (from about 128 tiles on the wide tile's reuse of
// a weight fragment over four MFMAs wins: 512 x 14336 over K 4096, 224 tiles, 42.6 against 71.5 us).
constexpr int64_t kNarrowTiles = 80;

template <int BQT, bool SBF, bool SAG, bool AUX, bool MAGIC, int ST, bool ONE, bool DUMP = false, typename G = Fast>
int launch_grouped_dma(const GroupedArgs& p, hipStream_t st) {
  constexpr int BM = G::kBM, BN = G::kBN, NW = G::kNW;
  const size_t smem = grouped_dma_lds<BQT, G>(SAG, p.K, p.group, ST, zu_groups_of(p));
  static_assert(ST * (G::kBM * G::kBK + BN * 64) >= NW * 32 * 36 * sizeof(float), "epilogue staging must fit");
  auto kern = qgemm_grouped_dma_kernel<BQT, SBF, SAG, AUX, MAGIC, ST, ONE, DUMP, G>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  const int64_t tiles = static_cast<int64_t>((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
  const unsigned ranges = p.ksplit > 0 ? static_cast<unsigned>(p.K / p.ksplit) : 1u;
  kern<<<dim3(static_cast<unsigned>(tiles), ranges), NW * 64, smem, st>>>(p);
  return check_launch("qgemm_grouped (dma)");
}

// Decode batches (at most 32 rows) of the sub-channel GEMM with groups of 128 and one scale per token: the four
// wavefronts of a workgroup share one 32 x 32 output tile and split K by groups (wavefront w takes groups w, w + 4,
// ...).  Each wavefront streams its own slabs through a private three-stage ring in LDS (direct-to-LDS loads, its own
// vmcnt waits, no barrier in the loop), multiplies a group with four MFMAs, folds it into f32 sums with the group's
// weight scale (parked in LDS at the start), and the four partial sums meet in LDS once, at the end.  Against the
// tile kernels that is four slabs in flight per workgroup and N / 32 workgroups of four independent wavefronts where
// a decode batch left the tile kernel one 16-MFMA chain per slab: the arithmetic per output element is the same
// (exact int32 partial per group, f32 fold, per-token scale and rounding at the end), the groups are added in another
// order.
template <int BQT, bool SBF>
__global__ void __launch_bounds__(256) qgemm_grouped_decode_kernel(GroupedArgs p) {
  constexpr bool W4 = (BQT == QWIX_INT4);
  constexpr int BK = 128, NWV = 4, ST = 3;
  constexpr int B_ROWB = W4 ? 64 : 128;
  constexpr int A_BYTES = 32 * BK, B_BYTES = 32 * B_ROWB, STAGE = A_BYTES + B_BYTES;
  constexpr int A_LOADS = A_BYTES / 1024, B_LOADS = B_BYTES / 1024, L = A_LOADS + B_LOADS;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int KT = p.K / BK;
  const int nw_max = (KT + NWV - 1) / NWV;              // groups of wavefront 0 (the most any wavefront has)
  const int nw = (KT - wave + NWV - 1) / NWV;           // groups of this wavefront: wave, wave + 4, ...
  const int tiles_n = (p.N + 31) / 32;
  const int m0 = (static_cast<int>(blockIdx.x) / tiles_n) * 32, n0 = (static_cast<int>(blockIdx.x) % tiles_n) * 32;
  uint8_t* wsm = smem + wave * (ST * STAGE + nw_max * 32 * static_cast<int>(sizeof(float)));
  float* scl = reinterpret_cast<float*>(wsm + ST * STAGE);  // [group of this wavefront][column of the tile]

  const uint8_t* a_base = p.A + static_cast<int64_t>(m0) * p.lda;
  const uint8_t* b_base = p.B + static_cast<int64_t>(n0) * p.ldb;
  uint32_t a_off[A_LOADS], b_off[B_LOADS];
#pragma unroll
  for (int j = 0; j < A_LOADS; ++j) {
    const int row = j * 8 + (lane >> 3);
    a_off[j] = static_cast<uint32_t>(min(row, p.M - 1 - m0)) * static_cast<uint32_t>(p.lda) + (((lane & 7) ^ swz128(row)) << 4);
  }
#pragma unroll
  for (int j = 0; j < B_LOADS; ++j) {
    int row, chunk;
    if constexpr (W4) {
      row = j * 16 + (lane >> 2);
      chunk = (lane & 3) ^ ((lane >> 4) & 3);
    } else {
      row = j * 8 + (lane >> 3);
      chunk = (lane & 7) ^ swz128(row);
    }
    b_off[j] = static_cast<uint32_t>(min(row, p.N - 1 - n0)) * static_cast<uint32_t>(p.ldb) + (chunk << 4);
  }
  auto issue_loads = [&](int s, int kt) __attribute__((always_inline)) {
    const uint8_t* ga = a_base + static_cast<int64_t>(kt) * BK;
    const uint8_t* gb = b_base + static_cast<int64_t>(kt) * B_ROWB;
    uint8_t* ls = wsm + s * STAGE;
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) QWIX_GLDS16(ga + a_off[j], ls + j * 1024);
#pragma unroll
    for (int j = 0; j < B_LOADS; ++j) QWIX_GLDS16(gb + b_off[j], ls + A_BYTES + j * 1024);
  };
  if (nw > 0) issue_loads(0, wave);
  if (nw > 1) issue_loads(1, wave + NWV);

  // the weight scales of this wavefront's groups, one column per lane: lanes 0-31 take the even, lanes 32-63 the odd ones
  const int frow = lane & 31, hx = lane >> 5;
  const int ncl = min(n0 + frow, p.N - 1);
  for (int i = hx; i < nw; i += 2) {
    const int64_t at = static_cast<int64_t>(wave + i * NWV) * p.N + ncl;
    float s;
    if constexpr (SBF) s = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.sb)[at]);
    else s = reinterpret_cast<const float*>(p.sb)[at];
    scl[i * 32 + frow] = s * (W4 ? 0.0625f : 1.0f);  // the widened int4 weights carry a factor 16, exactly
  }
  // (the compiler's wait for these loads covers the two slabs requested above as well: they are needed next anyway)

  const int a_row = frow * BK, a_sw = swz128(frow);
  const int b_row = frow * B_ROWB, b_sw = W4 ? ((frow >> 2) & 3) : swz128(frow);
  float accf[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) accf[r] = 0.f;
  constexpr int W2 = 0x0F70 | ((2 * L) & 0xF) | (((2 * L) >> 4) << 14), W1 = 0x0F70 | (L & 0xF) | ((L >> 4) << 14);

  int cur = 0;
  for (int i = 0; i < nw; ++i) {
    if (i + 2 < nw) issue_loads(cur == 0 ? 2 : cur - 1, wave + (i + 2) * NWV);  // the stage of slab i - 1
    // this wavefront's slab i has landed once at most the slabs requested after it are outstanding
    const int newer = min(nw - 1, i + 2) - i;
    if (newer >= 2) __builtin_amdgcn_s_waitcnt(W2);
    else if (newer == 1) __builtin_amdgcn_s_waitcnt(W1);
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    __builtin_amdgcn_sched_barrier(0);
    const uint8_t* sa_ = wsm + cur * STAGE + a_row;
    const uint8_t* sb_ = wsm + cur * STAGE + A_BYTES + b_row;
    v16i acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (W4) {
      v4i raw[2];
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) raw[pr] = *reinterpret_cast<const v4i*>(sb_ + (((2 * pr + hx) ^ b_sw) << 4));
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const int chunk = 4 * (ks >> 1) + 2 * hx + (ks & 1);
        const v4i fa = *reinterpret_cast<const v4i*>(sa_ + ((chunk ^ a_sw) << 4));
        v4i fb;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const unsigned w = static_cast<unsigned>(raw[ks >> 1][2 * (ks & 1) + h]);
          const unsigned ev = (w << 4) & 0xF0F0F0F0u, od = w & 0xF0F0F0F0u;  // nibbles 0,2,4,6 and 1,3,5,7, x 16
          fb[2 * h] = static_cast<int>(__builtin_amdgcn_perm(od, ev, 0x05010400));
          fb[2 * h + 1] = static_cast<int>(__builtin_amdgcn_perm(od, ev, 0x07030602));
        }
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, acc, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const int chunk = 2 * ks + hx;
        const v4i fa = *reinterpret_cast<const v4i*>(sa_ + ((chunk ^ a_sw) << 4));
        const v4i fb = *reinterpret_cast<const v4i*>(sb_ + ((chunk ^ b_sw) << 4));
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, acc, 0, 0, 0);
      }
    }
    const float sbg = scl[i * 32 + frow];
#pragma unroll
    for (int r = 0; r < 16; ++r) accf[r] = __builtin_fmaf(static_cast<float>(acc[r]), sbg, accf[r]);
    cur = cur == 2 ? 0 : cur + 1;
  }

  // the four partial sums meet in LDS (each wavefront writes into its own ring, then wavefront 0 adds them up)
  float* red = reinterpret_cast<float*>(wsm);
#pragma unroll
  for (int r = 0; r < 16; ++r) red[r * 64 + lane] = accf[r];
  __syncthreads();
  if (wave != 0) return;
  const int wstride = (ST * STAGE + nw_max * 32 * static_cast<int>(sizeof(float))) / static_cast<int>(sizeof(float));
#pragma unroll
  for (int w = 1; w < NWV; ++w)
#pragma unroll
    for (int r = 0; r < 16; ++r) accf[r] += red[w * wstride + r * 64 + lane];
  const bool t_bf16 = (p.t_dtype == QWIX_BF16);
  const int n = n0 + frow;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = m0 + 8 * (r >> 2) + 4 * hx + (r & 3);
    if (m >= p.M || n >= p.N) continue;
    float v = accf[r];
    if (p.sa != nullptr) v *= ld_scale(p.sa, p.sa_dtype, m);
    if (t_bf16) v = round_bf16(v);
    if (p.out_dtype == QWIX_BF16)
      reinterpret_cast<uint16_t*>(p.out)[static_cast<int64_t>(m) * p.ldo + n] = f32_to_bf16_bits(v);
    else
      reinterpret_cast<float*>(p.out)[static_cast<int64_t>(m) * p.ldo + n] = v;
  }
}

template <int BQT, bool SBF>
int launch_grouped_decode(const GroupedArgs& p, hipStream_t st) {
  constexpr int STAGE = 32 * 128 + 32 * (BQT == QWIX_INT4 ? 64 : 128);
  const int KT = p.K / 128, nw_max = (KT + 3) / 4;
  const size_t smem = 4 * (3 * static_cast<size_t>(STAGE) + static_cast<size_t>(nw_max) * 32 * sizeof(float));
  if (smem > kLdsMax) return -1;
  auto kern = qgemm_grouped_decode_kernel<BQT, SBF>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  const int64_t tiles = static_cast<int64_t>((p.M + 31) / 32) * ((p.N + 31) / 32);
  kern<<<dim3(static_cast<unsigned>(tiles)), 256, smem, st>>>(p);
  return check_launch("qgemm_grouped (decode)");
}

// Picks the instantiation.  Returns -1 when the tile's per-group activation scales do not fit in LDS (the caller
// then takes the register-staged kernel).
template <int BQT, bool SAG>
int dispatch_grouped_dma(const GroupedArgs& p, hipStream_t st) {
  const bool sbf = p.sb_dtype == QWIX_BF16;
  const bool three = grouped_dma_lds<BQT>(SAG, p.K, p.group, 3) <= kLdsMax;  // room for a third slab stage
  if (grouped_dma_lds<BQT>(SAG, p.K, p.group, 2, zu_groups_of(p)) > kLdsMax) return -1;
  if (p.acc_out != nullptr)  // parity runs
    return sbf ? launch_grouped_dma<BQT, true, SAG, true, false, 2, false, true>(p, st)
               : launch_grouped_dma<BQT, false, SAG, true, false, 2, false, true>(p, st);
  if (p.zu != nullptr)  // an asymmetric operand
    return sbf ? launch_grouped_dma<BQT, true, SAG, true, false, 2, false>(p, st)
               : launch_grouped_dma<BQT, false, SAG, true, false, 2, false>(p, st);
  if constexpr (!SAG) {
    // A decode batch against groups of 128 with one scale per token: the kernel that splits K over wavefronts, while
    // its N / 32 workgroups (each reads all the activation rows) are a few hundred.  int8 x int4, weights from HBM,
    // 16 rows: K 4096, N 4096 15.5 -> 8.6 us, N 14336 16.0 -> 12.3, K 14336, N 4096 76.6 -> 19.9, K 8192, N 8192
    // 27.2 -> 13.8; at N 28672 the narrow tiles are ahead (19.9 against 23.6 us), with int8 weights from N 14336 on.
    if (p.M <= 32 && p.group == Fast::kBK && !p.single && p.ga == 1 && (p.K / Fast::kBK) >= 4 &&
        p.N * (BQT == QWIX_INT4 ? 1 : 2) <= 16384 && 32 * p.lda < (int64_t{1} << 31) && 32 * p.ldb < (int64_t{1} << 31)) {
      const int rc = sbf ? launch_grouped_decode<BQT, true>(p, st) : launch_grouped_decode<BQT, false>(p, st);
      if (rc >= 0) return rc;
    }
    // Few 128 x 256 tiles (under a third of the CUs), or a decode batch: 128 x 64 tiles of two wavefronts, four times
    // the workgroups; 32 or 64 rows per tile up to 64 rows.  int8 x int4 in groups of 128, weights from HBM, K 4096,
    // N 4096, 16 / 64 / 128 / 512 rows: 35.7 / 36.5 / 38.4 / 39.0 us with the wide tile, 15.5 / 19.6 / 28.3 / 29.5 us now
    // (K 8192, N 8192: 64.1 / 65.0 / 67.7 / 69.9 -> 27.2 / 34.7 / 49.1 / 70.0 us).
    const int64_t wide = static_cast<int64_t>((p.M + Fast::kBM - 1) / Fast::kBM) * ((p.N + Fast::kBN - 1) / Fast::kBN);
    if (wide <= kNarrowTiles || p.M <= 64) {
      if (p.group == Fast::kBK && p.M <= 64) {  // decode batches: tiles of 32 or 64 rows
        if (sbf && p.t_dtype == QWIX_BF16)
          return p.M <= 32 ? launch_grouped_dma<BQT, true, false, false, true, 3, true, false, Narrow32>(p, st)
                           : launch_grouped_dma<BQT, true, false, false, true, 3, true, false, Narrow64>(p, st);
        if (!sbf)
          return p.M <= 32 ? launch_grouped_dma<BQT, false, false, false, false, 3, true, false, Narrow32>(p, st)
                           : launch_grouped_dma<BQT, false, false, false, false, 3, true, false, Narrow64>(p, st);
      }
      if (p.group == Fast::kBK) {
        if (sbf && p.t_dtype == QWIX_BF16) return launch_grouped_dma<BQT, true, false, false, true, 3, true, false, Narrow>(p, st);
        return sbf ? launch_grouped_dma<BQT, true, false, false, false, 3, true, false, Narrow>(p, st)
                   : launch_grouped_dma<BQT, false, false, false, false, 3, true, false, Narrow>(p, st);
      }
      return sbf ? launch_grouped_dma<BQT, true, false, false, false, 2, false, false, Narrow>(p, st)
                 : launch_grouped_dma<BQT, false, false, false, false, 2, false, false, Narrow>(p, st);
    }
  }
  if (p.group == Fast::kBK) {  // one slab per group
    if constexpr (!SAG) {
      // scaled partials that the reference keeps in bf16: the conversion-free fold
      if (sbf && p.t_dtype == QWIX_BF16) return launch_grouped_dma<BQT, true, false, false, true, 3, true>(p, st);
    }
    if (three)
      return sbf ? launch_grouped_dma<BQT, true, SAG, false, false, 3, true>(p, st)
                 : launch_grouped_dma<BQT, false, SAG, false, false, 3, true>(p, st);
    return sbf ? launch_grouped_dma<BQT, true, SAG, false, false, 2, true>(p, st)
               : launch_grouped_dma<BQT, false, SAG, false, false, 2, true>(p, st);
  }
  return sbf ? launch_grouped_dma<BQT, true, SAG, false, false, 2, false>(p, st)
             : launch_grouped_dma<BQT, false, SAG, false, false, 2, false>(p, st);
}

// The instantiations for e4m3 x e4m3 (no zero points, no int32 partials).
template <bool SAG>
int dispatch_grouped_f8(const GroupedArgs& p, hipStream_t st) {
  constexpr int Q = QWIX_E4M3;
  const bool sbf = p.sb_dtype == QWIX_BF16;
  if (grouped_dma_lds<Q>(SAG, p.K, p.group, 2) > kLdsMax) return -1;
  if (p.group == Fast::kBK) {
    if (grouped_dma_lds<Q>(SAG, p.K, p.group, 3) <= kLdsMax)
      return sbf ? launch_grouped_dma<Q, true, SAG, false, false, 3, true>(p, st)
                 : launch_grouped_dma<Q, false, SAG, false, false, 3, true>(p, st);
    return sbf ? launch_grouped_dma<Q, true, SAG, false, false, 2, true>(p, st)
               : launch_grouped_dma<Q, false, SAG, false, false, 2, true>(p, st);
  }
  return sbf ? launch_grouped_dma<Q, true, SAG, false, false, 2, false>(p, st)
             : launch_grouped_dma<Q, false, SAG, false, false, 2, false>(p, st);
}

// out[m, n] = cast(T(sa[m] * sum over ranges of ws[r][m][n])): what the tile kernel's epilogue does with its f32 sums,
// after the K ranges' partial sums are added in range order.  Four consecutive elements of (m, n) per thread.
__global__ void __launch_bounds__(256)
    grouped_reduce_kernel(const float* __restrict__ ws, int ranges, int M, int N, const void* __restrict__ sa,
                          int sa_dtype, int t_bf16, uint8_t* __restrict__ out, int out_dtype, int64_t ldo) {
  const int64_t total = static_cast<int64_t>(M) * N;
  const int64_t i0 = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i0 >= total) return;
  const bool vec = (N & 3) == 0;  // then the four share a row and the loads are 16-byte aligned
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (vec) {
    float4 w[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      w[j] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (j < ranges) w[j] = *reinterpret_cast<const float4*>(ws + j * total + i0);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < ranges) { v[0] += w[j].x; v[1] += w[j].y; v[2] += w[j].z; v[3] += w[j].w; }
  } else {
    for (int r = 0; r < ranges; ++r)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (i0 + e < total) v[e] += ws[r * total + i0 + e];
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int64_t i = i0 + e;
    if (i >= total) break;
    const int m = static_cast<int>(i / N), n = static_cast<int>(i % N);
    float t = v[e];
    if (sa != nullptr) t *= ld_scale(sa, sa_dtype, m);
    if (t_bf16) t = round_bf16(t);
    if (out_dtype == QWIX_BF16)
      reinterpret_cast<uint16_t*>(out)[static_cast<int64_t>(m) * ldo + n] = f32_to_bf16_bits(t);
    else
      reinterpret_cast<float*>(out)[static_cast<int64_t>(m) * ldo + n] = t;
  }
}
constexpr int kMaxRanges = 8;  // what grouped_reduce_kernel reads in one batch

// The K ranges of qwix_hip_qgemm_grouped_ws (0: none): for the narrow tiles (128 x 64, two workgroups per CU) of the
// fast kernel with one activation scale per row and symmetric operands, above the decode kernel's 32 rows.  A tile
// walks its slabs at about 0.78 us each (0.51 us up to 64 rows) after 3 us, however few tiles there are (weights from
// HBM); the ranges cost a second launch and their partial arrays written and read.
static int grouped_ranges(int64_t M, int64_t N, int64_t K, int64_t group, int b_qtype) {
  if (b_qtype == QWIX_E4M3 || M <= 32 || group <= 0 || group % 128 || K % group || group == K) return 0;
  const int64_t wide = ((M + Fast::kBM - 1) / Fast::kBM) * ((N + Fast::kBN - 1) / Fast::kBN);
  if (!(wide <= kNarrowTiles || M <= 64)) return 0;
  const int64_t tiles = ((M + 127) / 128) * ((N + 63) / 64);
  auto model = [&](int64_t sp) {
    const double rounds = static_cast<double>((sp * tiles + 511) / 512);
    const double walk = 3.0 + static_cast<double>(K / 128 / sp) * (M <= 64 ? 0.51 : 0.78) * rounds;
    return sp == 1 ? walk : walk + 3.5 + static_cast<double>(sp * M * N) * 8.0 / 4.0e6;
  };
  int best = 1;
  double best_us = model(1);
  for (int64_t sp = 2; sp <= kMaxRanges && sp * 1024 <= K; ++sp) {
    if (K % (sp * group)) continue;
    const double us = model(sp);
    if (us < 0.85 * best_us) { best = static_cast<int>(sp); best_us = us; }
  }
  return best > 1 ? best : 0;
}

// Per-group K-sums of quantized rows: out[row, g] = sum over the g-th group of `group` values of row `row`
// (int8, or packed int4).  One 16-byte chunk per thread; the chunks of a group that sit in `seg` adjacent
// lanes (a power of two that divides the chunks per group) are added by shuffles, the rest by integer
// atomics into the zero-filled output -- integer addition, so the order does not matter.
__global__ void __launch_bounds__(256) fill_i32_kernel(int32_t* p, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n) p[i] = 0;
}

template <bool W4>
__global__ void __launch_bounds__(256)
    ksum_groups_kernel(const uint8_t* __restrict__ q, int64_t ld, int64_t rows, int chunks_per_row, int cpg, int seg,
                       int G, int32_t* __restrict__ out) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t row = idx / chunks_per_row;
  const int c = static_cast<int>(idx % chunks_per_row);
  const bool valid = row < rows;
  int s = 0;
  if (valid) {
    const uint4 w = *reinterpret_cast<const uint4*>(q + row * ld + static_cast<int64_t>(c) * 16);
    const unsigned u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if constexpr (W4) {  // signed nibble = (nibble ^ 8) - 8
        const unsigned x = u[e] ^ 0x88888888u;
        const unsigned t = (x & 0x0F0F0F0Fu) + ((x >> 4) & 0x0F0F0F0Fu);
        s += static_cast<int>((t * 0x01010101u) >> 24) - 64;
      } else {             // signed byte = (byte ^ 0x80) - 128
        const unsigned x = u[e] ^ 0x80808080u;
        const unsigned t = (x & 0x00FF00FFu) + ((x >> 8) & 0x00FF00FFu);
        s += static_cast<int>((t & 0xFFFFu) + (t >> 16)) - 512;
      }
    }
  }
  for (int m = seg >> 1; m >= 1; m >>= 1) s += __shfl_xor(s, m, 64);
  if (valid && (c & (seg - 1)) == 0) atomicAdd(out + row * G + c / cpg, s);
}

}  // namespace
}  // namespace qwix

using namespace qwix;

extern "C" int qwix_hip_ksum_groups(const void* q, int qtype, int64_t ld_bytes, int64_t rows, int64_t K, int64_t group,
                                    int32_t* out, void* stream) {
  if (!q || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null argument");
  if (qtype != QWIX_INT8 && qtype != QWIX_INT4)
    return fail(QWIX_ERR_UNSUPPORTED, "K-sums are taken of int8 or int4 values (got qtype %d)", qtype);
  if (rows <= 0 || K <= 0 || group <= 0 || group % 128 || K % group)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "group %lld must be a multiple of 128 that divides K=%lld (rows=%lld)",
                (long long)group, (long long)K, (long long)rows);
  const int64_t row_bytes = qtype == QWIX_INT4 ? K / 2 : K, group_bytes = qtype == QWIX_INT4 ? group / 2 : group;
  if (ld_bytes % 16 || ld_bytes < row_bytes || !aligned16(q))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "rows must be 16-byte aligned and at least K values long");
  const int64_t chunks_per_row = row_bytes / 16, cpg = group_bytes / 16, G = K / group;
  if (chunks_per_row > INT32_MAX || rows * G > (int64_t{1} << 40))
    return fail(QWIX_ERR_UNSUPPORTED, "shape too large for the K-sum kernel");
  int seg = 1;
  while (seg < 64 && cpg % (2 * seg) == 0) seg *= 2;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t n_out = rows * G, n_chunks = rows * chunks_per_row;
  fill_i32_kernel<<<dim3(static_cast<unsigned>((n_out + 255) / 256)), 256, 0, st>>>(out, n_out);
  const dim3 grid(static_cast<unsigned>((n_chunks + 255) / 256));
  if (qtype == QWIX_INT4)
    ksum_groups_kernel<true><<<grid, 256, 0, st>>>(static_cast<const uint8_t*>(q), ld_bytes, rows,
                                                   static_cast<int>(chunks_per_row), static_cast<int>(cpg), seg,
                                                   static_cast<int>(G), out);
  else
    ksum_groups_kernel<false><<<grid, 256, 0, st>>>(static_cast<const uint8_t*>(q), ld_bytes, rows,
                                                    static_cast<int>(chunks_per_row), static_cast<int>(cpg), seg,
                                                    static_cast<int>(G), out);
  return check_launch("ksum_groups");
}

static int grouped_impl(const void* a, int64_t lda, const void* b, int64_t ldb_bytes, int b_qtype, int64_t M, int64_t N,
                        int64_t K, int64_t group, const void* sa, int sa_dtype, int64_t ga, const void* sb, int sb_dtype,
                        const int32_t* zu, int64_t zu_row_stride, int64_t zu_group_stride, const int32_t* zv,
                        int64_t zv_col_stride, int64_t zv_group_stride, void* out, int out_dtype, int64_t ldo,
                        int exact, int32_t* acc_out, void* stream, void* workspace = nullptr,
                        size_t workspace_bytes = 0) {
  if (!a || !b || !out || !sb) return fail(QWIX_ERR_INVALID_ARGUMENT, "null a/b/out/sb");
  if (M <= 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad GEMM shape M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                (long long)K);
  if (b_qtype != QWIX_INT8 && b_qtype != QWIX_INT4 && b_qtype != QWIX_E4M3)
    return fail(QWIX_ERR_UNSUPPORTED, "grouped GEMM takes int8, int4 or e4m3 weights (got qtype %d)", b_qtype);
  if (b_qtype == QWIX_E4M3 && (zu || acc_out))
    return fail(QWIX_ERR_UNSUPPORTED, "e4m3 operands have neither zero points nor int32 partials");
  if (group <= 0 || group % 128 || K % group)
    return fail(QWIX_ERR_UNSUPPORTED, "group %lld must be a multiple of 128 that divides K=%lld", (long long)group,
                (long long)K);
  const int64_t brow = b_qtype == QWIX_INT4 ? K / 2 : K;
  if (lda % 16 || ldb_bytes % 16 || lda < K || ldb_bytes < brow || !aligned16(a) || !aligned16(b))
    return fail(QWIX_ERR_UNSUPPORTED, "lda/ldb must be multiples of 16 bytes and a/b 16-byte aligned");
  if (ga != 1 && ga != K / group) return fail(QWIX_ERR_INVALID_ARGUMENT, "ga must be 1 or K/group, got %lld", (long long)ga);
  auto ok_s = [](int d) { return d == QWIX_F32 || d == QWIX_BF16; };
  if ((sa && !ok_s(sa_dtype)) || !ok_s(sb_dtype) || !ok_s(out_dtype))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "scale and output dtypes must be f32 or bf16");
  if (ldo < N || !aligned16(out)) return fail(QWIX_ERR_INVALID_ARGUMENT, "bad output leading dimension");
  if ((zu == nullptr) != (zv == nullptr))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "zu and zv come together (zero points and the other operand's K-sums)");
  if (zu && (zu_row_stride < 0 || zu_group_stride < 0 || zv_col_stride < 0 || zv_group_stride < 0))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "negative zero-point stride");
  GroupedArgs p{};
  p.A = static_cast<const uint8_t*>(a); p.lda = lda;
  p.B = static_cast<const uint8_t*>(b); p.ldb = ldb_bytes;
  p.M = static_cast<int>(M); p.N = static_cast<int>(N); p.K = static_cast<int>(K); p.group = static_cast<int>(group);
  p.sa = sa; p.sa_dtype = sa_dtype; p.ga = static_cast<int>(ga);
  p.sb = sb; p.sb_dtype = sb_dtype;
  p.t_dtype = (sb_dtype == QWIX_F32 || (sa && sa_dtype == QWIX_F32)) ? QWIX_F32 : QWIX_BF16;
  p.acc_dtype = QWIX_F32;
  if (b_qtype == QWIX_E4M3) {
    // float operands accumulate in the result type (qarray.py:781-821): the caller's out dtype
    p.acc_dtype = out_dtype;
    if (out_dtype == QWIX_F32) p.t_dtype = QWIX_F32;
  }
  p.out = static_cast<uint8_t*>(out); p.out_dtype = out_dtype; p.ldo = ldo;
  p.acc_out = acc_out;
  p.zu = zu; p.zu_sm = zu_row_stride; p.zu_sg = zu_group_stride;
  p.zv = zv; p.zv_sn = zv_col_stride; p.zv_sg = zv_group_stride;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool row_strides_fit = 128 * lda < (int64_t{1} << 31) && 256 * ldb_bytes < (int64_t{1} << 31);
  // One group: there is no sum of partials to keep in f32, so both modes give the reference's roundings.
  p.single = (b_qtype != QWIX_E4M3 && group == K) ? 1 : 0;
  if (p.single) exact = 1;
  if (b_qtype == QWIX_E4M3) {
    if (!exact && row_strides_fit) {
      const int rc = (sa != nullptr && ga > 1) ? dispatch_grouped_f8<true>(p, st) : dispatch_grouped_f8<false>(p, st);
      if (rc >= 0) return rc;
    }
    return launch_grouped<QWIX_E4M3, true>(p, st);
  }
  if ((!exact || p.single) && row_strides_fit) {
    // per-group activation scales ride along in LDS: the tile's scales must fit behind the slab stages
    const bool sag = sa != nullptr && ga > 1;
    // K in ranges with f32 partial sums in the caller's workspace, where the narrow tiles are few
    const int ranges = (workspace && !exact && !sag && !zu && !acc_out && aligned16(workspace))
                           ? grouped_ranges(M, N, K, group, b_qtype) : 0;
    if (ranges > 0 && workspace_bytes >= static_cast<size_t>(ranges) * M * N * 4) {
      GroupedArgs q = p;
      q.ksplit = static_cast<int>(K / ranges);
      q.sa = nullptr;
      q.out = static_cast<uint8_t*>(workspace); q.out_dtype = QWIX_F32; q.ldo = N;
      const int rc = b_qtype == QWIX_INT4 ? dispatch_grouped_dma<QWIX_INT4, false>(q, st)
                                          : dispatch_grouped_dma<QWIX_INT8, false>(q, st);
      if (rc > 0) return rc;
      if (rc == 0) {
        const int64_t threads = (M * N + 3) / 4;
        grouped_reduce_kernel<<<dim3(static_cast<unsigned>((threads + 255) / 256)), 256, 0, st>>>(
            static_cast<const float*>(workspace), ranges, p.M, p.N, sa, sa_dtype, p.t_dtype == QWIX_BF16 ? 1 : 0,
            static_cast<uint8_t*>(out), out_dtype, ldo);
        return check_launch("qgemm_grouped (K ranges)");
      }
    }
    int rc;
    if (b_qtype == QWIX_INT4)
      rc = sag ? dispatch_grouped_dma<QWIX_INT4, true>(p, st) : dispatch_grouped_dma<QWIX_INT4, false>(p, st);
    else
      rc = sag ? dispatch_grouped_dma<QWIX_INT8, true>(p, st) : dispatch_grouped_dma<QWIX_INT8, false>(p, st);
    if (rc >= 0) return rc;
  }
  if (b_qtype == QWIX_INT4)
    return exact ? launch_grouped<QWIX_INT4, true>(p, st) : launch_grouped<QWIX_INT4, false>(p, st);
  return exact ? launch_grouped<QWIX_INT8, true>(p, st) : launch_grouped<QWIX_INT8, false>(p, st);
}

extern "C" int qwix_hip_qgemm_grouped(const void* a, int64_t lda, const void* b, int64_t ldb_bytes, int b_qtype,
                                      int64_t M, int64_t N, int64_t K, int64_t group, const void* sa, int sa_dtype,
                                      int64_t ga, const void* sb, int sb_dtype, void* out, int out_dtype, int64_t ldo,
                                      int exact, int32_t* acc_out, void* stream) {
  return grouped_impl(a, lda, b, ldb_bytes, b_qtype, M, N, K, group, sa, sa_dtype, ga, sb, sb_dtype, nullptr, 0, 0,
                      nullptr, 0, 0, out, out_dtype, ldo, exact, acc_out, stream);
}

extern "C" size_t qwix_hip_qgemm_grouped_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t group, int b_qtype) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  return static_cast<size_t>(grouped_ranges(M, N, K, group, b_qtype)) * M * N * 4;
}

extern "C" int qwix_hip_qgemm_grouped_ws(const void* a, int64_t lda, const void* b, int64_t ldb_bytes, int b_qtype,
                                         int64_t M, int64_t N, int64_t K, int64_t group, const void* sa, int sa_dtype,
                                         int64_t ga, const void* sb, int sb_dtype, void* out, int out_dtype, int64_t ldo,
                                         int exact, int32_t* acc_out, void* workspace, size_t workspace_bytes,
                                         void* stream) {
  return grouped_impl(a, lda, b, ldb_bytes, b_qtype, M, N, K, group, sa, sa_dtype, ga, sb, sb_dtype, nullptr, 0, 0,
                      nullptr, 0, 0, out, out_dtype, ldo, exact, acc_out, stream, workspace, workspace_bytes);
}

extern "C" int qwix_hip_qgemm_grouped_zp(const void* a, int64_t lda, const void* b, int64_t ldb_bytes, int b_qtype,
                                         int64_t M, int64_t N, int64_t K, int64_t group, const void* sa, int sa_dtype,
                                         int64_t ga, const void* sb, int sb_dtype, const int32_t* zu,
                                         int64_t zu_row_stride, int64_t zu_group_stride, const int32_t* zv,
                                         int64_t zv_col_stride, int64_t zv_group_stride, void* out, int out_dtype,
                                         int64_t ldo, int exact, int32_t* acc_out, void* stream) {
  if (!zu || !zv) return fail(QWIX_ERR_INVALID_ARGUMENT, "null zu/zv");
  return grouped_impl(a, lda, b, ldb_bytes, b_qtype, M, N, K, group, sa, sa_dtype, ga, sb, sb_dtype, zu, zu_row_stride,
                      zu_group_stride, zv, zv_col_stride, zv_group_stride, out, out_dtype, ldo, exact, acc_out, stream);
}

// Rotate, quantize, multiply in one call (the functional content of the reference's fused Hadamard kernel,
// qwix/contrib/kernels/fused_hadamard_quantized_matmul.py:349-414, with the numerics of the unfused path:
// hadamard_rot.py:133-190, then quantize, then _fast_dot_general): the rotation + per-token or per-group quantize kernel
// writes int8 rows and their scales into the caller's workspace, the sub-channel GEMM reads them.  Bit-identical to
// qwix_hip_fwht_quantize followed by qwix_hip_qgemm_grouped -- or, when the workspace is larger than required by at
// least qwix_hip_qgemm_grouped_workspace_bytes, by qwix_hip_qgemm_grouped_ws on that surplus (K in ranges).
static size_t had_align(size_t v) { return (v + 255) & ~size_t{255}; }

extern "C" size_t qwix_hip_qgemm_hadamard_act_workspace_bytes(int64_t M, int64_t K, int64_t act_tile, int x_dtype) {
  if (M <= 0 || K <= 0 || act_tile <= 0 || K % act_tile) return 0;
  const size_t es = x_dtype == QWIX_BF16 ? 2 : 4;
  return had_align(static_cast<size_t>(M) * K) + had_align(static_cast<size_t>(M) * (K / act_tile) * es);
}

extern "C" int qwix_hip_qgemm_hadamard_act(const void* x, int x_dtype, int64_t M, int64_t N, int64_t K, const void* pre_sign,
                                           const void* post_sign, float out_scale, int64_t act_tile, const void* b,
                                           int64_t ldb_bytes, int b_qtype, int64_t group, const void* sb, int sb_dtype,
                                           void* out, int out_dtype, int64_t ldo, void* workspace, size_t workspace_bytes,
                                           void* stream) {
  if (!x || !b || !sb || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null x/b/sb/out");
  if (M <= 0 || N <= 0 || K <= 0 || group <= 0)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad shape M=%lld N=%lld K=%lld group=%lld", (long long)M, (long long)N,
                (long long)K, (long long)group);
  // the activations carry one scale per token (act_tile == K) or one per token and weight group
  if (act_tile != K && act_tile != group)
    return fail(QWIX_ERR_UNSUPPORTED, "activation tile %lld: K (per token) or the weight's group %lld", (long long)act_tile,
                (long long)group);
  const size_t need = qwix_hip_qgemm_hadamard_act_workspace_bytes(M, K, act_tile, x_dtype);
  if (need == 0 || !workspace || workspace_bytes < need || !aligned16(workspace))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "workspace of %zu bytes required, got %zu", need, workspace_bytes);
  uint8_t* q = static_cast<uint8_t*>(workspace);
  uint8_t* sa = q + had_align(static_cast<size_t>(M) * K);
  if (int e = qwix_hip_fwht_quantize(x, x_dtype, M, K, pre_sign, post_sign, out_scale, act_tile, QWIX_INT8, q, sa, stream))
    return e;
  // what the caller provides beyond `need` serves the GEMM's K ranges (qwix_hip_qgemm_grouped_workspace_bytes; `need`
  // is a multiple of 256, so the rest is aligned like the workspace)
  const size_t rest = workspace_bytes - need;
  return grouped_impl(q, K, b, ldb_bytes, b_qtype, M, N, K, group, sa, x_dtype, K / act_tile, sb, sb_dtype, nullptr, 0, 0,
                      nullptr, 0, 0, out, out_dtype, ldo, 0, nullptr, stream, rest ? q + need : nullptr, rest);
}
