// Quantized GEMMs on the gfx950 matrix cores (MFMA), dequantize-on-output.
//
//   out[m,n] = epilogue( sum_k a[m,k] * b[n,k] )      a: (M,K), b: (N,K), both K-contiguous
//
// One workgroup of 4 wavefronts (2 x 2) owns a BM x BN tile of the output.  K is walked in BK-byte
// slabs: global -> registers -> LDS (two LDS stages, rows padded by 16 bytes so that the 16-byte
// operand reads of 8 consecutive lanes touch all 32 banks once), operands are read back as
// 16-byte fragments and fed to v_mfma_i32_32x32x32_i8 / v_mfma_f32_32x32x64_f8f6f4.
// The MFMA "A" operand is fed from b and the "B" operand from a, so that each lane ends up with
// 4 consecutive n for a single m: output rows are written with 8/16-byte vector stores.
// Workgroup ids are remapped so that the 8 XCDs (round-robin dispatch) each work on a compact
// block of tiles and share their slabs through their own L2.
#include <type_traits>

#include "common.h"

namespace qwix {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kPad = 16;

// Epilogue description.  The reference scales the accumulator as ((T(acc) * sa) * sb) with one
// rounding per step in the promoted dtype; which of those roundings are to bf16 is decided on the
// host (r0: the converted accumulator, r1: after the lhs scale, r2: after the rhs scale).
struct Epilogue {
  const void* sa;  // per m, or null
  const void* sb;  // per n, or null
  int sa_dtype, sb_dtype, out_dtype;
  int r0, r1, r2;
};

// XCD-aware tile order: consecutive hardware workgroup ids go to different XCDs; give every XCD a
// contiguous run of logical ids, and walk tiles in column groups of 8 tile-rows for L2 reuse.
__device__ __forceinline__ void tile_coords(int tiles_m, int tiles_n, int* tm, int* tn) {
  const int nb = gridDim.x;
  int pid = blockIdx.x;
  if ((nb & 7) == 0) pid = (pid & 7) * (nb >> 3) + (pid >> 3);
  constexpr int GM = 8;
  const int per_group = GM * tiles_n;
  const int group = pid / per_group;
  const int first_m = group * GM;
  const int gsz = min(tiles_m - first_m, GM);
  *tm = first_m + (pid % per_group) % gsz;
  *tn = (pid % per_group) / gsz;
}

__device__ __forceinline__ float load_scale(const void* p, int dtype, int64_t i) {
  return dtype == QWIX_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i])
                            : reinterpret_cast<const float*>(p)[i];
}

// acc[i][j][r]: m = m_base + i*32 + lane%32,  n = n_base + j*32 + 8*(r/4) + 4*(lane/32) + r%4.
template <int OUT, int TM, int TN, typename AccT>
__device__ __forceinline__ void write_tile(const AccT (&acc)[TM][TN], const Epilogue& ep, int m_base, int n_base,
                                           int lane, int M, int N, uint8_t* __restrict__ out, int64_t ldo) {
  const bool vec_ok = (N % 4 == 0);
  const bool r0 = ep.r0 != 0, r1 = ep.r1 != 0, r2 = ep.r2 != 0;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m_base + i * 32 + (lane & 31);
    const bool m_ok = m < M;
    const float sa = (ep.sa != nullptr && m_ok) ? load_scale(ep.sa, ep.sa_dtype, m) : 1.f;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int n = n_base + j * 32 + 8 * qd + 4 * (lane >> 5);
        if (m_ok && n < N) {
          if constexpr (OUT == QWIX_I32) {
            int* o = reinterpret_cast<int*>(out) + static_cast<int64_t>(m) * ldo + n;
            if (vec_ok) {
              *reinterpret_cast<int4*>(o) = make_int4(static_cast<int>(acc[i][j][4 * qd]), static_cast<int>(acc[i][j][4 * qd + 1]),
                                                      static_cast<int>(acc[i][j][4 * qd + 2]), static_cast<int>(acc[i][j][4 * qd + 3]));
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r)
                if (n + r < N) o[r] = static_cast<int>(acc[i][j][4 * qd + r]);
            }
          } else {
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const float sb = (ep.sb != nullptr && n + r < N) ? load_scale(ep.sb, ep.sb_dtype, n + r) : 1.f;
              float t = static_cast<float>(acc[i][j][4 * qd + r]);
              t = r0 ? round_bf16(t) : t;
              t *= sa;
              t = r1 ? round_bf16(t) : t;
              t *= sb;
              v[r] = r2 ? round_bf16(t) : t;
            }
            if constexpr (OUT == QWIX_BF16) {
              uint16_t* o = reinterpret_cast<uint16_t*>(out) + static_cast<int64_t>(m) * ldo + n;
              if (vec_ok) {
                *reinterpret_cast<uint2*>(o) =
                    make_uint2(f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16),
                               f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16));
              } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                  if (n + r < N) o[r] = f32_to_bf16_bits(v[r]);
              }
            } else {
              float* o = reinterpret_cast<float*>(out) + static_cast<int64_t>(m) * ldo + n;
              if (vec_ok) {
                *reinterpret_cast<float4*>(o) = make_float4(v[0], v[1], v[2], v[3]);
              } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                  if (n + r < N) o[r] = v[r];
              }
            }
          }
        }
      }
    }
  }
}

// QT: QWIX_INT8 or QWIX_E4M3.  Wave tile = (BM/2) x (BN/2) = TM x TN MFMA tiles of 32x32.
// Software pipeline: while the MFMAs of k-step s run, the fragments of k-step s+1 are read from
// LDS into a second register set; the slab for the next iteration is fetched from global memory
// at the top of the iteration, written to the other LDS stage before the last k-step, and the
// workgroup barrier plus the first fragment read of the next slab hide behind that last k-step.
template <int QT, int BM, int BN, int BK>
__global__ void __launch_bounds__(256)
    qgemm_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                 int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  constexpr bool IS_INT = (QT == QWIX_INT8);
  constexpr int LDS_STRIDE = BK + kPad;
  constexpr int TM = BM / 64, TN = BN / 64;
  constexpr int KSTEP = IS_INT ? 32 : 64;         // K elements (= bytes) per MFMA
  constexpr int NK = BK / KSTEP;
  static_assert(NK >= 2 && NK % 2 == 0, "the fragment double buffer needs an even number of k-steps");
  constexpr int CH = BK / 16;                      // 16-byte chunks per tile row
  constexpr int A_CHUNKS = BM * CH / 256, B_CHUNKS = BN * CH / 256;
  static_assert(BM * CH % 256 == 0 && BN * CH % 256 == 0, "tile/thread mismatch");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int STAGE = (BM + BN) * LDS_STRIDE;  // stage s: A tile at s*STAGE, B tile right after it

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int tile_m, tile_n;
  tile_coords((M + BM - 1) / BM, (N + BN - 1) / BN, &tile_m, &tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  using AccT = typename std::conditional<IS_INT, v16i, v16f>::type;
  using FragT = typename std::conditional<IS_INT, v4i, v8i>::type;
  AccT acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  uint4 ra[A_CHUNKS], rb[B_CHUNKS];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * 256, row = c / CH, kc = c % CH;
      const int m = m0 + row, k = k0 + kc * 16;
      ra[i] = make_uint4(0, 0, 0, 0);
      if (m < M && k < K) ra[i] = *reinterpret_cast<const uint4*>(A + static_cast<int64_t>(m) * lda + k);
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
      const int c = tid + i * 256, row = c / CH, kc = c % CH;
      const int n = n0 + row, k = k0 + kc * 16;
      rb[i] = make_uint4(0, 0, 0, 0);
      if (n < N && k < K) rb[i] = *reinterpret_cast<const uint4*>(B + static_cast<int64_t>(n) * ldb + k);
    }
  };
  auto store_lds = [&](int s) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * 256, row = c / CH, kc = c % CH;
      *reinterpret_cast<uint4*>(smem + s * STAGE + row * LDS_STRIDE + kc * 16) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
      const int c = tid + i * 256, row = c / CH, kc = c % CH;
      *reinterpret_cast<uint4*>(smem + s * STAGE + (BM + row) * LDS_STRIDE + kc * 16) = rb[i];
    }
  };

  FragT fa[2][TM], fb[2][TN];
  const int a_off = (wm * (BM / 2) + (lane & 31)) * LDS_STRIDE + (lane >> 5) * (KSTEP / 2);
  const int b_off = (BM + wn * (BN / 2) + (lane & 31)) * LDS_STRIDE + (lane >> 5) * (KSTEP / 2);
  auto read_frags = [&](int s, int ks, int buf) {
    const uint8_t* pa = smem + s * STAGE + a_off + ks * KSTEP;
    const uint8_t* pb = smem + s * STAGE + b_off + ks * KSTEP;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if constexpr (IS_INT) {
        fa[buf][i] = *reinterpret_cast<const v4i*>(pa + i * 32 * LDS_STRIDE);
      } else {
        const v4i lo = *reinterpret_cast<const v4i*>(pa + i * 32 * LDS_STRIDE);
        const v4i hi = *reinterpret_cast<const v4i*>(pa + i * 32 * LDS_STRIDE + 16);
        fa[buf][i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if constexpr (IS_INT) {
        fb[buf][j] = *reinterpret_cast<const v4i*>(pb + j * 32 * LDS_STRIDE);
      } else {
        const v4i lo = *reinterpret_cast<const v4i*>(pb + j * 32 * LDS_STRIDE);
        const v4i hi = *reinterpret_cast<const v4i*>(pb + j * 32 * LDS_STRIDE + 16);
        fb[buf][j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    }
  };
  auto mfma_step = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if constexpr (IS_INT)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
        else
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0, 0, 0, 0);
      }
  };

  const int KT = (K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  read_frags(0, 0, 0);
  for (int kt = 0; kt < KT; ++kt) {
    const int cur = kt & 1;
    const bool has_next = kt + 1 < KT;
    if (has_next) load_global((kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks + 1 < NK; ++ks) {
      read_frags(cur, ks + 1, (ks + 1) & 1);
      mfma_step(ks & 1);
    }
    if (has_next) store_lds(cur ^ 1);
    __syncthreads();
    if (has_next) read_frags(cur ^ 1, 0, 0);
    mfma_step((NK - 1) & 1);
  }

  const int m_base = m0 + wm * (BM / 2), n_base = n0 + wn * (BN / 2);
  if (ep.out_dtype == QWIX_BF16) {
    write_tile<QWIX_BF16, TM, TN>(acc, ep, m_base, n_base, lane, M, N, out, ldo);
  } else if (ep.out_dtype == QWIX_F32) {
    write_tile<QWIX_F32, TM, TN>(acc, ep, m_base, n_base, lane, M, N, out, ldo);
  } else {
    if constexpr (IS_INT) write_tile<QWIX_I32, TM, TN>(acc, ep, m_base, n_base, lane, M, N, out, ldo);
  }
}

template <int QT, int BM, int BN, int BK>
int launch_qgemm(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
                 const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  constexpr size_t smem = 2 * (BM + BN) * (BK + kPad);
  auto kern = qgemm_kernel<QT, BM, BN, BK>;
  static bool configured = false;  // idempotent attribute, benign if raced
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
    if (e != hipSuccess) return fail(QWIX_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    configured = true;
  }
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  kern<<<dim3(static_cast<unsigned>(tiles)), 256, smem, st>>>(static_cast<const uint8_t*>(a), lda,
                                                              static_cast<const uint8_t*>(b), ldb, static_cast<int>(M),
                                                              static_cast<int>(N), static_cast<int>(K), ep,
                                                              static_cast<uint8_t*>(out), ldo);
  return check_launch("qgemm");
}

}  // namespace
}  // namespace qwix

using namespace qwix;

extern "C" int qwix_hip_qgemm(const void* a, int64_t lda, const void* b, int64_t ldb, int qtype, int64_t M,
                              int64_t N, int64_t K, const void* sa, int sa_dtype, const void* sb, int sb_dtype,
                              int acc_dtype, void* out, int out_dtype, int64_t ldo, void* stream) {
  if (!a || !b || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null a/b/out");
  if (M <= 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad GEMM shape M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                (long long)K);
  if (qtype != QWIX_INT8 && qtype != QWIX_E4M3)
    return fail(QWIX_ERR_UNSUPPORTED, "qgemm supports int8 x int8 and e4m3 x e4m3 operands (got qtype %d)", qtype);
  if (K % 16 || lda % 16 || ldb % 16 || lda < K || ldb < K || !aligned16(a) || !aligned16(b))
    return fail(QWIX_ERR_UNSUPPORTED, "K, lda, ldb must be multiples of 16 bytes and a/b 16-byte aligned "
                "(K=%lld lda=%lld ldb=%lld)", (long long)K, (long long)lda, (long long)ldb);
  if (ldo < N || !aligned16(out) || (N % 4 == 0 && ldo % 4 != 0))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad output leading dimension %lld for N=%lld", (long long)ldo, (long long)N);
  auto ok_s = [](int d) { return d == QWIX_F32 || d == QWIX_BF16; };
  if ((sa && !ok_s(sa_dtype)) || (sb && !ok_s(sb_dtype)))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "scale dtypes must be f32 or bf16");
  if (out_dtype == QWIX_I32 && qtype != QWIX_INT8)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "raw int32 accumulators exist for int8 operands only");
  if (out_dtype != QWIX_I32 && !ok_s(out_dtype)) return fail(QWIX_ERR_INVALID_ARGUMENT, "bad out dtype %d", out_dtype);
  if (qtype == QWIX_E4M3 && !ok_s(acc_dtype)) return fail(QWIX_ERR_INVALID_ARGUMENT, "bad accumulator dtype %d", acc_dtype);
  // Dtype chain of the reference epilogue: int32 adopts the first scale's dtype (through f32); a
  // float accumulator starts in acc_dtype; each multiply happens in the promotion of both sides.
  Epilogue ep{sa, sb, sa_dtype, sb_dtype, out_dtype, 0, 0, 0};
  int cur = (qtype == QWIX_INT8) ? QWIX_I32 : acc_dtype;
  if (cur == QWIX_BF16) ep.r0 = 1;
  auto step = [&](const void* s, int s_dtype, int* r_after) {
    if (!s) return;
    const int t = (cur == QWIX_I32) ? s_dtype : ((cur == QWIX_F32 || s_dtype == QWIX_F32) ? QWIX_F32 : QWIX_BF16);
    if (cur == QWIX_I32 && t == QWIX_BF16) ep.r0 = 1;
    *r_after = (t == QWIX_BF16);
    cur = t;
  };
  step(sa, sa_dtype, &ep.r1);
  step(sb, sb_dtype, &ep.r2);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool big = (M >= 1024 && N >= 1024);
  if (qtype == QWIX_INT8) {
    if (big) return launch_qgemm<QWIX_INT8, 256, 256, 128>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    return launch_qgemm<QWIX_INT8, 128, 128, 128>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  }
  if (big) return launch_qgemm<QWIX_E4M3, 256, 256, 128>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  return launch_qgemm<QWIX_E4M3, 128, 128, 128>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
}
