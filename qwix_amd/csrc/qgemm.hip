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

struct Epilogue {
  const void* sa;  // per m
  const void* sb;  // per n
  int sa_dtype, sb_dtype, acc_dtype, out_dtype;
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

// Scale-and-cast one accumulator exactly as the reference does: convert to the scale dtype (int32
// goes through f32), one rounding per multiply, lhs scale first.
template <bool IS_INT>
__device__ __forceinline__ float apply_scales(float acc_f, const Epilogue& ep, float sa, float sb) {
  float v = acc_f;
  int cur;  // dtype tag of v
  if constexpr (IS_INT) {
    cur = QWIX_I32;
  } else {
    cur = ep.acc_dtype;
    if (cur == QWIX_BF16) v = round_bf16(v);
  }
  if (ep.sa != nullptr) {
    const int t = (cur == QWIX_I32) ? ep.sa_dtype : ((cur == QWIX_F32 || ep.sa_dtype == QWIX_F32) ? QWIX_F32 : QWIX_BF16);
    if (t == QWIX_BF16) v = round_bf16(round_bf16(v) * sa); else v = v * sa;
    cur = t;
  }
  if (ep.sb != nullptr) {
    const int t = (cur == QWIX_I32) ? ep.sb_dtype : ((cur == QWIX_F32 || ep.sb_dtype == QWIX_F32) ? QWIX_F32 : QWIX_BF16);
    if (t == QWIX_BF16) v = round_bf16(round_bf16(v) * sb); else v = v * sb;
    cur = t;
  }
  return v;
}

__device__ __forceinline__ float load_scale(const void* p, int dtype, int64_t i) {
  return dtype == QWIX_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i])
                            : reinterpret_cast<const float*>(p)[i];
}

// QT: QWIX_INT8 or QWIX_E4M3.  Wave tile = (BM/2) x (BN/2) = TM x TN MFMA tiles of 32x32.
template <int QT, int BM, int BN, int BK>
__global__ void __launch_bounds__(256)
    qgemm_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                 int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  constexpr bool IS_INT = (QT == QWIX_INT8);
  constexpr int LDS_STRIDE = BK + kPad;
  constexpr int TM = BM / 64, TN = BN / 64;
  constexpr int KSTEP = IS_INT ? 32 : 64;         // K elements (= bytes) per MFMA
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
      ra[i] = (m < M && k < K) ? *reinterpret_cast<const uint4*>(A + static_cast<int64_t>(m) * lda + k)
                               : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
      const int c = tid + i * 256, row = c / CH, kc = c % CH;
      const int n = n0 + row, k = k0 + kc * 16;
      rb[i] = (n < N && k < K) ? *reinterpret_cast<const uint4*>(B + static_cast<int64_t>(n) * ldb + k)
                               : make_uint4(0, 0, 0, 0);
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
  auto compute = [&](int s) {
    const uint8_t* pa = smem + s * STAGE + (wm * (BM / 2) + (lane & 31)) * LDS_STRIDE;
    const uint8_t* pb = smem + s * STAGE + (BM + wn * (BN / 2) + (lane & 31)) * LDS_STRIDE;
#pragma unroll
    for (int ks = 0; ks < BK / KSTEP; ++ks) {
      if constexpr (IS_INT) {
        const int off = ks * 32 + (lane >> 5) * 16;
        v4i fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const v4i*>(pa + i * 32 * LDS_STRIDE + off);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[j] = *reinterpret_cast<const v4i*>(pb + j * 32 * LDS_STRIDE + off);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[i], acc[i][j], 0, 0, 0);
      } else {
        const int off = ks * 64 + (lane >> 5) * 32;
        v8i fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const v4i lo = *reinterpret_cast<const v4i*>(pa + i * 32 * LDS_STRIDE + off);
          const v4i hi = *reinterpret_cast<const v4i*>(pa + i * 32 * LDS_STRIDE + off + 16);
          fa[i] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const v4i lo = *reinterpret_cast<const v4i*>(pb + j * 32 * LDS_STRIDE + off);
          const v4i hi = *reinterpret_cast<const v4i*>(pb + j * 32 * LDS_STRIDE + off + 16);
          fb[j] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j], fa[i], acc[i][j], 0, 0, 0, 0, 0, 0);
      }
    }
  };

  const int KT = (K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < KT) load_global((kt + 1) * BK);
    compute(cur);
    if (kt + 1 < KT) store_lds(cur ^ 1);
    __syncthreads();
  }

  // Epilogue.  acc[i][j][r]: m = m0 + wm*BM/2 + i*32 + lane%32,
  //                          n = n0 + wn*BN/2 + j*32 + 8*(r/4) + 4*(lane/32) + r%4.
  const bool vec_ok = (N % 4 == 0);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + wm * (BM / 2) + i * 32 + (lane & 31);
    if (m >= M) continue;
    const float sa = ep.sa ? load_scale(ep.sa, ep.sa_dtype, m) : 1.f;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int n = n0 + wn * (BN / 2) + j * 32 + 8 * qd + 4 * (lane >> 5);
        if (n >= N) continue;
        if (ep.out_dtype == QWIX_I32) {
          if constexpr (IS_INT) {
            int* o = reinterpret_cast<int*>(out) + static_cast<int64_t>(m) * ldo + n;
            if (vec_ok) {
              *reinterpret_cast<int4*>(o) = make_int4(acc[i][j][4 * qd], acc[i][j][4 * qd + 1],
                                                      acc[i][j][4 * qd + 2], acc[i][j][4 * qd + 3]);
            } else {
              for (int r = 0; r < 4 && n + r < N; ++r) o[r] = acc[i][j][4 * qd + r];
            }
          }
          continue;
        }
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float sb = (ep.sb && n + r < N) ? load_scale(ep.sb, ep.sb_dtype, n + r) : 1.f;
          v[r] = apply_scales<IS_INT>(static_cast<float>(acc[i][j][4 * qd + r]), ep, sa, sb);
        }
        if (ep.out_dtype == QWIX_BF16) {
          uint16_t* o = reinterpret_cast<uint16_t*>(out) + static_cast<int64_t>(m) * ldo + n;
          if (vec_ok) {
            *reinterpret_cast<uint2*>(o) =
                make_uint2(f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16),
                           f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16));
          } else {
            for (int r = 0; r < 4 && n + r < N; ++r) o[r] = f32_to_bf16_bits(v[r]);
          }
        } else {
          float* o = reinterpret_cast<float*>(out) + static_cast<int64_t>(m) * ldo + n;
          if (vec_ok) {
            *reinterpret_cast<float4*>(o) = make_float4(v[0], v[1], v[2], v[3]);
          } else {
            for (int r = 0; r < 4 && n + r < N; ++r) o[r] = v[r];
          }
        }
      }
    }
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
  Epilogue ep{sa, sb, sa_dtype, sb_dtype, acc_dtype, out_dtype};
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool big = (M >= 1024 && N >= 1024);
  if (qtype == QWIX_INT8) {
    if (big) return launch_qgemm<QWIX_INT8, 256, 256, 64>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    return launch_qgemm<QWIX_INT8, 128, 128, 64>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  }
  if (big) return launch_qgemm<QWIX_E4M3, 256, 256, 64>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  return launch_qgemm<QWIX_E4M3, 128, 128, 64>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
}
