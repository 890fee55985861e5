// Quantized GEMMs on the gfx950 matrix cores (MFMA), dequantize-on-output.
//
//   out[m,n] = epilogue( sum_k a[m,k] * b[n,k] )      a: (M,K), b: (N,K), both K-contiguous
//
// Tile bodies (device functions of a tile origin and a row limit, shared by all entry points):
//   qgemm_tile      register-staged 128 x 128 tile, any K that is a multiple of 16
//   qgemm_dma_tile  K % 128 == 0: 128-byte K slabs go global -> LDS directly, two stages (three or four where a
//                   problem's tiles are so few per CU that nothing else covers the latency of the loads)
//   qgemm_pp_tile   256 x 256, long K: two wavefront groups half a slab out of phase (ping-pong)
// Kernels around them: dense (one tile per workgroup, XCD-aware tile order), batched (blockIdx.y
// selects the problem), ragged (rows in groups whose sizes live in device memory, one weight panel
// per group), and a skinny kernel for M <= 32 that streams the weights once.
// K is walked in slabs through LDS; rows are stored so that the 16-byte operand reads of 8
// consecutive lanes touch all 32 banks once (padding in the register-staged body, an XOR swizzle in
// the others); operands are read back as 16-byte fragments and fed to v_mfma_i32_32x32x32_i8 /
// v_mfma_f32_32x32x64_f8f6f4.  The MFMA "A" operand is fed from b and the "B" operand from a, so
// that each lane ends up with 4 consecutive n for a single m.
#include <cstdlib>
#include <type_traits>

#include "common.h"

namespace qwix {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kPad = 16;
// Operand tag of the tile bodies for bf16 x bf16 (the float contraction of the dequantize-first path); the
// byte geometry is that of int8: a 128-byte K slab is four MFMA k-steps of 32 bytes per row (16 bf16 values).
constexpr int kOpBf16 = 16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// Swizzle key of the kernels in this file: 16-byte chunk c of the 128-byte LDS row r sits at chunk position
// c ^ swz8(r).  Eight consecutive rows then cover all eight chunk positions; over the sixteen rows that the LDS
// serves per clock for a ds_read_b128 this still leaves two-way bank conflicts, which the sixteen-row key of
// common.h (swz128) removes.  Measured side by side on one box, the conflict-free key is nevertheless 2-5 %
// SLOWER here (int8 4096^3: 72.1 against 70.3 us; 8192^3: 494 against 485 us; the 8-expert ragged GEMM 578
// against 551 us; e4m3 and the one-tile-row kernel unchanged): these kernels run at the board's power limit,
// where faster fragment reads buy nothing and cost clock.  So the eight-row key stays.
__device__ __forceinline__ int swz8(int row) { return row & 7; }

// Epilogue description.  The reference scales the accumulator as ((T(acc) * sa) * sb) with one
// rounding per step in the promoted dtype; which of those roundings are to bf16 is decided on the
// host (r0: the converted accumulator, r1: after the lhs scale, r2: after the rhs scale).
struct Epilogue {
  const void* sa;  // per m, or null
  const void* sb;  // per n, or null
  int sa_dtype, sb_dtype, out_dtype;
  int r0, r1, r2;
  // Zero-point correction of an asymmetric operand (int8 only): acc[m,n] -= zu[m] * zv[n], where one
  // vector holds the zero points and the other the K-sums of the opposite operand's quantized values.
  const int32_t* zu;
  const int32_t* zv;
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
// All scales a lane needs are fetched before its first store, so that the stores (which the
// compiler must keep ordered with loads that may alias) do not serialise the global-load latency.
template <int OUT, int TM, int TN, typename AccT>
__device__ __forceinline__ void write_tile(const AccT (&acc)[TM][TN], const Epilogue& ep, int m_base, int n_base,
                                           int lane, int M, int N, uint8_t* __restrict__ out, int64_t ldo) {
  const bool vec_ok = (N % 4 == 0);
  const bool r0 = ep.r0 != 0, r1 = ep.r1 != 0, r2 = ep.r2 != 0;
  float sav[TM];
  float sbv[TN][4][4];
  if constexpr (OUT != QWIX_I32) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = m_base + i * 32 + (lane & 31);
      sav[i] = (ep.sa != nullptr && m < M) ? load_scale(ep.sa, ep.sa_dtype, m) : 1.f;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int n = n_base + j * 32 + 8 * qd + 4 * (lane >> 5);
#pragma unroll
        for (int r = 0; r < 4; ++r) sbv[j][qd][r] = 1.f;
        if (ep.sb != nullptr) {
          if (vec_ok && n < N) {  // n % 4 == 0: one 8- or 16-byte load
            if (ep.sb_dtype == QWIX_BF16) {
              const uint2 w = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(ep.sb) + n);
              sbv[j][qd][0] = __uint_as_float(w.x << 16);
              sbv[j][qd][1] = __uint_as_float(w.x & 0xFFFF0000u);
              sbv[j][qd][2] = __uint_as_float(w.y << 16);
              sbv[j][qd][3] = __uint_as_float(w.y & 0xFFFF0000u);
            } else {
              const float4 w = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(ep.sb) + n);
              sbv[j][qd][0] = w.x; sbv[j][qd][1] = w.y; sbv[j][qd][2] = w.z; sbv[j][qd][3] = w.w;
            }
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (n + r < N) sbv[j][qd][r] = load_scale(ep.sb, ep.sb_dtype, n + r);
          }
        }
      }
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m_base + i * 32 + (lane & 31);
    const bool m_ok = m < M;
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
              float t;
              if constexpr (std::is_same<AccT, v16i>::value) {
                int a = acc[i][j][4 * qd + r];
                if (ep.zu != nullptr) a -= ep.zu[m] * ep.zv[min(n + r, N - 1)];
                t = static_cast<float>(a);
              } else {
                t = static_cast<float>(acc[i][j][4 * qd + r]);
              }
              t = r0 ? round_bf16(t) : t;
              t *= sav[i];
              t = r1 ? round_bf16(t) : t;
              t *= sbv[j][qd][r];
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
// The tile at rows [m0, m0 + BM) x columns [n0, n0 + BN); rows from M on are neither read nor stored.
template <int QT, int BM, int BN, int BK>
__device__ __forceinline__ void qgemm_tile(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B,
                                           int64_t ldb, int m0, int n0, int M, int N, int K, const Epilogue& ep,
                                           uint8_t* __restrict__ out, int64_t ldo) {
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
__global__ void __launch_bounds__(256)
    qgemm_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                 int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  int tile_m, tile_n;
  tile_coords((M + BM - 1) / BM, (N + BN - 1) / BN, &tile_m, &tile_n);
  qgemm_tile<QT, BM, BN, BK>(A, lda, B, ldb, tile_m * BM, tile_n * BN, M, N, K, ep, out, ldo);
}

// Fast path (K % 128 == 0): the slabs go from global memory straight into LDS
// (global_load_lds_dwordx4: no staging registers, no ds_write instructions).  Each wave-level load
// fills one contiguous KiB of LDS = 8 tile rows x 128 bytes; inside a row the eight 16-byte k-chunks
// are stored at position (chunk ^ swz8(row)), chosen by having each lane fetch the matching global
// chunk, so that the fragment reads of 16 consecutive rows hit all 64 banks.  Rows past M / N are
// clamped to the last valid row (their results are never stored).  Loads for slab kt+1 are issued
// while the MFMAs of slab kt run; the workgroup barrier at the end of the slab waits for them.
// The workgroup is WGM x WGN wavefronts; with 8 wavefronts (two per SIMD) the issue time of one
// wavefront's loads and fragment reads hides behind the other's MFMAs.
// EPI: 0 = no bf16 rounding in the epilogue, 1 = every step rounds to bf16, 2 = flags at run time,
// 3 = flags at run time and zero-point correction, 4 = every step rounds to bf16 and zero-point correction.
#define QWIX_GLDS16(gptr, lptr)                                                                       \
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gptr),             \
                                   (__attribute__((address_space(3))) void*)(lptr), 16, 0, 0)
// The same load from a wave-uniform base pointer plus a per-lane 32-bit byte offset.  The offset is made opaque next to
// the load: the address is then a scalar base register plus a 32-bit vector offset, where an offset that the compiler
// widens to 64 bits ahead of the loop occupies two registers for the whole kernel and costs a 64-bit vector add per load.
#define QWIX_GLDS16_AT(gbase, off32, lptr)                                                            \
  do {                                                                                                \
    uint32_t qwix_off_ = (off32);                                                                     \
    asm volatile("" : "+v"(qwix_off_));                                                               \
    QWIX_GLDS16((gbase) + qwix_off_, lptr);                                                           \
  } while (0)
// The same with the offset variable made opaque in its own register (no copy per load): measured 1 % faster in the
// ping-pong kernel's slab loop, and 20 % slower in the one-slab batched kernel, which therefore takes the form above.
#define QWIX_GLDS16_AT_INPLACE(gbase, off32, lptr)                                                    \
  do {                                                                                                \
    asm volatile("" : "+v"(off32));                                                                   \
    QWIX_GLDS16((gbase) + (off32), lptr);                                                             \
  } while (0)

// The per-row and per-column scales of one wavefront's part of the tile, in the accumulator layout
// (acc[i][j][r]: m = m_base + i*32 + lane%32, n = n_base + j*32 + 8*(r/4) + 4*(lane/32) + r%4).
template <int OUT, int TM, int TN>
__device__ __forceinline__ void fetch_scales(const Epilogue& ep, int m_base, int n_base, int M, int N, int lane,
                                             float (&sav)[TM], float (&sbv)[TN][4][4]) {
  if constexpr (OUT != QWIX_I32) {
    const bool vec_ok = (N % 4 == 0);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = m_base + i * 32 + (lane & 31);
      sav[i] = (ep.sa != nullptr && m < M) ? load_scale(ep.sa, ep.sa_dtype, m) : 1.f;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int n = n_base + j * 32 + 8 * qd + 4 * (lane >> 5);
#pragma unroll
        for (int r = 0; r < 4; ++r) sbv[j][qd][r] = 1.f;
        if (ep.sb != nullptr) {
          if (vec_ok && n < N) {  // n % 4 == 0: one 8- or 16-byte load
            if (ep.sb_dtype == QWIX_BF16) {
              const uint2 w = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(ep.sb) + n);
              sbv[j][qd][0] = __uint_as_float(w.x << 16);
              sbv[j][qd][1] = __uint_as_float(w.x & 0xFFFF0000u);
              sbv[j][qd][2] = __uint_as_float(w.y << 16);
              sbv[j][qd][3] = __uint_as_float(w.y & 0xFFFF0000u);
            } else {
              const float4 w = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(ep.sb) + n);
              sbv[j][qd][0] = w.x; sbv[j][qd][1] = w.y; sbv[j][qd][2] = w.z; sbv[j][qd][3] = w.w;
            }
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (n + r < N) sbv[j][qd][r] = load_scale(ep.sb, ep.sb_dtype, n + r);
          }
        }
      }
  }
}

template <int OUT, int EPI, int TM, int TN, int NWAVES, int LDS_BYTES, bool SYNC = true, typename AccT>
__device__ __forceinline__ void staged_epilogue(const AccT (&acc)[TM][TN], const float (&sav)[TM],
                                                const float (&sbv)[TN][4][4], const Epilogue& ep, int m_base,
                                                int n_base, int M, int N, uint8_t* __restrict__ out, int64_t ldo,
                                                uint8_t* smem, int wave, int lane) {
  constexpr int WTN = TN * 32;
  // ---- epilogue.  acc[i][j][r]: m = m_base + i*32 + lane%32, n = n_base + j*32 + 8*(r/4) + 4*(lane/32) + r%4.
  // The scaled values are staged through this wavefront's own slice of LDS, 32 rows at a time, and
  // leave with 16-byte stores that cover whole 128-byte row segments (a direct store from the MFMA
  // layout would write 16-byte pieces of 32 different rows per instruction).
  using OutT = typename std::conditional<OUT == QWIX_BF16, uint16_t, uint32_t>::type;
  constexpr int ES = sizeof(OutT);
  constexpr int ROWB = WTN * ES + 16;            // staged row pitch in bytes (padded against bank conflicts)
  constexpr int CPR = WTN * ES / 16;             // 16-byte chunks per staged row
  constexpr int EPC = 16 / ES;                   // elements per chunk
  static_assert(NWAVES * 32 * ROWB <= LDS_BYTES, "epilogue staging does not fit in LDS");
  constexpr bool ZP = (EPI == 3 || EPI == 4);  // zero-point correction
  constexpr bool ALL = (EPI == 1 || EPI == 4), RUNTIME = (EPI == 2 || EPI == 3);
  const bool r0 = RUNTIME ? ep.r0 != 0 : ALL, r1 = RUNTIME ? ep.r1 != 0 : ALL, r2 = RUNTIME ? ep.r2 != 0 : ALL;
  int zuv[TM];
  if constexpr (ZP) {
#pragma unroll
    for (int i = 0; i < TM; ++i) zuv[i] = ep.zu[min(m_base + i * 32 + (lane & 31), M - 1)];
  }
  if constexpr (SYNC) __syncthreads();  // every wavefront is done with the slabs; LDS becomes staging space
  uint8_t* stg = smem + wave * (32 * ROWB);
  const bool row_vec = (reinterpret_cast<uintptr_t>(out) % 16 == 0) && ((ldo * ES) % 16 == 0);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    float sa = 1.f;
    if constexpr (OUT != QWIX_I32) sa = sav[i];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        uint8_t* dst = stg + (lane & 31) * ROWB + (j * 32 + 8 * qd + 4 * (lane >> 5)) * ES;
        if constexpr (OUT == QWIX_I32) {
          *reinterpret_cast<int4*>(dst) = make_int4(static_cast<int>(acc[i][j][4 * qd]), static_cast<int>(acc[i][j][4 * qd + 1]),
                                                    static_cast<int>(acc[i][j][4 * qd + 2]), static_cast<int>(acc[i][j][4 * qd + 3]));
        } else if constexpr (ALL && OUT == QWIX_BF16) {
          // Every step rounds to bf16 and the result is bf16: round two values per v_cvt_pk_bf16_f32,
          // and let the last rounding produce the packed output directly.
          uint32_t w[2];
          int zvv[4] = {0, 0, 0, 0};
          if constexpr (ZP) {
            const int n = n_base + j * 32 + 8 * qd + 4 * (lane >> 5);
#pragma unroll
            for (int r = 0; r < 4; ++r) zvv[r] = ep.zv[min(n + r, N - 1)];
          }
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            uint32_t pk;
            if constexpr (ZP)
              pk = pack_bf16x2(static_cast<float>(static_cast<int>(acc[i][j][4 * qd + 2 * h]) - zuv[i] * zvv[2 * h]),
                               static_cast<float>(static_cast<int>(acc[i][j][4 * qd + 2 * h + 1]) - zuv[i] * zvv[2 * h + 1]));
            else
              pk = pack_bf16x2(static_cast<float>(acc[i][j][4 * qd + 2 * h]),
                               static_cast<float>(acc[i][j][4 * qd + 2 * h + 1]));
            pk = pack_bf16x2(__uint_as_float(pk << 16) * sa, __uint_as_float(pk & 0xFFFF0000u) * sa);
            w[h] = pack_bf16x2(__uint_as_float(pk << 16) * sbv[j][qd][2 * h],
                               __uint_as_float(pk & 0xFFFF0000u) * sbv[j][qd][2 * h + 1]);
          }
          *reinterpret_cast<uint2*>(dst) = make_uint2(w[0], w[1]);
        } else {
          float v[4];
          int zvv[4] = {0, 0, 0, 0};
          if constexpr (ZP) {
            const int n = n_base + j * 32 + 8 * qd + 4 * (lane >> 5);
#pragma unroll
            for (int r = 0; r < 4; ++r) zvv[r] = ep.zv[min(n + r, N - 1)];
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float t;
            if constexpr (ZP) t = static_cast<float>(static_cast<int>(acc[i][j][4 * qd + r]) - zuv[i] * zvv[r]);
            else t = static_cast<float>(acc[i][j][4 * qd + r]);
            if (r0) t = round_bf16(t);
            t *= sa;
            if (r1) t = round_bf16(t);
            t *= sbv[j][qd][r];
            if (r2) t = round_bf16(t);
            v[r] = t;
          }
          if constexpr (OUT == QWIX_BF16)
            *reinterpret_cast<uint2*>(dst) =
                make_uint2(f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16),
                           f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16));
          else
            *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        }
      }
    // read back row-major: chunk c of the 32 x CPR grid -> row c / CPR, 16-byte column c % CPR
#pragma unroll
    for (int c0 = 0; c0 < 32 * CPR; c0 += 64) {
      const int c = c0 + lane, row = c / CPR, cc = c % CPR;
      const uint4 v = *reinterpret_cast<const uint4*>(stg + row * ROWB + cc * 16);
      const int mo = m_base + i * 32 + row, no = n_base + cc * EPC;
      if (mo < M && no < N) {
        OutT* o = reinterpret_cast<OutT*>(out) + static_cast<int64_t>(mo) * ldo + no;
        if (row_vec && no + EPC <= N) {
          __builtin_nontemporal_store(__builtin_bit_cast(v4i, v), reinterpret_cast<v4i*>(o));
        } else {
          const OutT* e = reinterpret_cast<const OutT*>(&v);
#pragma unroll
          for (int t = 0; t < EPC; ++t)
            if (no + t < N) o[t] = e[t];
        }
      }
    }
  }
}

// NST: slab stages of the direct-to-LDS tile body.  Two by default; four for the 64 x 64 tile of small problems while
// its workgroups are at most two per CU: they have nothing else to cover the latency of weights that come from HBM
// (three slabs in flight instead of one; with more workgroups per CU the LDS the stages take costs more than it gives).
template <int QT, int BM, int BN, int WGM, int WGN, int OUT, int EPI, int NST = 2>
__device__ __forceinline__ void qgemm_dma_tile(const uint8_t* __restrict__ A, int64_t lda,
                                               const uint8_t* __restrict__ B, int64_t ldb, int m0, int n0, int M,
                                               int N, int K, const Epilogue& ep, uint8_t* __restrict__ out,
                                               int64_t ldo) {
  constexpr bool IS_INT = (QT == QWIX_INT8);
  constexpr bool IS_BF = (QT == kOpBf16);
  constexpr bool B16 = IS_INT || IS_BF;  // 16 bytes per lane and k-step
  constexpr int BK = 128;
  constexpr int NWAVES = WGM * WGN;
  constexpr int WTM = BM / WGM, WTN = BN / WGN;   // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int KSTEP = B16 ? 32 : 64;
  constexpr int NK = BK / KSTEP;
  constexpr int ROWS = BM + BN;
  constexpr int STAGE = ROWS * BK;
  constexpr int LOADS = ROWS / 8 / NWAVES;  // 1 KiB loads per wavefront per slab
  static_assert(ROWS % (8 * NWAVES) == 0 && (BM / 8) % LOADS == 0, "each wavefront loads from one operand");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  using AccT = typename std::conditional<IS_INT, v16i, v16f>::type;
  using FragT = typename std::conditional<B16, v4i, v8i>::type;
  AccT acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  // ---- loader: a wave-uniform base pointer plus this lane's 32-bit offset for each row group
  const int lr = lane >> 3;                       // row inside the 8-row group
  const bool from_a = (wave * LOADS * 8) < BM;    // wave-uniform
  const uint8_t* gbase = from_a ? A : B;
  const int64_t gld = from_a ? lda : ldb;
  const int glim = from_a ? (M - 1) : (N - 1);
  const int grow0 = from_a ? (m0 + wave * LOADS * 8) : (n0 + wave * LOADS * 8 - BM);
  uint32_t goff[LOADS];
#pragma unroll
  for (int j = 0; j < LOADS; ++j)
    goff[j] = static_cast<uint32_t>(min(grow0 + j * 8 + lr, glim)) * static_cast<uint32_t>(gld) +
              (((lane & 7) ^ swz8((wave * LOADS + j) * 8 + lr)) << 4);  // the global k-chunk that lands at position lane & 7
  auto issue_loads = [&](int s, int k0) {
    const uint8_t* gk = gbase + k0;
#pragma unroll
    for (int j = 0; j < LOADS; ++j) QWIX_GLDS16_AT(gk, goff[j], smem + s * STAGE + (wave * LOADS + j) * 1024);
  };

  // ---- fragment addresses: row r, k-chunk c lives at r*128 + ((c ^ swz8(r)) << 4); wave tiles start at multiples of 32
  const int a_row = (wm * WTM + (lane & 31)) * BK;
  const int b_row = (BM + wn * WTN + (lane & 31)) * BK;
  const int hx = lane >> 5, x7 = swz8(lane & 31);
  FragT fa[2][TM], fb[2][TN];
  auto read_frags = [&](int s, int ks, int buf) {
    const uint8_t* base = smem + s * STAGE;
    if constexpr (B16) {
      const int off = ((ks * 2 + hx) ^ x7) << 4;
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[buf][i] = *reinterpret_cast<const v4i*>(base + a_row + i * 32 * BK + off);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[buf][j] = *reinterpret_cast<const v4i*>(base + b_row + j * 32 * BK + off);
    } else {
      const int off = ((ks * 4 + hx * 2) ^ x7) << 4;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const v4i lo = *reinterpret_cast<const v4i*>(base + a_row + i * 32 * BK + off);
        const v4i hi = *reinterpret_cast<const v4i*>(base + a_row + i * 32 * BK + (off ^ 16));
        fa[buf][i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const v4i lo = *reinterpret_cast<const v4i*>(base + b_row + j * 32 * BK + off);
        const v4i hi = *reinterpret_cast<const v4i*>(base + b_row + j * 32 * BK + (off ^ 16));
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
        else if constexpr (IS_BF)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fb[buf][j]),
                                                              __builtin_bit_cast(bf16x8, fa[buf][i]), acc[i][j], 0, 0, 0);
        else
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0, 0, 0, 0);
      }
  };
  // Interleave hints for one k-step: MFMAs in pairs, a fragment read after each pair, and a slab load
  // after each pair while loads remain.
  auto hint_kstep = [&](int n_loads) {
    constexpr int MF = TM * TN, RD = (B16 ? 1 : 2) * (TM + TN);
#pragma unroll
    for (int g = 0; g < MF; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                       // MFMA
      if (g < RD) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);           // DS read
      if (g < n_loads) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);      // VMEM read (LDS DMA)
    }
  };

  const int m_base = m0 + wm * WTM, n_base = n0 + wn * WTN;
  float sbv[TN][4][4];
  // The scale vectors are fetched before the main loop: at the start of the epilogue they would be a
  // cold two-microsecond round trip with nothing to hide behind.
  float sav[TM];
  fetch_scales<OUT, TM, TN>(ep, m_base, n_base, M, N, lane, sav, sbv);
  const int KT = K / BK;
  if constexpr (NST > 2) {
    // Slabs kt + 1 .. kt + NST - 1 are in flight while slab kt is multiplied.  At the end of slab kt: wait until only
    // the loads of the slabs after kt + 1 are outstanding, barrier (everyone's part of slab kt + 1 has landed, everyone
    // is done reading slab kt), and the stage of slab kt is requested again at the start of slab kt + 1.
    auto wait_for = [&](int newer) __attribute__((always_inline)) {  // `newer`: slabs requested after the awaited one
      static_assert((NST == 3 || NST == 4) && 2 * LOADS < 64, "wait counts are written out for three or four stages");
      // vmcnt is a six-bit field in two pieces: bits 3:0 and 15:14
      constexpr int W2 = 0x0F70 | ((2 * LOADS) & 0xF) | (((2 * LOADS) >> 4) << 14);
      constexpr int W1 = 0x0F70 | (LOADS & 0xF) | ((LOADS >> 4) << 14);
      if (newer >= 2) __builtin_amdgcn_s_waitcnt(W2);
      else if (newer == 1) __builtin_amdgcn_s_waitcnt(W1);
      else __builtin_amdgcn_s_waitcnt(0x0F70);
    };
#pragma unroll
    for (int s = 0; s < NST - 1; ++s)
      if (s < KT) issue_loads(s, s * BK);
    wait_for(min(KT - 1, NST - 2));
    __builtin_amdgcn_s_barrier();
    read_frags(0, 0, 0);
    int cur = 0;
    for (int kt = 0; kt < KT; ++kt) {
      const int nxt = cur + 1 == NST ? 0 : cur + 1;
      if (kt + NST - 1 < KT) issue_loads(cur == 0 ? NST - 1 : cur - 1, (kt + NST - 1) * BK);  // the stage of slab kt - 1
#pragma unroll
      for (int ks = 0; ks + 1 < NK; ++ks) {
        read_frags(cur, ks + 1, (ks + 1) & 1);
        mfma_step(ks & 1);
        hint_kstep(ks == 0 ? LOADS : 0);
      }
      mfma_step((NK - 1) & 1);
      if (kt + 1 < KT) {
        wait_for(min(KT - 1, kt + NST - 1) - (kt + 1));
        __builtin_amdgcn_s_barrier();
        read_frags(nxt, 0, 0);
      }
      cur = nxt;
    }
    staged_epilogue<OUT, EPI, TM, TN, NWAVES, NST * STAGE>(acc, sav, sbv, ep, m_base, n_base, M, N, out, ldo, smem, wave,
                                                             lane);
    return;
  }
  issue_loads(0, 0);
  __syncthreads();
  read_frags(0, 0, 0);
  // All loads of a slab are issued during its first k-step, giving them the rest of the slab to land.
  for (int kt = 0; kt < KT - 1; ++kt) {
    const int cur = kt & 1;
    issue_loads(cur ^ 1, (kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks + 1 < NK; ++ks) {
      read_frags(cur, ks + 1, (ks + 1) & 1);
      mfma_step(ks & 1);
      hint_kstep(ks == 0 ? LOADS : 0);
    }
    mfma_step((NK - 1) & 1);
    __syncthreads();
    read_frags(cur ^ 1, 0, 0);
  }
  {  // last slab: nothing left to fetch
    const int cur = (KT - 1) & 1;
#pragma unroll
    for (int ks = 0; ks + 1 < NK; ++ks) {
      read_frags(cur, ks + 1, (ks + 1) & 1);
      mfma_step(ks & 1);
    }
    mfma_step((NK - 1) & 1);
  }

  staged_epilogue<OUT, EPI, TM, TN, NWAVES, 2 * STAGE>(acc, sav, sbv, ep, m_base, n_base, M, N, out, ldo, smem, wave,
                                                         lane);
}

template <int QT, int BM, int BN, int WGM, int WGN, int OUT, int EPI, int NST = 2>
__global__ void __launch_bounds__(WGM * WGN * 64)
    qgemm_dma_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                     int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  int tile_m, tile_n;
  tile_coords((M + BM - 1) / BM, (N + BN - 1) / BN, &tile_m, &tile_n);
  qgemm_dma_tile<QT, BM, BN, WGM, WGN, OUT, EPI, NST>(A, lda, B, ldb, tile_m * BM, tile_n * BN, M, N, K, ep, out, ldo);
}

template <int QT, int BM, int BN, int WGM, int WGN, int OUT, int EPI, int NST = 2>
int launch_dma(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
               const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  constexpr size_t smem = NST * (BM + BN) * 128;
  auto kern = qgemm_dma_kernel<QT, BM, BN, WGM, WGN, OUT, EPI, NST>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  kern<<<dim3(static_cast<unsigned>(tiles)), WGM * WGN * 64, smem, st>>>(
      static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, static_cast<int>(M),
      static_cast<int>(N), static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo);
  return check_launch("qgemm (dma)");
}

// Picks the epilogue specialisation: (bf16 out, all-bf16 rounding), (f32 out, no rounding), raw int32,
// or the run-time-flag version for mixed scale dtypes.
template <int QT, int BM, int BN, int WGM, int WGN, int NST = 2>
int dispatch_dma(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
                 const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  const bool all = ep.r0 && ep.r1 && ep.r2, none = !ep.r0 && !ep.r1 && !ep.r2;
  if (ep.out_dtype == QWIX_I32) {
    if constexpr (QT == QWIX_INT8) return launch_dma<QT, BM, BN, WGM, WGN, QWIX_I32, 0, NST>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    return fail(QWIX_ERR_INVALID_ARGUMENT, "int32 output needs int8 operands");
  }
  if (ep.zu != nullptr) {
    if constexpr (QT == QWIX_INT8) {
      if (ep.out_dtype == QWIX_BF16) return launch_dma<QT, BM, BN, WGM, WGN, QWIX_BF16, 3, NST>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      return launch_dma<QT, BM, BN, WGM, WGN, QWIX_F32, 3, NST>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    }
    return fail(QWIX_ERR_UNSUPPORTED, "zero-point correction needs int8 operands");
  }
  if (ep.out_dtype == QWIX_BF16) {
    if (all) return launch_dma<QT, BM, BN, WGM, WGN, QWIX_BF16, 1, NST>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    return launch_dma<QT, BM, BN, WGM, WGN, QWIX_BF16, 2, NST>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  }
  if (none) return launch_dma<QT, BM, BN, WGM, WGN, QWIX_F32, 0, NST>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  return launch_dma<QT, BM, BN, WGM, WGN, QWIX_F32, 2, NST>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
}

// ------------------------------------------------------------------------------------------------
// One tile row of at most 64 rows against a wide weight (a batch of decode tokens): the weight bytes dominate
// and every one of them is needed once.  A workgroup is NW (2 or 4) wavefronts side by side along N, each with all
// 32 * TM rows and 32 columns of its own; since no two wavefronts share a weight column, the weights go from
// global memory straight into registers (64 contiguous bytes per lane and slab, K permuted to match: lane
// half h holds bytes 64 h .. 64 h + 63 of the 128-byte slab row, and k-step s multiplies bytes 64 h + 16 s ..),
// while the activations go through LDS by direct-to-LDS loads as in the other kernels.  Both are fetched
// DEPTH - 1 slabs ahead (DEPTH LDS stages, DEPTH register sets; 8 in the build): a wavefront waits until all
// but its newest DEPTH - 2 groups of loads have landed (vmcnt counts in order; 6 groups of at most 6 loads stay
// under the counter's limit of 63), meets the others at a barrier, issues the group DEPTH - 1 slabs ahead into
// the stage the barrier has just freed, and multiplies.  Measured with weights from HBM, K 4096, N 14336,
// against the 128 x 128 two-stage tile and the weight-streaming kernel: 32 rows 26.2 / 36.6 / 26.1 us, 64 rows
// 26.6 / 36.8 / 48.0 us; 64 rows, K 8192, N 28672: 57.0 / 73.6 / 156.6 us (with four stages and compiler-
// tracked loads: 31.5 and 65.0 us for the two 64-row cases).  Workgroups of 64 columns then brought the 64-row
// case at N 14336 to 20.4 us and the 32-row case to 17.6 us.  With 128 rows every wavefront reads all 128
// activation rows from LDS per slab for its 32 columns, and a workgroup's stages take 96 KB, one workgroup per
// CU: that variant (six stages) pays while one round of 64-column workgroups covers N, and not under the
// ragged grid (64 groups of 128 rows: 232 against 228 us for the two-stage tile).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {  // vmcnt only: expcnt 7 and lgkmcnt 15 stay open
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

template <int QT, int OUT, int EPI, int TM, int DEPTH, int NW>
__device__ __forceinline__ void qgemm_mid_tile(const uint8_t* __restrict__ A, int64_t lda,
                                               const uint8_t* __restrict__ B, int64_t ldb, int m0, int n0, int M,
                                               int N, int K, const Epilogue& ep, uint8_t* __restrict__ out,
                                               int64_t ldo, int kshift) {
  constexpr bool IS_INT = (QT == QWIX_INT8);
  constexpr int BK = 128, TN = 1;  // TM: 32-row blocks of the tile; DEPTH: slabs of loads kept going, plus one
  constexpr int KSTEP = IS_INT ? 32 : 64;
  constexpr int NK = BK / KSTEP;
  constexpr int ASTAGE = 32 * TM * BK;  // 4 KB of activations per 32 rows and slab
  constexpr int PW = 4 * TM / NW;       // 1 KB pieces (8 rows) of a slab of activations that a wavefront fetches
  static_assert(PW * NW == 4 * TM, "the wavefronts share the activation rows evenly");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  using AccT = typename std::conditional<IS_INT, v16i, v16f>::type;
  using FragT = typename std::conditional<IS_INT, v4i, v8i>::type;
  AccT acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][0][r] = 0;

  const int m_base = m0, n_base = n0 + wave * 32;
  float sav[TM];
  float sbv[TN][4][4];
  fetch_scales<OUT, TM, TN>(ep, m_base, n_base, M, N, lane, sav, sbv);  // oldest loads: done before any slab

  // activations: 32 * TM rows of 128 bytes per slab = 4 * TM pieces of 1 KB (8 rows), PW per wavefront
  const int lr = lane >> 3;
  uint32_t aoff[PW];
#pragma unroll
  for (int j = 0; j < PW; ++j)
    aoff[j] = static_cast<uint32_t>(min(m0 + (wave * PW + j) * 8 + lr, M - 1)) * static_cast<uint32_t>(lda) +
              (((lane & 7) ^ swz8((wave * PW + j) * 8 + lr)) << 4);
  // weights: column n_base + lane % 32, bytes 64 * (lane / 32) .. of the slab
  const int hx = lane >> 5, x7 = swz8(lane & 31);
  const uint32_t boff = static_cast<uint32_t>(min(n_base + (lane & 31), N - 1)) * static_cast<uint32_t>(ldb) + hx * 64;
  v4i breg[DEPTH][4];
  const int KT = K / BK;
  auto issue_group = [&](int kt, int st) {  // PW direct-to-LDS loads + 4 register loads per lane
    kt += kshift;  // this workgroup's first slab (below KT): the slabs are walked from there, wrapping around
    if (kt >= KT) kt -= KT;
    const uint8_t* ga = A + kt * BK;
#pragma unroll
    for (int j = 0; j < PW; ++j) QWIX_GLDS16_AT(ga, aoff[j], smem + st * ASTAGE + (wave * PW + j) * 1024);
    // Issued as asm so that the compiler does not track them: its own waits for these registers, merged over
    // the loop's back edge, come out as vmcnt(0) once per trip and would drain every load in flight.  The
    // explicit waits below are what guarantees that a register set has landed before it is multiplied.
    const uint8_t* gb = B + kt * BK;
    asm volatile("global_load_dwordx4 %0, %4, %5\n\t"
                 "global_load_dwordx4 %1, %4, %5 offset:16\n\t"
                 "global_load_dwordx4 %2, %4, %5 offset:32\n\t"
                 "global_load_dwordx4 %3, %4, %5 offset:48"
                 : "=&v"(breg[st][0]), "=&v"(breg[st][1]), "=&v"(breg[st][2]), "=&v"(breg[st][3])
                 : "v"(boff), "s"(gb)
                 : "memory");
  };
  const int a_row = (lane & 31) * BK;
  FragT fa[2][TM];
  auto read_a = [&](int st, int ks, int buf) {
    const uint8_t* base = smem + st * ASTAGE + a_row;
    if constexpr (IS_INT) {
      const int off = ((hx * 4 + ks) ^ x7) << 4;
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[buf][i] = *reinterpret_cast<const v4i*>(base + i * 32 * BK + off);
    } else {
      const int off = ((hx * 4 + ks * 2) ^ x7) << 4;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const v4i lo = *reinterpret_cast<const v4i*>(base + i * 32 * BK + off);
        const v4i hi = *reinterpret_cast<const v4i*>(base + i * 32 * BK + (off ^ 16));
        fa[buf][i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    }
  };
  auto barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

#pragma unroll
  for (int d = 0; d < DEPTH - 1; ++d)
    if (d < KT) issue_group(d, d);
  for (int kt0 = 0; kt0 < KT; kt0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int kt = kt0 + d;
      if (kt < KT) {  // the same for the whole workgroup
        // the groups after kt (PW + 4 loads each, at most DEPTH - 2 of them) may stay in flight
        constexpr int G = PW + 4;
        static_assert((DEPTH - 2) * G <= 63, "vmcnt is a 6-bit counter");
        static_assert(DEPTH >= 4 && DEPTH <= 8, "the wait below lists the cases");
        const int rem = KT - 1 - kt;
        __builtin_amdgcn_sched_barrier(0);
        switch (rem < DEPTH - 2 ? rem : DEPTH - 2) {
          case 0: wait_vmcnt<0>(); break;
          case 1: wait_vmcnt<G>(); break;
          case 2: wait_vmcnt<2 * G>(); break;
          case 3: wait_vmcnt<3 * G>(); break;
          case 4: wait_vmcnt<4 * G>(); break;
          case 5: wait_vmcnt<(5 * G < 63 ? 5 * G : 63)>(); break;  // 5, 6: not reached unless DEPTH is 7, 8
          default: wait_vmcnt<(6 * G < 63 ? 6 * G : 63)>(); break;
        }
        barrier();  // slab kt is in LDS from every wavefront, and everyone is done reading slab kt - 1
        // The compiler does not know that these registers were in flight until the wait above: pin them here, so
        // that no read or copy of them can be scheduled (or have been hoisted) in front of that wait.
#pragma unroll
        for (int r = 0; r < 4; ++r) asm volatile("" : "+v"(breg[d][r]));
        if (kt + DEPTH - 1 < KT) issue_group(kt + DEPTH - 1, (d + DEPTH - 1) % DEPTH);
        __builtin_amdgcn_sched_barrier(0);
        read_a(d, 0, 0);
#pragma unroll
        for (int ks = 0; ks < NK; ++ks) {
          if (ks + 1 < NK) read_a(d, ks + 1, (ks + 1) & 1);
          FragT fb;
          if constexpr (IS_INT) {
            fb = breg[d][ks];
          } else {
            const v4i lo = breg[d][2 * ks], hi = breg[d][2 * ks + 1];
            fb = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          }
#pragma unroll
          for (int i = 0; i < TM; ++i) {
            if constexpr (IS_INT)
              acc[i][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb, fa[ks & 1][i], acc[i][0], 0, 0, 0);
            else
              acc[i][0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb, fa[ks & 1][i], acc[i][0], 0, 0, 0, 0, 0, 0);
          }
        }
      }
    }
  }
  constexpr int kLds = DEPTH * ASTAGE > 20480 ? DEPTH * ASTAGE : 20480;  // the launch provides at least 20 KB
  staged_epilogue<OUT, EPI, TM, TN, NW, kLds>(acc, sav, sbv, ep, m_base, n_base, M, N, out, ldo, smem, wave,
                                                         lane);
}

template <int QT, int OUT, int EPI, int TM, int DEPTH, int NW>
__global__ void __launch_bounds__(64 * NW)
    qgemm_mid_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb, int M,
                     int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo, int kmul) {
  const int kshift = static_cast<int>((blockIdx.x * static_cast<unsigned>(kmul)) % static_cast<unsigned>(K / 128));
  qgemm_mid_tile<QT, OUT, EPI, TM, DEPTH, NW>(A, lda, B, ldb, blockIdx.y * (32 * TM), blockIdx.x * (32 * NW), M, N, K,
                                              ep, out, ldo, kshift);
}

// ------------------------------------------------------------------------------------------------
// The same one tile row when N is so small that 32-column workgroups do not fill the chip (N up to 8192): the
// KW wavefronts of a workgroup share its 32 columns and split K instead, wavefront w taking slabs w, w + KW, ...
// Activations and weights both go from global memory straight into registers, in the same permuted K order
// (lane half h holds bytes 64 h .. 64 h + 63 of a row's 128-byte slab, for its activation rows as for its
// weight column), so the main loop touches no LDS and has no barrier: every wavefront runs its own pipeline
// of DEPTH register sets, waiting only on its own loads (explicit vmcnt, loads issued as asm as above).  At the
// end the partial accumulators meet in LDS, and wavefront i adds up and stores the i-th block of 32 rows.
// int32 partials add exactly; for e4m3 the f32 sums are those of K / (128 KW) slabs each, added in wavefront order.
template <int QT, int OUT, int EPI, int TM, int DEPTH, int KW>
__global__ void __launch_bounds__(64 * KW)
    qgemm_ksplit_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb, int M,
                        int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo, int kmul) {
  constexpr bool IS_INT = (QT == QWIX_INT8);
  constexpr int BK = 128;
  constexpr int NK = IS_INT ? 4 : 2;  // MFMAs per slab and 32-row block
  constexpr int G = 4 * TM + 4;       // loads per slab and lane
  static_assert((DEPTH - 2) * G <= 63, "vmcnt is a 6-bit counter");
  static_assert(DEPTH >= 3 && DEPTH <= 8 && TM <= KW, "the waits and the final reduction list these cases");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n0 = blockIdx.x * 32;

  using AccT = typename std::conditional<IS_INT, v16i, v16f>::type;
  using FragT = typename std::conditional<IS_INT, v4i, v8i>::type;
  AccT acc[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0;
  float sav[TM];
  float sbv[1][4][4];
  fetch_scales<OUT, TM, 1>(ep, 0, n0, M, N, lane, sav, sbv);  // oldest loads: done before any slab is used

  const int hx = lane >> 5;
  uint32_t aoff[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i)
    aoff[i] = static_cast<uint32_t>(min(i * 32 + (lane & 31), M - 1)) * static_cast<uint32_t>(lda) + hx * 64;
  const uint32_t boff = static_cast<uint32_t>(min(n0 + (lane & 31), N - 1)) * static_cast<uint32_t>(ldb) + hx * 64;
  v4i areg[DEPTH][TM][4], breg[DEPTH][4];
  const int KT = K / BK;
  const int kshift = static_cast<int>((blockIdx.x * static_cast<unsigned>(kmul)) % static_cast<unsigned>(KT));
  auto issue_group = [&](int kt, int st) {  // 4 TM + 4 register loads per lane, not tracked by the compiler
    kt += kshift;
    if (kt >= KT) kt -= KT;
    const uint8_t* ga = A + kt * BK;
    const uint8_t* gb = B + kt * BK;
#pragma unroll
    for (int i = 0; i < TM; ++i)
      asm volatile("global_load_dwordx4 %0, %4, %5\n\t"
                   "global_load_dwordx4 %1, %4, %5 offset:16\n\t"
                   "global_load_dwordx4 %2, %4, %5 offset:32\n\t"
                   "global_load_dwordx4 %3, %4, %5 offset:48"
                   : "=&v"(areg[st][i][0]), "=&v"(areg[st][i][1]), "=&v"(areg[st][i][2]), "=&v"(areg[st][i][3])
                   : "v"(aoff[i]), "s"(ga)
                   : "memory");
    asm volatile("global_load_dwordx4 %0, %4, %5\n\t"
                 "global_load_dwordx4 %1, %4, %5 offset:16\n\t"
                 "global_load_dwordx4 %2, %4, %5 offset:32\n\t"
                 "global_load_dwordx4 %3, %4, %5 offset:48"
                 : "=&v"(breg[st][0]), "=&v"(breg[st][1]), "=&v"(breg[st][2]), "=&v"(breg[st][3])
                 : "v"(boff), "s"(gb)
                 : "memory");
  };

  const int mine = KT > wave ? (KT - wave + KW - 1) / KW : 0;  // slabs of this wavefront: wave + j * KW
#pragma unroll
  for (int d = 0; d < DEPTH - 1; ++d)
    if (d < mine) issue_group(wave + d * KW, d);
  for (int j0 = 0; j0 < mine; j0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int j = j0 + d;
      if (j < mine) {  // the same for the whole wavefront
        const int rem = mine - 1 - j;  // the groups after j (at most DEPTH - 2 of them) may stay in flight
        __builtin_amdgcn_sched_barrier(0);
        switch (rem < DEPTH - 2 ? rem : DEPTH - 2) {
          case 0: wait_vmcnt<0>(); break;
          case 1: wait_vmcnt<G>(); break;
          case 2: wait_vmcnt<(2 * G < 63 ? 2 * G : 63)>(); break;
          case 3: wait_vmcnt<(3 * G < 63 ? 3 * G : 63)>(); break;
          case 4: wait_vmcnt<(4 * G < 63 ? 4 * G : 63)>(); break;
          case 5: wait_vmcnt<(5 * G < 63 ? 5 * G : 63)>(); break;
          default: wait_vmcnt<(6 * G < 63 ? 6 * G : 63)>(); break;
        }
        __builtin_amdgcn_sched_barrier(0);
        // pin the set that has just landed: nothing may read or copy it in front of the wait above
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          asm volatile("" : "+v"(breg[d][r]));
#pragma unroll
          for (int i = 0; i < TM; ++i) asm volatile("" : "+v"(areg[d][i][r]));
        }
        // set (d - 1) was multiplied one slab ago: refill it DEPTH - 1 slabs ahead
        if (j + DEPTH - 1 < mine) issue_group(wave + (j + DEPTH - 1) * KW, (d + DEPTH - 1) % DEPTH);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < NK; ++ks) {
          FragT fb;
          if constexpr (IS_INT) {
            fb = breg[d][ks];
          } else {
            const v4i lo = breg[d][2 * ks], hi = breg[d][2 * ks + 1];
            fb = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          }
#pragma unroll
          for (int i = 0; i < TM; ++i) {
            if constexpr (IS_INT) {
              acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb, areg[d][i][ks], acc[i], 0, 0, 0);
            } else {
              const v4i lo = areg[d][i][2 * ks], hi = areg[d][i][2 * ks + 1];
              const v8i fa = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
              acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb, fa, acc[i], 0, 0, 0, 0, 0, 0);
            }
          }
        }
      }
    }
  }
  // partial accumulators -> LDS (behind the 20 KB that the epilogue stages through), [wave][block][register][lane]
  constexpr int kStage = 20480;
  using Word = typename std::conditional<IS_INT, int, float>::type;
  Word* part = reinterpret_cast<Word*>(smem + kStage);
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) part[((wave * TM + i) * 16 + r) * 64 + lane] = acc[i][r];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (wave == i) {  // wavefront i finishes block i
      AccT total[1][1];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        Word t = part[((0 * TM + i) * 16 + r) * 64 + lane];
#pragma unroll
        for (int w = 1; w < KW; ++w) t += part[((w * TM + i) * 16 + r) * 64 + lane];
        total[0][0][r] = t;
      }
      const float sav1[1] = {sav[i]};
      staged_epilogue<OUT, EPI, 1, 1, KW, kStage, false>(total, sav1, sbv, ep, i * 32, n0, M, N, out, ldo, smem, wave, lane);
    }
  }
}

template <int QT, int OUT, int EPI = 2>
int launch_mid(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
               const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  // LDS: kDepth stages of activations, and at least the 18 KB the epilogue stages through
#define QWIX_MID(TMM, NWW) QWIX_MID_D(TMM, NWW, ((4 * TMM / NWW + 4) * 6 <= 63 ? 8 : 6))
#define QWIX_MID_D(TMM, NWW, DD)                                                                                  \
  {                                                                                                               \
    constexpr int kDepth = DD; /* the groups in flight must stay under vmcnt's 63 */                               \
    constexpr size_t smem = kDepth * 32 * TMM * 128 > 20480 ? kDepth * 32 * TMM * 128 : 20480;                     \
    auto kern = qgemm_mid_kernel<QT, OUT, EPI, TMM, kDepth, NWW>;                                                 \
    static LdsGrant granted;                                                                                      \
    if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;                        \
    kern<<<dim3(static_cast<unsigned>((N + 32 * NWW - 1) / (32 * NWW)),                                           \
                static_cast<unsigned>((M + 32 * TMM - 1) / (32 * TMM))), 64 * NWW, smem, st>>>(                    \
        static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, static_cast<int>(M),            \
        static_cast<int>(N), static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo, kmul);                     \
  }
  // Workgroups of 2 wavefronts (64 columns) for up to 32 rows, and for 64 rows while 128-column workgroups
  // would leave CUs without one: twice the workgroups, twice the CUs that pull weights.  Measured, weights
  // from HBM, 2 / 4 wavefronts, K 4096, N 14336: 32 rows 17.5 / 23.4 us, 64 rows 20.3 / 26.4 us; K 8192,
  // N 8192: 23.9 / 37.4 and 30.5 / 42.8 us; K 8192, N 28672: 51.8 / 54.2 and 62.6 / 55.0 us.
  const bool narrow = (N + 127) / 128 < 192;
  // Up to N 8192 and 64 rows a workgroup is a single wavefront (32 columns): 10 to 15 % less again (64 rows,
  // K 4096, N 4096 / 6144: 16.6 / 16.3 against 19.6 / 18.7 us; K 14336, N 4096: 44.1 against 52.6 us).
  // Workgroup b starts at slab 5 b (mod K / 128) and wraps around: with a power-of-two row pitch all workgroups
  // would otherwise ask the same few memory channels for the same K offset of their rows at the same time
  // (K 8192, N 28672, 64 rows: 49.3 against 54.9 us; K 4096, N 14336, 32 rows: 16.2 against 17.6 us).  Integer
  // sums do not depend on the order; e4m3 sums are then added in an order that depends on the column block.
  constexpr int kmul = 5;
  // N up to 8192: four wavefronts split K over the same 32 columns (32 rows, K 4096, N 6144: 12.3 against 14.2 us
  // for single-wavefront workgroups, K 8192, N 8192: 19.5 against 22.0 us; 64 rows: 5 % less).
  if (M <= 64 && (N + 63) / 64 <= 128 && K >= 1024) {
#define QWIX_KSPLIT(TMM, DD)                                                                                      \
  {                                                                                                               \
    constexpr int kKW = 4;                                                                                        \
    constexpr size_t smem = 20480 + kKW * TMM * 4096;                                                             \
    auto kern = qgemm_ksplit_kernel<QT, OUT, EPI, TMM, DD, kKW>;                                                  \
    static LdsGrant granted;                                                                                      \
    if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;                        \
    kern<<<dim3(static_cast<unsigned>((N + 31) / 32)), 64 * kKW, smem, st>>>(                                     \
        static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, static_cast<int>(M),            \
        static_cast<int>(N), static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo, kmul);                     \
  }
    if (M <= 32) QWIX_KSPLIT(1, 6)
    else QWIX_KSPLIT(2, 4)
#undef QWIX_KSPLIT
  } else if (M <= 64 && (N + 63) / 64 <= 128) {
    if (M <= 32) QWIX_MID(1, 1)
    else QWIX_MID(2, 1)
  } else if (M <= 32) {
    QWIX_MID(1, 2)
  } else if (M > 128) {
    QWIX_MID_D(4, 2, 4)  // two tile rows side by side: four stages, 64 KB, two workgroups per CU
  } else if (M > 64) {
    if ((N + 63) / 64 <= 256) QWIX_MID(4, 2)
    else QWIX_MID(4, 4)
  } else {
    if (narrow) QWIX_MID(2, 2)
    else QWIX_MID(2, 4)
  }
#undef QWIX_MID
#undef QWIX_MID_D
  return check_launch("qgemm (one tile row)");
}

// ------------------------------------------------------------------------------------------------
// Ping-pong variant of the 256 x 256 kernel for long K.  The eight wavefronts form two groups (the
// upper and the lower 128 rows of the tile; the two wavefronts that share a SIMD are in different
// groups) that run half a slab out of phase: while one group is in its memory phase (read all
// fragments of a slab from LDS into registers, issue its direct-to-LDS loads of A), the other is in
// its compute phase (the slab's MFMAs back to back at raised priority, one load of B after each
// k-step), so the matrix pipe of every SIMD always has a wavefront that does little else.  Two
// workgroup barriers per slab keep the phases aligned; one extra barrier at the start of the lower
// group and at the end of the upper group produces the offset.
//   LDS: A in two stages of 32 KB, B in three (160 KB in all).  A wavefront loads 32 rows of A (its
// group's half) for the next slab and 32 rows of B for the slab after that; the third B stage is
// what makes room for loading B two slabs ahead, which gives those loads three phases to land and
// lets them be issued from the compute phase without a wait behind them.  Every load is waited for
// by the wavefront that issued it (vmcnt, oldest first) before the barrier that publishes it.
template <int QT, int OUT, int EPI>
__device__ __forceinline__ void qgemm_pp_tile(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B,
                                              int64_t ldb, int m0, int n0, int M, int N, int K, const Epilogue& ep,
                                              uint8_t* __restrict__ out, int64_t ldo) {
  constexpr bool IS_INT = (QT == QWIX_INT8);
  constexpr bool IS_BF = (QT == kOpBf16);
  constexpr bool B16 = IS_INT || IS_BF;  // 16 bytes per lane and k-step
  constexpr int BM = 256, BN = 256, BK = 128, WGN = 4;
  constexpr int TM = 4, TN = 2;                 // wave tile 128 x 64
  constexpr int KSTEP = B16 ? 32 : 64, NK = BK / KSTEP;
  constexpr int A_STAGE = BM * BK, B_STAGE = BN * BK, B_BASE = 2 * A_STAGE;
  constexpr int LDS_BYTES = 2 * A_STAGE + 3 * B_STAGE;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;   // wm is also the phase group

  using AccT = typename std::conditional<IS_INT, v16i, v16f>::type;
  using FragT = typename std::conditional<B16, v4i, v8i>::type;
  AccT acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  // ---- loader: this wavefront brings rows [wm*128 + wn*32, +32) of A and of B, 8 rows per instruction
  const int lr = lane >> 3;
  const int lrow0 = wm * 128 + wn * 32;
  uint32_t goffa[4], goffb[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t lc = static_cast<uint32_t>((lane & 7) ^ swz8(lrow0 + j * 8 + lr));
    goffa[j] = static_cast<uint32_t>(min(m0 + lrow0 + j * 8 + lr, M - 1)) * static_cast<uint32_t>(lda) + lc * 16;
    goffb[j] = static_cast<uint32_t>(min(n0 + lrow0 + j * 8 + lr, N - 1)) * static_cast<uint32_t>(ldb) + lc * 16;
  }
  auto load_a = [&](int kt) {  // own half of the A rows of slab kt
    const uint8_t* gk = A + kt * BK;
    uint8_t* dst = smem + (kt & 1) * A_STAGE + lrow0 * BK;
#pragma unroll
    for (int j = 0; j < 4; ++j) QWIX_GLDS16_AT_INPLACE(gk, goffa[j], dst + j * 1024);
  };
  auto load_b = [&](int kt, int stage) {  // own half of the B rows of slab kt
    const uint8_t* gk = B + kt * BK;
    uint8_t* dst = smem + B_BASE + stage * B_STAGE + lrow0 * BK;
#pragma unroll
    for (int j = 0; j < 4; ++j) QWIX_GLDS16_AT_INPLACE(gk, goffb[j], dst + j * 1024);
  };

  // ---- fragments of a whole slab
  const int a_row = (wm * 128 + (lane & 31)) * BK;
  const int b_row = B_BASE + (wn * 64 + (lane & 31)) * BK;
  const int hx = lane >> 5, x7 = swz8(lane & 31);
  FragT fa[NK][TM], fb[NK][TN];
  auto read_slab = [&](int a_stage, int b_stage) {
    const uint8_t* pa = smem + a_stage * A_STAGE + a_row;
    const uint8_t* pb = smem + b_stage * B_STAGE + b_row;
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      if constexpr (B16) {
        const int off = ((ks * 2 + hx) ^ x7) << 4;
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[ks][i] = *reinterpret_cast<const v4i*>(pa + i * 32 * BK + off);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[ks][j] = *reinterpret_cast<const v4i*>(pb + j * 32 * BK + off);
      } else {
        const int off = ((ks * 4 + hx * 2) ^ x7) << 4;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const v4i lo = *reinterpret_cast<const v4i*>(pa + i * 32 * BK + off);
          const v4i hi = *reinterpret_cast<const v4i*>(pa + i * 32 * BK + (off ^ 16));
          fa[ks][i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const v4i lo = *reinterpret_cast<const v4i*>(pb + j * 32 * BK + off);
          const v4i hi = *reinterpret_cast<const v4i*>(pb + j * 32 * BK + (off ^ 16));
          fb[ks][j] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
      }
    }
  };
  // s_waitcnt on vmcnt only (expcnt 7, lgkmcnt 15 stay open): all but the newest `left` direct-to-LDS
  // loads of this wavefront have landed
  auto wait_loads = [&](int left) {  // left: 0 or 4
    if (left == 0) __builtin_amdgcn_s_waitcnt(0x0F70); else __builtin_amdgcn_s_waitcnt(0x0F74);
  };
  auto barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  const int KT = K / BK;  // >= 2
  // The scale vectors are first needed in the epilogue, where a cold fetch (address translation plus a trip
  // to HBM) would stall every wavefront with nothing to hide behind.  Touch this wavefront's pieces of them
  // now, under the equally cold first slab loads: 128 row scales and 64 column scales, 8 / 4 bytes per lane.
  uint32_t warm_a = 0, warm_b = 0;
  if constexpr (OUT != QWIX_I32) {
    const int m_base = m0 + wm * 128, n_base = n0 + wn * 64;
    if (ep.sa != nullptr) {
      const int64_t es = ep.sa_dtype == QWIX_BF16 ? 2 : 4;
      const int64_t want = (static_cast<int64_t>(m_base) * es + lane * 8) & ~int64_t{3}, last = (M * es - 4) & ~int64_t{3};
      const int64_t off = want < last ? want : last;
      warm_a = *reinterpret_cast<const uint32_t*>(static_cast<const uint8_t*>(ep.sa) + off);
    }
    if (ep.sb != nullptr) {
      const int64_t es = ep.sb_dtype == QWIX_BF16 ? 2 : 4;
      const int64_t want = (static_cast<int64_t>(n_base) * es + lane * 4) & ~int64_t{3}, last = (N * es - 4) & ~int64_t{3};
      const int64_t off = want < last ? want : last;
      warm_b = *reinterpret_cast<const uint32_t*>(static_cast<const uint8_t*>(ep.sb) + off);
    }
  }
  // ---- prologue: A of slab 0, B of slabs 0 and 1 (each wavefront its rows)
  load_a(0);
  load_b(0, 0);
  load_b(1, 1);
  wait_loads(0);
  asm volatile("" ::"v"(warm_a), "v"(warm_b));  // the touches above have landed too; their values are not used
  barrier();
  if (wm == 1) barrier();  // the lower group starts half a slab late

  // B is loaded two slabs ahead, during the compute phase, one load after each k-step's MFMAs (those
  // loads have three phases to land); A one slab ahead, in the memory phase.  The waits before the
  // barriers leave the four loads just issued in flight and cover the four issued one phase earlier.
  int bst = 0;  // B stage of slab kt = kt % 3
  // One slab; whether A of the next slab and B of the one after it are still to be requested is known at compile time,
  // so that the steady state is one basic block (a branch would end the scheduling regions that the fences below
  // delimit): the loop runs the slabs that request both, the last two slabs follow it.
  auto slab = [&](int kt, auto more_a_tag, auto more_b_tag) __attribute__((always_inline)) {
    constexpr bool more_a = decltype(more_a_tag)::value, more_b = decltype(more_b_tag)::value;
    // memory phase
    read_slab(kt & 1, bst);
    __builtin_amdgcn_sched_barrier(0);  // fragment reads first: the loads below may not slip in front of them
    if constexpr (more_a) {
      load_a(kt + 1);
      wait_loads(4);
    } else {
      wait_loads(0);
    }
    barrier();
    // compute phase
    const int bst2 = bst == 0 ? 2 : bst - 1;  // (kt + 2) % 3
    const uint8_t* gkb = B + (kt + 2) * BK;
    uint8_t* dstb = smem + B_BASE + bst2 * B_STAGE + lrow0 * BK;
    __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          if constexpr (IS_INT)
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ks][j], fa[ks][i], acc[i][j], 0, 0, 0);
          else if constexpr (IS_BF)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fb[ks][j]),
                                                                __builtin_bit_cast(bf16x8, fa[ks][i]), acc[i][j], 0, 0, 0);
          else
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[ks][j], fa[ks][i], acc[i][j], 0, 0, 0, 0, 0, 0);
        }
      if constexpr (more_b) {
#pragma unroll
        for (int j = ks * (4 / NK); j < (ks + 1) * (4 / NK); ++j) QWIX_GLDS16_AT_INPLACE(gkb, goffb[j], dstb + j * 1024);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_setprio(0);
    if constexpr (more_b) wait_loads(4); else wait_loads(0);
    barrier();
    bst = bst == 2 ? 0 : bst + 1;
  };
  using T_ = std::true_type;
  using F_ = std::false_type;
  int kt = 0;
  for (; kt + 2 < KT; ++kt) slab(kt, T_{}, T_{});
  if (kt + 1 < KT) {
    slab(kt, T_{}, F_{});
    ++kt;
  }
  slab(kt, F_{}, F_{});
  if (wm == 0) barrier();

  const int m_base = m0 + wm * 128, n_base = n0 + wn * 64;
  float sav[TM];
  float sbv[TN][4][4];
  fetch_scales<OUT, TM, TN>(ep, m_base, n_base, M, N, lane, sav, sbv);
  staged_epilogue<OUT, EPI, TM, TN, 8, LDS_BYTES>(acc, sav, sbv, ep, m_base, n_base, M, N, out, ldo, smem, wave, lane);
}

template <int QT, int OUT, int EPI>
__global__ void __launch_bounds__(512)
    qgemm_pp_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb, int M,
                    int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  int tile_m, tile_n;
  tile_coords((M + 255) / 256, (N + 255) / 256, &tile_m, &tile_n);
  qgemm_pp_tile<QT, OUT, EPI>(A, lda, B, ldb, tile_m * 256, tile_n * 256, M, N, K, ep, out, ldo);
}

template <int QT, int OUT, int EPI>
int launch_pp(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
              const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  constexpr size_t smem = 5 * 256 * 128;
  auto kern = qgemm_pp_kernel<QT, OUT, EPI>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
  kern<<<dim3(static_cast<unsigned>(tiles)), 512, smem, st>>>(
      static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, static_cast<int>(M),
      static_cast<int>(N), static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo);
  return check_launch("qgemm (ping-pong)");
}

template <int QT>
int dispatch_pp(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
                const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  const bool all = ep.r0 && ep.r1 && ep.r2, none = !ep.r0 && !ep.r1 && !ep.r2;
  if (ep.zu != nullptr) {
    if constexpr (QT == QWIX_INT8) {
      if (ep.out_dtype == QWIX_BF16 && all) return launch_pp<QT, QWIX_BF16, 4>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      if (ep.out_dtype == QWIX_BF16) return launch_pp<QT, QWIX_BF16, 3>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      return launch_pp<QT, QWIX_F32, 3>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    }
    return fail(QWIX_ERR_UNSUPPORTED, "zero-point correction needs int8 operands");
  }
  if (ep.out_dtype == QWIX_BF16) {
    if (all) return launch_pp<QT, QWIX_BF16, 1>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    return launch_pp<QT, QWIX_BF16, 2>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  }
  if (none) return launch_pp<QT, QWIX_F32, 0>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  return launch_pp<QT, QWIX_F32, 2>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
}

template <int QT, int BM, int BN, int BK>
int launch_qgemm(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
                 const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  constexpr size_t smem = 2 * (BM + BN) * (BK + kPad);
  auto kern = qgemm_kernel<QT, BM, BN, BK>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  kern<<<dim3(static_cast<unsigned>(tiles)), 256, smem, st>>>(static_cast<const uint8_t*>(a), lda,
                                                              static_cast<const uint8_t*>(b), ldb, static_cast<int>(M),
                                                              static_cast<int>(N), static_cast<int>(K), ep,
                                                              static_cast<uint8_t*>(out), ldo);
  return check_launch("qgemm");
}

// ------------------------------------------------------------------------------------------------
// Ragged GEMM (mixture-of-experts): the rows of A are split into consecutive groups whose sizes are
// read from device memory; the rows of group g meet B_g, the g-th (N, K) panel.  Rows that belong
// to no group (past the sum of the sizes) come out as zeros.  No host synchronisation: the grid
// is sized for the worst case, floor(M / BM) + G + 1 tile rows, and every workgroup finds its
// tile by walking the group sizes (wave-uniform scalar work); workgroups past the last tile exit.
struct Ragged {
  const int32_t* group_sizes;  // G entries
  int G;
  int64_t b_group_stride;   // bytes between consecutive B panels
  int64_t sb_group_stride;  // elements between the rhs scale vectors of consecutive groups (0: one shared vector)
};

constexpr int kRaggedChunk = 16;  // consecutive tile ids that run on one XCD

// Returns 0: no tile, 1: a tile of group *g, 2: a tile of rows that belong to no group.
// Tile ids are numbered group by group; inside a group they walk 8 tile rows per column so that
// tiles that run together share operand panels.  Runs of kRaggedChunk ids are dealt out to the 8
// XCDs in turn, which also spreads the unused ids at the end over all of them.
template <int BM, int BN>
__device__ __forceinline__ int ragged_tile(const Ragged& rg, int M, int N, int* g, int* m0, int* m_lim, int* n0) {
  int pid = blockIdx.x;  // gridDim.x % (8 * kRaggedChunk) == 0
  {
    const int k = pid >> 3, x = pid & 7;
    pid = ((k / kRaggedChunk) * 8 + x) * kRaggedChunk + k % kRaggedChunk;
  }
  const int tiles_n = (N + BN - 1) / BN;
  int row = 0, first = 0, kind = 0;
  for (int i = 0; i <= rg.G; ++i) {
    // sizes are clamped so that no group reaches past row M; the pass i == G covers the rows left over
    const int sz = i < rg.G ? min(max(rg.group_sizes[i], 0), M - row) : M - row;
    const int nt = (sz + BM - 1) / BM;
    const int cnt = nt * tiles_n;
    if (kind == 0 && pid < first + cnt) {
      constexpr int GM = 8;
      const int r = pid - first, per = GM * tiles_n;
      const int fm = (r / per) * GM, gsz = min(nt - fm, GM);
      *g = i;
      *m0 = row + (fm + (r % per) % gsz) * BM;
      *m_lim = row + sz;
      *n0 = ((r % per) / gsz) * BN;
      kind = i < rg.G ? 1 : 2;
    }
    first += cnt;
    row += sz;
  }
  return kind;
}

template <int BM, int BN, typename OutT>
__device__ __forceinline__ void zero_tile(uint8_t* out, int64_t ldo, int m0, int m_lim, int n0, int N, int nthreads) {
  const int rows = min(BM, m_lim - m0), cols = min(BN, N - n0);
  for (int idx = threadIdx.x; idx < rows * cols; idx += nthreads)
    reinterpret_cast<OutT*>(out)[static_cast<int64_t>(m0 + idx / cols) * ldo + n0 + idx % cols] = 0;
}

__device__ __forceinline__ Epilogue group_epilogue(const Epilogue& ep, const Ragged& rg, int g) {
  Epilogue e = ep;
  if (ep.sb != nullptr)
    e.sb = static_cast<const uint8_t*>(ep.sb) + g * rg.sb_group_stride * (ep.sb_dtype == QWIX_BF16 ? 2 : 4);
  return e;
}

template <int QT, int BM, int BN, int WGM, int WGN, int OUT>
__global__ void __launch_bounds__(WGM * WGN * 64)
    qgemm_ragged_dma_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                            Ragged rg, int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  int g, m0, m_lim, n0;
  const int kind = ragged_tile<BM, BN>(rg, M, N, &g, &m0, &m_lim, &n0);
  if (kind == 0) return;
  using OutT = typename std::conditional<OUT == QWIX_BF16, uint16_t, uint32_t>::type;
  if (kind == 2) {
    zero_tile<BM, BN, OutT>(out, ldo, m0, m_lim, n0, N, WGM * WGN * 64);
    return;
  }
  const Epilogue e = group_epilogue(ep, rg, g);
  qgemm_dma_tile<QT, BM, BN, WGM, WGN, OUT, (OUT == QWIX_I32 ? 0 : 2)>(A, lda, B + g * rg.b_group_stride, ldb, m0, n0,
                                                                        m_lim, N, K, e, out, ldo);
}

inline unsigned ragged_grid(int64_t M, int64_t N, int64_t G, int BM, int BN) {
  const int64_t tiles = (M / BM + G + 1) * ((N + BN - 1) / BN);
  const int64_t unit = 8 * kRaggedChunk;
  return static_cast<unsigned>((tiles + unit - 1) / unit * unit);
}

template <int QT, int OUT, int EPI>
__global__ void __launch_bounds__(512)
    qgemm_ragged_pp_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                           Ragged rg, int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  int g, m0, m_lim, n0;
  const int kind = ragged_tile<256, 256>(rg, M, N, &g, &m0, &m_lim, &n0);
  if (kind == 0) return;
  using OutT = typename std::conditional<OUT == QWIX_BF16, uint16_t, uint32_t>::type;
  if (kind == 2) {
    zero_tile<256, 256, OutT>(out, ldo, m0, m_lim, n0, N, 512);
    return;
  }
  const Epilogue e = group_epilogue(ep, rg, g);
  qgemm_pp_tile<QT, OUT, EPI>(A, lda, B + g * rg.b_group_stride, ldb, m0, n0, m_lim, N, K, e, out, ldo);
}

template <int QT, int OUT, int EPI>
int launch_ragged_pp_epi(const void* a, int64_t lda, const void* b, int64_t ldb, const Ragged& rg, int64_t M, int64_t N,
                         int64_t K, const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  constexpr size_t smem = 5 * 256 * 128;
  auto kern = qgemm_ragged_pp_kernel<QT, OUT, EPI>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  kern<<<dim3(ragged_grid(M, N, rg.G, 256, 256)), 512, smem, st>>>(
      static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, rg, static_cast<int>(M),
      static_cast<int>(N), static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo);
  return check_launch("ragged qgemm (ping-pong)");
}
// The epilogue's rounding flags at compile time when every step rounds to bf16 (bf16 scales, bf16 result) or none
// does (f32 throughout), as the dense dispatch does; at run time otherwise.
template <int QT, int OUT>
int launch_ragged_pp(const void* a, int64_t lda, const void* b, int64_t ldb, const Ragged& rg, int64_t M, int64_t N,
                     int64_t K, const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  const bool all = ep.r0 && ep.r1 && ep.r2, none = !ep.r0 && !ep.r1 && !ep.r2;
  if (OUT == QWIX_BF16 && all) return launch_ragged_pp_epi<QT, OUT, 1>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
  if (OUT == QWIX_F32 && none) return launch_ragged_pp_epi<QT, OUT, 0>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
  return launch_ragged_pp_epi<QT, OUT, 2>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
}

template <int QT, int BM, int BN, int BK>
__global__ void __launch_bounds__(256)
    qgemm_ragged_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                        Ragged rg, int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  int g, m0, m_lim, n0;
  const int kind = ragged_tile<BM, BN>(rg, M, N, &g, &m0, &m_lim, &n0);
  if (kind == 0) return;
  if (kind == 2) {
    if (ep.out_dtype == QWIX_BF16) zero_tile<BM, BN, uint16_t>(out, ldo, m0, m_lim, n0, N, 256);
    else zero_tile<BM, BN, uint32_t>(out, ldo, m0, m_lim, n0, N, 256);
    return;
  }
  const Epilogue e = group_epilogue(ep, rg, g);
  qgemm_tile<QT, BM, BN, BK>(A, lda, B + g * rg.b_group_stride, ldb, m0, n0, m_lim, N, K, e, out, ldo);
}

template <int QT, int BM, int BN, int WGM, int WGN, int OUT>
int launch_ragged_dma(const void* a, int64_t lda, const void* b, int64_t ldb, const Ragged& rg, int64_t M, int64_t N,
                      int64_t K, const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  constexpr size_t smem = 2 * (BM + BN) * 128;
  auto kern = qgemm_ragged_dma_kernel<QT, BM, BN, WGM, WGN, OUT>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  kern<<<dim3(ragged_grid(M, N, rg.G, BM, BN)), WGM * WGN * 64, smem, st>>>(
      static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, rg, static_cast<int>(M),
      static_cast<int>(N), static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo);
  return check_launch("ragged qgemm (dma)");
}

// The one-tile-row body (deep prefetch of the weights into registers) under the ragged grid, for groups of
// a few dozen rows: tiles of 64 rows x 128 columns waste fewer rows at the ragged end of a group than 128-row
// tiles do, and such groups are bound by the streaming of their weight panels.
template <int QT, int OUT, int TM, int DEPTH, int NW>
__global__ void __launch_bounds__(64 * NW)
    qgemm_ragged_mid_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                            Ragged rg, int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  constexpr int BM = 32 * TM, BN = 32 * NW;
  int g, m0, m_lim, n0;
  const int kind = ragged_tile<BM, BN>(rg, M, N, &g, &m0, &m_lim, &n0);
  if (kind == 0) return;
  using OutT = typename std::conditional<OUT == QWIX_BF16, uint16_t, uint32_t>::type;
  if (kind == 2) {
    zero_tile<BM, BN, OutT>(out, ldo, m0, m_lim, n0, N, 64 * NW);
    return;
  }
  const Epilogue e = group_epilogue(ep, rg, g);
  const int kshift = static_cast<int>((blockIdx.x * 5u) % static_cast<unsigned>(K / 128));
  qgemm_mid_tile<QT, OUT, 2, TM, DEPTH, NW>(A, lda, B + g * rg.b_group_stride, ldb, m0, n0, m_lim, N, K, e, out, ldo,
                                            kshift);
}

template <int QT, int OUT>
int launch_ragged_mid(const void* a, int64_t lda, const void* b, int64_t ldb, const Ragged& rg, int64_t M, int64_t N,
                      int64_t K, const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  constexpr int TM = 2, NW = 4, kDepth = 8;
  constexpr size_t smem = kDepth * 32 * TM * 128;  // 64 KB of activation stages (the epilogue needs 18 KB)
  auto kern = qgemm_ragged_mid_kernel<QT, OUT, TM, kDepth, NW>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  kern<<<dim3(ragged_grid(M, N, rg.G, 32 * TM, 32 * NW)), 64 * NW, smem, st>>>(
      static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, rg, static_cast<int>(M),
      static_cast<int>(N), static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo);
  return check_launch("ragged qgemm (one tile row per 64 rows)");
}

template <int QT, int BM, int BN, int WGM, int WGN>
int dispatch_ragged_dma(const void* a, int64_t lda, const void* b, int64_t ldb, const Ragged& rg, int64_t M, int64_t N,
                        int64_t K, const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  if (ep.out_dtype == QWIX_I32) {
    if constexpr (QT == QWIX_INT8) return launch_ragged_dma<QT, BM, BN, WGM, WGN, QWIX_I32>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
    return fail(QWIX_ERR_INVALID_ARGUMENT, "int32 output needs int8 operands");
  }
  if (ep.out_dtype == QWIX_BF16) return launch_ragged_dma<QT, BM, BN, WGM, WGN, QWIX_BF16>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
  return launch_ragged_dma<QT, BM, BN, WGM, WGN, QWIX_F32>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
}

template <int QT>
int launch_ragged(const void* a, int64_t lda, const void* b, int64_t ldb, const Ragged& rg, int64_t M, int64_t N,
                  int64_t K, const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  constexpr int BM = 128, BN = 128, BK = 128;
  constexpr size_t smem = 2 * (BM + BN) * (BK + kPad);
  auto kern = qgemm_ragged_kernel<QT, BM, BN, BK>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  kern<<<dim3(ragged_grid(M, N, rg.G, BM, BN)), 256, smem, st>>>(
      static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, rg, static_cast<int>(M),
      static_cast<int>(N), static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo);
  return check_launch("ragged qgemm");
}

// ------------------------------------------------------------------------------------------------
// Batched GEMM: blockIdx.y selects one of `batch` independent problems of the same shape (the batch
// axes of dot_general); operands, scale vectors and outputs of consecutive problems are a fixed
// stride apart.  Same tile bodies as the dense kernels.
struct Batched {
  int64_t a_stride, b_stride;    // bytes
  int64_t sa_stride, sb_stride;  // elements (0: the vector is shared by all problems)
  int64_t out_stride;            // elements
};

__device__ __forceinline__ Epilogue batch_epilogue(const Epilogue& ep, const Batched& bs, int z) {
  Epilogue e = ep;
  if (ep.sa != nullptr)
    e.sa = static_cast<const uint8_t*>(ep.sa) + z * bs.sa_stride * (ep.sa_dtype == QWIX_BF16 ? 2 : 4);
  if (ep.sb != nullptr)
    e.sb = static_cast<const uint8_t*>(ep.sb) + z * bs.sb_stride * (ep.sb_dtype == QWIX_BF16 ? 2 : 4);
  return e;
}

template <int QT, int BM, int BN, int WGM, int WGN, int OUT>
__global__ void __launch_bounds__(WGM * WGN * 64)
    qgemm_batched_dma_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                             Batched bs, int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  const int z = blockIdx.y;
  int tile_m, tile_n;
  tile_coords((M + BM - 1) / BM, (N + BN - 1) / BN, &tile_m, &tile_n);
  const Epilogue e = batch_epilogue(ep, bs, z);
  constexpr int ES = OUT == QWIX_BF16 ? 2 : 4;
  qgemm_dma_tile<QT, BM, BN, WGM, WGN, OUT, (OUT == QWIX_I32 ? 0 : 2)>(
      A + z * bs.a_stride, lda, B + z * bs.b_stride, ldb, tile_m * BM, tile_n * BN, M, N, K, e,
      out + z * bs.out_stride * ES, ldo);
}

template <int QT, int BM, int BN, int BK>
__global__ void __launch_bounds__(256)
    qgemm_batched_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                         Batched bs, int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  const int z = blockIdx.y;
  int tile_m, tile_n;
  tile_coords((M + BM - 1) / BM, (N + BN - 1) / BN, &tile_m, &tile_n);
  const Epilogue e = batch_epilogue(ep, bs, z);
  const int es = ep.out_dtype == QWIX_BF16 ? 2 : 4;
  qgemm_tile<QT, BM, BN, BK>(A + z * bs.a_stride, lda, B + z * bs.b_stride, ldb, tile_m * BM, tile_n * BN, M, N, K, e,
                             out + z * bs.out_stride * es, ldo);
}

template <int QT, int OUT>
int launch_batched_dma(const void* a, int64_t lda, const void* b, int64_t ldb, const Batched& bs, int64_t batch,
                       int64_t M, int64_t N, int64_t K, const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  constexpr int BM = 128, BN = 128;
  constexpr size_t kStage = (BM + BN) * 128;
  constexpr size_t kStaging = 4 * 32 * (64 * (OUT == QWIX_BF16 ? 2 : 4) + 16);  // epilogue: 4 wavefronts x 32 padded rows
  // A single slab (K = 128, e.g. the head dimension of attention scores) never touches the second stage:
  // half the LDS lets more workgroups share a CU, which is what hides the latency of such short tiles.
  const size_t smem = K == 128 ? (kStage > kStaging ? kStage : kStaging) : 2 * kStage;
  auto kern = qgemm_batched_dma_kernel<QT, BM, BN, 2, 2, OUT>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  kern<<<dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(batch)), 256, smem, st>>>(
      static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, bs, static_cast<int>(M),
      static_cast<int>(N), static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo);
  return check_launch("batched qgemm (dma)");
}

template <int QT>
int launch_batched(const void* a, int64_t lda, const void* b, int64_t ldb, const Batched& bs, int64_t batch,
                   int64_t M, int64_t N, int64_t K, const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  if (K % 128 == 0) {
    if (ep.out_dtype == QWIX_I32) {
      if constexpr (QT == QWIX_INT8) return launch_batched_dma<QT, QWIX_I32>(a, lda, b, ldb, bs, batch, M, N, K, ep, out, ldo, st);
      return fail(QWIX_ERR_INVALID_ARGUMENT, "int32 output needs int8 operands");
    }
    if (ep.out_dtype == QWIX_BF16) return launch_batched_dma<QT, QWIX_BF16>(a, lda, b, ldb, bs, batch, M, N, K, ep, out, ldo, st);
    return launch_batched_dma<QT, QWIX_F32>(a, lda, b, ldb, bs, batch, M, N, K, ep, out, ldo, st);
  }
  constexpr int BM = 128, BN = 128, BK = 128;
  constexpr size_t smem = 2 * (BM + BN) * (BK + kPad);
  auto kern = qgemm_batched_kernel<QT, BM, BN, BK>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  kern<<<dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(batch)), 256, smem, st>>>(
      static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, bs, static_cast<int>(M),
      static_cast<int>(N), static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo);
  return check_launch("batched qgemm");
}

}  // namespace
}  // namespace qwix

using namespace qwix;

namespace qwix {
namespace {

// ------------------------------------------------------------------------------------------------
// Skinny GEMM (decode: a handful of tokens against a whole weight matrix).  The 128 x 128 tiles of
// the kernels above would leave most CUs idle and most MFMA rows empty; here the weight matrix is
// streamed exactly once: a workgroup owns NT tiles of 16 output columns, its 16 wavefronts split
// K, each with two 128-byte blocks of loads in flight, and the int32 (or f32) partial tiles meet
// in LDS.  int8: v_mfma_i32_16x16x64_i8, a lane holds 32 consecutive k of one row (two MFMAs);
// e4m3: one v_mfma_f32_16x16x128_f8f6f4.  The int32 sum does not depend on the split, so results
// are bit-identical to the tiled kernels'; the epilogue is the same rounding chain.
typedef int v8i_s __attribute__((ext_vector_type(8)));
typedef float v4f_s __attribute__((ext_vector_type(4)));
constexpr int kSkinnyWaves = 16;

// One 16-row block of the weight-streaming GEMM: rows row0 .. row0 + 15 (below M) against columns n_base ..
// n_base + 16 * NT - 1, by a workgroup of WAVES wavefronts that split K.
template <int QT, int NT, int WAVES = kSkinnyWaves>
__device__ __forceinline__ void skinny_block(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B,
                                             int64_t ldb, int row0, int M, int n_base, int N, int K, const Epilogue& ep,
                                             uint8_t* __restrict__ out, int64_t ldo) {
  constexpr bool IS_INT = (QT == QWIX_INT8);
  using AccT = typename std::conditional<IS_INT, v4i, v4f_s>::type;
  __shared__ AccT red[WAVES][NT][64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int nblk = K / 128;
  const int per_wave = (nblk + WAVES - 1) / WAVES;
  // Which slice of K a wavefront takes rotates with the workgroup: in step, all workgroups would ask the same few
  // memory channels for the same K offset of their rows at the same time (4096 x 14336 int8, 16 rows: 14.5 -> 13.9 us).
  const int slice = (wave + static_cast<int>(blockIdx.x)) % WAVES;
  const int kb0 = min(nblk, slice * per_wave), kb1 = min(nblk, kb0 + per_wave);

  // wave-uniform bases + fixed 32-bit lane offsets; rows of A past M and columns past N are clamped
  const uint8_t* a_base = A + static_cast<int64_t>(row0) * lda;
  const uint8_t* b_base = B + static_cast<int64_t>(n_base) * ldb;
  const uint32_t a_off = static_cast<uint32_t>(min(col, M - 1 - row0)) * static_cast<uint32_t>(lda) + kq * 32;
  uint32_t b_off[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
    b_off[t] = static_cast<uint32_t>(min(t * 16 + col, N - 1 - n_base)) * static_cast<uint32_t>(ldb) + kq * 32;

  AccT acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[t][r] = 0;

  struct Blk {
    v4i x[2];
    v4i w[NT][2];
  };
  auto load_blk = [&](int kb, Blk* b) {
    const uint8_t* ap = a_base + kb * 128 + a_off;
    b->x[0] = *reinterpret_cast<const v4i*>(ap);
    b->x[1] = *reinterpret_cast<const v4i*>(ap + 16);
    const uint8_t* bp = b_base + kb * 128;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      b->w[t][0] = *reinterpret_cast<const v4i*>(bp + b_off[t]);
      b->w[t][1] = *reinterpret_cast<const v4i*>(bp + b_off[t] + 16);
    }
  };
  auto compute_blk = [&](const Blk& b) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if constexpr (IS_INT) {
        acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b.x[0], b.w[t][0], acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b.x[1], b.w[t][1], acc[t], 0, 0, 0);
      } else {
        const v8i_s xa = {b.x[0][0], b.x[0][1], b.x[0][2], b.x[0][3], b.x[1][0], b.x[1][1], b.x[1][2], b.x[1][3]};
        const v8i_s wb = {b.w[t][0][0], b.w[t][0][1], b.w[t][0][2], b.w[t][0][3],
                          b.w[t][1][0], b.w[t][1][1], b.w[t][1][2], b.w[t][1][3]};
        acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(xa, wb, acc[t], 0, 0, 0, 0, 0, 0);
      }
    }
  };
  for (int kb = kb0; kb < kb1; kb += 2) {
    Blk b0, b1;
    const bool two = kb + 1 < kb1;
    load_blk(kb, &b0);
    if (two) load_blk(kb + 1, &b1);
    compute_blk(b0);
    if (two) compute_blk(b1);
  }

#pragma unroll
  for (int t = 0; t < NT; ++t) red[wave][t][lane] = acc[t];
  __syncthreads();
  // result lane layout: column n = lane % 16, row m = 4 * (lane / 16) + r
  const bool r0 = ep.r0 != 0, r1 = ep.r1 != 0, r2 = ep.r2 != 0;
  for (int idx = tid; idx < NT * 256; idx += WAVES * 64) {
    const int t = idx >> 8, r = (idx >> 6) & 3, l = idx & 63;
    const int m = row0 + 4 * (l >> 4) + r, n = n_base + t * 16 + (l & 15);
    if (m >= M || n >= N) continue;
    float v;
    if constexpr (IS_INT) {
      int a = 0;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) a += red[w][t][l][r];
      if (ep.out_dtype == QWIX_I32) {
        reinterpret_cast<int*>(out)[static_cast<int64_t>(m) * ldo + n] = a;
        continue;
      }
      if (ep.zu != nullptr) a -= ep.zu[m] * ep.zv[n];
      v = static_cast<float>(a);
    } else {
      v = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) v += red[w][t][l][r];
    }
    if (r0) v = round_bf16(v);
    if (ep.sa != nullptr) v *= load_scale(ep.sa, ep.sa_dtype, m);
    if (r1) v = round_bf16(v);
    if (ep.sb != nullptr) v *= load_scale(ep.sb, ep.sb_dtype, n);
    if (r2) v = round_bf16(v);
    if (ep.out_dtype == QWIX_BF16)
      reinterpret_cast<uint16_t*>(out)[static_cast<int64_t>(m) * ldo + n] = f32_to_bf16_bits(v);
    else
      reinterpret_cast<float*>(out)[static_cast<int64_t>(m) * ldo + n] = v;
  }
}

template <int QT, int NT>
__global__ void __launch_bounds__(kSkinnyWaves * 64)
    qgemm_skinny_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb, int M,
                        int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  skinny_block<QT, NT>(A, lda, B, ldb, blockIdx.y * 16, M, blockIdx.x * (16 * NT), N, K, ep, out, ldo);
}

// The same block with smaller workgroups, for weights of hundreds of megabytes (an output projection over a
// large vocabulary): once there are several rounds of workgroups per CU, small ones overlap each other's load,
// reduce and store phases (one row, K 4096, N 131072: 4.9 -> 6.0 TB/s with 4 wavefronts x 16 columns).  Taken for
// up to 4 rows only: with 16 rows the narrow column groups re-read the activation fragment too often (8 wavefronts
// x 32 columns: between -8 % and +10 % depending on K), and at decode sizes of tens of megabytes, where all
// workgroups fit the chip at once, the 16-wavefront shape stays ahead (58.7 MB: 4.1 TB/s against 3.2 - 3.9).
template <int QT, int NT, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    qgemm_skinny_small_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                              int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  skinny_block<QT, NT, WAVES>(A, lda, B, ldb, blockIdx.y * 16, M, blockIdx.x * (16 * NT), N, K, ep, out, ldo);
}

template <int QT>
int launch_skinny(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
                  const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  const unsigned gy = static_cast<unsigned>((M + 15) / 16);
  if (N * K >= (int64_t{192} << 20) && M <= 4) {
#define QWIX_SKINNY_SMALL(NTT, WVV)                                                                                \
  qgemm_skinny_small_kernel<QT, NTT, WVV><<<dim3(static_cast<unsigned>((N + 16 * NTT - 1) / (16 * NTT)), gy), WVV * 64, \
                                            0, st>>>(static_cast<const uint8_t*>(a), lda,                             \
                                                     static_cast<const uint8_t*>(b), ldb, static_cast<int>(M),        \
                                                     static_cast<int>(N), static_cast<int>(K), ep,                     \
                                                     static_cast<uint8_t*>(out), ldo)
    QWIX_SKINNY_SMALL(1, 4);
#undef QWIX_SKINNY_SMALL
    return check_launch("qgemm (skinny)");
  }
#define QWIX_SKINNY(NTT)                                                                                         \
  qgemm_skinny_kernel<QT, NTT><<<dim3(static_cast<unsigned>((N + 16 * NTT - 1) / (16 * NTT)), gy), kSkinnyWaves * 64, \
                                 0, st>>>(static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, \
                                          static_cast<int>(M), static_cast<int>(N), static_cast<int>(K), ep,       \
                                          static_cast<uint8_t*>(out), ldo)
  // wider column groups reuse the activation fragments; narrower ones keep every CU busy
  if (N >= 192 * 64)
    QWIX_SKINNY(4);
  else if (N >= 192 * 32)
    QWIX_SKINNY(2);
  else
    QWIX_SKINNY(1);
#undef QWIX_SKINNY
  return check_launch("qgemm (skinny)");
}

// Ragged variant for a few rows per group (mixture-of-experts decode): blockIdx.y is the group, whose rows are
// found from the group sizes by every wavefront for itself; the workgroup streams that group's weight columns
// once per 16 rows.  blockIdx.y == G clears the rows that belong to no group.
template <int QT, int NT, int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
    qgemm_ragged_skinny_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb,
                               Ragged rg, int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  const int g = blockIdx.y, lane = threadIdx.x & 63;
  const int n_base = blockIdx.x * (16 * NT);
  long long before = 0;
  for (int i = lane; i < g; i += 64) before += max(rg.group_sizes[i], 0);
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) before += __shfl_xor(before, m, 64);
  const int start = static_cast<int>(min(before, static_cast<long long>(M)));
  if (g == rg.G) {  // rows past the last group: zeros
    const int cols = min(16 * NT, N - n_base);
    for (int idx = threadIdx.x; idx < (M - start) * cols; idx += WAVES * 64) {
      const int64_t at = static_cast<int64_t>(start + idx / cols) * ldo + n_base + idx % cols;
      if (ep.out_dtype == QWIX_BF16) reinterpret_cast<uint16_t*>(out)[at] = 0;
      else reinterpret_cast<uint32_t*>(out)[at] = 0;
    }
    return;
  }
  const int end = static_cast<int>(min(before + max(rg.group_sizes[g], 0), static_cast<long long>(M)));
  const Epilogue e = group_epilogue(ep, rg, g);
  const uint8_t* bg = B + g * rg.b_group_stride;
  for (int row0 = start; row0 < end; row0 += 16) {  // the trip count is the same for the whole workgroup
    skinny_block<QT, NT, WAVES>(A, lda, bg, ldb, row0, end, n_base, N, K, e, out, ldo);
    __syncthreads();  // the partial sums in LDS are reused by the next pass
  }
}

template <int QT>
int launch_ragged_skinny(const void* a, int64_t lda, const void* b, int64_t ldb, const Ragged& rg, int64_t M, int64_t N,
                         int64_t K, const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  const unsigned gy = static_cast<unsigned>(rg.G + 1);
  // Small workgroups: 4 wavefronts, and the fewer rows a group has, the narrower the column group (the
  // activation fragment is re-read per column group, which costs as much as the weights once a group has 16
  // rows).  Measured at 64 groups x 4 rows, K 2048, N 4096, in GB/s of weights: 16 wavefronts x 64 columns
  // 4260, 8 x 32 4700, 4 x 64 4680, 4 x 32 4810, 4 x 16 5120, 2 x 16 5060, 1 x 16 4980.
  constexpr int kWaves = 4;
#define QWIX_RSKINNY(NTT)                                                                                          \
  qgemm_ragged_skinny_kernel<QT, NTT, kWaves><<<dim3(static_cast<unsigned>((N + 16 * NTT - 1) / (16 * NTT)), gy), \
                                                kWaves * 64, 0, st>>>(static_cast<const uint8_t*>(a), lda,          \
                                                                      static_cast<const uint8_t*>(b), ldb, rg,        \
                                                                      static_cast<int>(M), static_cast<int>(N),      \
                                                                      static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo)
  if (M <= 4 * static_cast<int64_t>(rg.G))
    QWIX_RSKINNY(1);
  else if (M <= 8 * static_cast<int64_t>(rg.G))
    QWIX_RSKINNY(2);
  else
    QWIX_RSKINNY(4);
#undef QWIX_RSKINNY
  return check_launch("ragged qgemm (skinny)");
}

// ------------------------------------------------------------------------------------------------
// Decode with the activation quantization folded in (int8, M <= 32 per call): the float activations are
// what the kernel reads.  Every workgroup keeps its 16 rows in registers (the 16 wavefronts split K as in
// the skinny kernel, a lane holds the 32 consecutive k of one row that its MFMA operand needs), finds the
// rows' absmax (lanes of a row by shuffle, wavefronts through LDS; a maximum does not depend on the order),
// derives the scale exactly as the stand-alone quantize kernel does, quantizes its registers and goes on
// as the skinny kernel.  The quantized values and scales are bit-identical to quantize-then-multiply; they
// are recomputed by every workgroup from L2 (16 x K activations against 16 * NT x K weights), which is
// cheaper than a kernel launch of its own as long as K is short.  KB: 128-wide K blocks per wavefront
// (K <= 2048 * KB; only KB = 1 is instantiated).
template <typename D, int NT, int KB>
__global__ void __launch_bounds__(kSkinnyWaves * 64)
    qgemm_skinny_fused_kernel(const uint8_t* __restrict__ X, int64_t ldx, const uint8_t* __restrict__ B, int64_t ldb,
                              int M, int N, int K, Epilogue ep, uint8_t* __restrict__ out, int64_t ldo) {
  constexpr int ES = D::kTag == QWIX_BF16 ? 2 : 4;   // bytes per activation
  constexpr int XV = 32 * ES / 16;                    // 16-byte loads per lane and K block (32 elements)
  __shared__ v4i red[kSkinnyWaves][NT][64];
  __shared__ float rowmax[kSkinnyWaves][16];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 15, kq = lane >> 4;
  const int n_base = blockIdx.x * (16 * NT), row0 = blockIdx.y * 16;
  const int nblk = K / 128;
  const int kb0 = wave * KB, kb1 = min(nblk, kb0 + KB);  // nblk <= 16 * KB

  const uint8_t* x_base = X + static_cast<int64_t>(row0) * ldx * ES;
  const uint8_t* b_base = B + static_cast<int64_t>(n_base) * ldb;
  const uint32_t x_off = static_cast<uint32_t>(min(col, M - 1 - row0)) * static_cast<uint32_t>(ldx * ES) + kq * 32 * ES;
  uint32_t b_off[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
    b_off[t] = static_cast<uint32_t>(min(t * 16 + col, N - 1 - n_base)) * static_cast<uint32_t>(ldb) + kq * 32;

  // ---- this lane's activations and weights for all of its K blocks
  uint4 xr[KB][XV];
  v4i w[KB][NT][2];
#pragma unroll
  for (int j = 0; j < KB; ++j) {
    const int kb = kb0 + j;
#pragma unroll
    for (int v = 0; v < XV; ++v) xr[j][v] = make_uint4(0, 0, 0, 0);
    if (kb < kb1) {
      const uint8_t* xp = x_base + static_cast<int64_t>(kb) * 128 * ES + x_off;
#pragma unroll
      for (int v = 0; v < XV; ++v) xr[j][v] = *reinterpret_cast<const uint4*>(xp + 16 * v);
      const uint8_t* bp = b_base + kb * 128;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        w[j][t][0] = *reinterpret_cast<const v4i*>(bp + b_off[t]);
        w[j][t][1] = *reinterpret_cast<const v4i*>(bp + b_off[t] + 16);
      }
    }
  }

  // ---- absmax of the 16 rows
  float mx = 0.f;
#pragma unroll
  for (int j = 0; j < KB; ++j)
#pragma unroll
    for (int v = 0; v < XV; ++v) {
      float f[D::kVec];
      unpack16<D>(xr[j][v], f);
#pragma unroll
      for (int e = 0; e < D::kVec; ++e) mx = fmaxf(mx, __builtin_fabsf(f[e]));
    }
  mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  if (lane < 16) rowmax[wave][lane] = mx;
  __syncthreads();
  mx = rowmax[0][col];
#pragma unroll
  for (int wv = 1; wv < kSkinnyWaves; ++wv) mx = fmaxf(mx, rowmax[wv][col]);
  const float s = sym_scale<D, QWIX_INT8>(mx);  // the scale of row `col`, as the quantize kernel derives it
  const Divider<D, false, false> div(s);

  // ---- quantize the registers, multiply
  v4i acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[t][e] = 0;
#pragma unroll
  for (int j = 0; j < KB; ++j) {
    if (kb0 + j < kb1) {
      uint32_t qw[8];  // 32 int8 values, 4 per word, in k order
      constexpr int PER = D::kVec / 4;  // words a 16-byte vector turns into
#pragma unroll
      for (int v = 0; v < XV; ++v) {
        float f[D::kVec];
        unpack16<D>(xr[j][v], f);
#pragma unroll
        for (int h = 0; h < PER; ++h)
          qw[v * PER + h] = pack4_low_bytes(rne_bits_clamped(div(f[4 * h]), -128.f, 127.f),
                                            rne_bits_clamped(div(f[4 * h + 1]), -128.f, 127.f),
                                            rne_bits_clamped(div(f[4 * h + 2]), -128.f, 127.f),
                                            rne_bits_clamped(div(f[4 * h + 3]), -128.f, 127.f));
      }
      const v4i x0 = {static_cast<int>(qw[0]), static_cast<int>(qw[1]), static_cast<int>(qw[2]), static_cast<int>(qw[3])};
      const v4i x1 = {static_cast<int>(qw[4]), static_cast<int>(qw[5]), static_cast<int>(qw[6]), static_cast<int>(qw[7])};
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, w[j][t][0], acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x1, w[j][t][1], acc[t], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int t = 0; t < NT; ++t) red[wave][t][lane] = acc[t];
  // the row scales in the result's lane layout: row m = 4 * (lane / 16) + e of the block
  __shared__ float srow[16];
  if (wave == 0 && lane < 16) srow[lane] = s;
  __syncthreads();
  const bool r0 = ep.r0 != 0, r1 = ep.r1 != 0, r2 = ep.r2 != 0;
  for (int idx = tid; idx < NT * 256; idx += kSkinnyWaves * 64) {
    const int t = idx >> 8, e = (idx >> 6) & 3, l = idx & 63;
    const int mr = 4 * (l >> 4) + e;
    const int m = row0 + mr, n = n_base + t * 16 + (l & 15);
    if (m >= M || n >= N) continue;
    int a = 0;
#pragma unroll
    for (int wv = 0; wv < kSkinnyWaves; ++wv) a += red[wv][t][l][e];
    float v = static_cast<float>(a);
    if (r0) v = round_bf16(v);
    v *= srow[mr];
    if (r1) v = round_bf16(v);
    if (ep.sb != nullptr) v *= load_scale(ep.sb, ep.sb_dtype, n);
    if (r2) v = round_bf16(v);
    if (ep.out_dtype == QWIX_BF16)
      reinterpret_cast<uint16_t*>(out)[static_cast<int64_t>(m) * ldo + n] = f32_to_bf16_bits(v);
    else
      reinterpret_cast<float*>(out)[static_cast<int64_t>(m) * ldo + n] = v;
  }
}

template <typename D, int KB>
int launch_skinny_fused(const void* x, int64_t ldx, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
                        const Epilogue& ep, void* out, int64_t ldo, hipStream_t st) {
  const unsigned gy = static_cast<unsigned>((M + 15) / 16);
#define QWIX_FUSED(NTT)                                                                                              \
  qgemm_skinny_fused_kernel<D, NTT, KB><<<dim3(static_cast<unsigned>((N + 16 * NTT - 1) / (16 * NTT)), gy),         \
                                          kSkinnyWaves * 64, 0, st>>>(static_cast<const uint8_t*>(x), ldx,           \
                                                                      static_cast<const uint8_t*>(b), ldb,           \
                                                                      static_cast<int>(M), static_cast<int>(N),      \
                                                                      static_cast<int>(K), ep, static_cast<uint8_t*>(out), ldo)
  if (N >= 192 * 32)
    QWIX_FUSED(2);
  else
    QWIX_FUSED(1);
#undef QWIX_FUSED
  return check_launch("qgemm (skinny, fused activation quantize)");
}

// out[r] = sum_k q[r, k] over int8 rows: one wavefront per row, 16 bytes per lane and trip.
__global__ void __launch_bounds__(256) ksum_i8_kernel(const int8_t* __restrict__ q, int64_t ld, int rows, int K,
                                                      int32_t* __restrict__ out) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= rows) return;
  const int8_t* p = q + static_cast<int64_t>(row) * ld;
  int s = 0;
  for (int k = lane * 16; k < K; k += 64 * 16) {  // K % 16 == 0
    const int4 w = *reinterpret_cast<const int4*>(p + k);
    const int u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) s += (u[e] << 24 >> 24) + (u[e] << 16 >> 24) + (u[e] << 8 >> 24) + (u[e] >> 24);
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) s += __shfl_xor(s, m, 64);
  if (lane == 0) out[row] = s;
}

// ------------------------------------------------------------------------------------------------
// bf16 activations x int4 weights with K-group scales, beyond the decode batch (prefill): the weights are dequantized
// inside the workgroup instead of in a pass of their own.  A 256 x 128 tile on 8 wavefronts (64 x 64 each),
// v_mfma_f32_32x32x16_bf16, K in slabs of 64 elements (128 bytes of a row of activations), 160 KB of LDS.
//   The packed weights come in whole 128-byte lines: one direct-to-LDS load per 8 rows fetches 256 elements of
// K per row, four slabs' worth (a superslab), into one of two raw buffers; the next superslab and its four scales
// (untracked loads) are requested in the first slab of this one.  While slab kt is multiplied, slab kt + 1 of the
// weight tile is converted: every thread takes 16 nibbles of one row out of the raw buffer, turns them into
// bf16(q * scale) -- the value the reference's dequantize gives (qarray.py:692-708, computed in f32 and rounded to
// bf16: exact for bf16 scales, one more rounding for f32 scales, as qwix_hip_dequantize_rm does) -- and writes them
// where the dense bf16 kernel expects the weight slab (same XOR swizzle), a quarter of the work in front of each of
// the slab's four k-steps.  The activations go through three LDS stages by direct-to-LDS loads requested two slabs
// ahead (four stages, three slabs in the 128-row tile).  One barrier per slab; the wait in front of it is counted
// (vmcnt), so that the requests of the slab that ends (in the 128-row tile: and of the one before) stay in flight: a
// full wait there costs a memory round trip per slab (87 us instead of 65 at 512 x 14336 x 4096).
//   LDS is read and written through ext_vector types only (v4i, qwix_v2i).  Through HIP's struct vectors (uint2,
// uint4) the compiler cannot tell the access from the destinations of the direct-to-LDS loads in flight and puts
// an s_waitcnt vmcnt(0) in front of it, which turns every counted wait into a full one.
// Results are bit-identical to qwix_hip_dequantize_rm + qwix_hip_gemm_bf16: the same bf16 weights, the same MFMA,
// K walked in the same order.
// BN = 64 (tiles of 256 x 64, wavefronts of 64 x 32, 128 KB of LDS) is for calls whose 128-column tiles would leave
// more than half of the CUs without a workgroup: a workgroup's time is mostly its MFMAs and the conversion, which
// both halve, while its activation traffic stays.
// BITS = 8: int8 weights.  A row's 128-byte line would hold only two slabs, too few to request a buffer ahead, so
// they come as 64-byte pieces, one slab per request (16 rows per load instruction), into a ring of four buffers:
// slab kt + 3 is requested in slab kt, behind the activations of slab kt + 2 (128-row tile: kt + 4 behind kt + 3, into
// the buffer that was read in slab kt - 1).  With 64-column tiles on eight requesting wavefronts the upper half of
// a load instruction's lanes repeats the lower half's rows (every wavefront issues one load per slab, so that all
// count their requests alike); the repeated rows land in padding.  A byte b holds q = (b ^ 0x80) - 128 and
// q * scale = fma(b ^ 0x80, scale, -128 scale), exact as for the nibbles.  BITS = 9 stands for e4m3 weights: the same
// bytes, converted by v_cvt_pk_f32_fp8 (two per instruction) and multiplied by the scale.
// ZP: asymmetric weights, (q - zero_point) * scale with one int8 zero point per scale.  It is requested with the scale
// and joins the offset of the storage format: bf16 scales fma(u, scale, -(offset + zp) scale), every term still exact
// in f32 (nine bits times eight); f32 scales float(u - offset - zp) * scale, the integer difference first, because
// (offset + zp) * scale would no longer be exact.
// BM = 128 (tiles of 128 x 64) is for calls of at most 128 rows: half the MFMAs and half the activation loads per
// workgroup of the 256-row tile, whose upper half would multiply padding.  Its eight wavefronts split the work: four
// multiply (64 x 32 each) and load nothing, four only request the operands, three slabs ahead, and wait for them; a
// wavefront issues in order, so one that requests and multiplies stands at a load instruction while the memory
// pipeline is full and its SIMD's matrix core idles (requests, conversion and MFMAs added up to the run time: 10 +
// 4 + 7 us on top of 9.4 us of skeleton at 128 x 4096 x 4096, int8; 34 -> 29 us at 128 x 14336 x 4096).  The
// requesting wavefronts also dequantize int4 weights (35.6 -> 29.3 us against 32.6 with the conversion between the
// MFMAs); bytes convert faster between the MFMAs (28.5 against 32.8 us).  The requesting wavefronts end after the last
// slab: a wavefront that has ended no longer counts at the workgroup's barriers.
//   In the 256-row tiles every wavefront requests and multiplies; there the four activation loads of a slab are issued
// one per k-step instead of together (512 x 4096 x 4096: int4 47 -> 42 us, int8 50 -> 45 us).
template <int OUT, bool SBF, int BM, int BN, int BITS, bool ZP>
__global__ void __launch_bounds__(512)
    wgemm_wq_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ Q, int64_t ldq,
                    const void* __restrict__ S, const int8_t* __restrict__ Z, int M, int N, int K, int group,
                    uint8_t* __restrict__ out, int64_t ldo, int ksplit) {
  static_assert((BM == 256 && (BN == 128 || BN == 64)) || (BM == 128 && BN == 64), "tiles of 256 x 128, 256 x 64, 128 x 64");
  if (ksplit > 0) {
    // K split over blockIdx.y: this workgroup contracts elements [y ksplit, (y + 1) ksplit) -- ksplit a multiple of 256,
    // and a multiple or a divisor of the group, so that a range starts a group or lies inside one -- and writes its tile
    // of the y-th M x N partial (the host passes OUT = f32 and ldo = N); every operand pointer moves to the range's
    // first element (the scales': to the group that holds it).
    const int k0 = static_cast<int>(blockIdx.y) * ksplit;
    A += static_cast<int64_t>(k0) * 2;
    Q += (BITS >= 8) ? k0 : k0 / 2;
    S = static_cast<const char*>(S) + static_cast<int64_t>(k0 / group) * N * (SBF ? 2 : 4);
    if constexpr (ZP) Z += static_cast<int64_t>(k0 / group) * N;
    out += static_cast<int64_t>(blockIdx.y) * M * N * 4;
    K = ksplit;
  }
  constexpr int WGN = 2, WN = BN / WGN, TM = 2, TN = WN / 32, NWAVES = BM / 32, NTHREADS = NWAVES * 64;
  constexpr int BK = 128, NK = 4;  // bytes of an activation row per slab (64 elements); k-steps of 16 elements
  static_assert(BITS == 4 || BITS == 8 || BITS == 9, "int4, int8 or (9) e4m3 weights");
  constexpr bool W8 = BITS >= 8;   // one byte per weight
  constexpr bool F8 = BITS == 9;   // e4m3: the byte converts to f32 directly; no offset, no zero point
  static_assert(!(F8 && ZP), "float weights have no zero point");
  // raw weights: int4 two buffers of a superslab (BN x 128 bytes), int8 four of a slab (1 KB per wavefront)
  constexpr int A_STAGE = BM * BK, C_STAGE = BN * BK, R_STAGE = W8 ? NWAVES * 1024 : BN * 128;
  // slabs between the request of activations and their use; the 128-row tile has the LDS for one more
  constexpr int AL = BM == 128 ? 3 : 2, AST = AL + 1;
  static_assert(AL == 2 || AL == 3, "the last four slabs are the only special ones");
  constexpr int C_BASE = AST * A_STAGE, R_BASE = C_BASE + 2 * C_STAGE, LDS_BYTES = R_BASE + (W8 ? 4 : 2) * R_STAGE;  // <= 160 KB
  constexpr int RPW = BN / NWAVES;  // weight rows per wavefront: 16 or 8
  constexpr int NQ = W8 ? 1 : RPW / 8;  // direct-to-LDS loads of weights per wavefront and request
  constexpr int TPR = NTHREADS / BN;    // converter threads per weight row: 4 or 8
  constexpr int NPT = 64 / TPR;     // elements per thread and slab: 16 or 8
  constexpr int NCQ = NPT / 4;      // conversion steps of four elements: 4 or 2
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;
  // SPEC: as many wavefronts again that only request the operands (rows and weight rows of wavefront wave - NWAVES)
  constexpr bool SPEC = BM == 128;
  const bool loader = SPEC && wave >= NWAVES;
  // who dequantizes: the requesting wavefronts for int4 (measured 32.6 -> 30.2 us at 128 x 14336 x 4096), the multiplying
  // ones for bytes (30.4 against 32.8 us)
  constexpr bool LC = SPEC && !W8;
  const int ldw = SPEC ? (wave & (NWAVES - 1)) : wave;
  int tile_m, tile_n;
  tile_coords((M + BM - 1) / BM, (N + BN - 1) / BN, &tile_m, &tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  v16f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // ---- loaders: 8 rows x 128 bytes per instruction; the global 16-byte chunk that lands at position lane & 7
  const int lr = lane >> 3;
  uint32_t goffa[4], goffq[NQ];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = ldw * 32 + j * 8 + lr;
    goffa[j] = static_cast<uint32_t>(min(m0 + row, M - 1)) * static_cast<uint32_t>(lda) + (((lane & 7) ^ swz8(row)) << 4);
  }
#pragma unroll
  for (int j = 0; j < NQ; ++j) {
    if constexpr (W8) {  // 16 rows x 64 bytes per instruction (64-column tiles: 8 rows, twice)
      const int row = ldw * RPW + ((lane >> 2) & (RPW - 1));
      goffq[j] = static_cast<uint32_t>(min(n0 + row, N - 1)) * static_cast<uint32_t>(ldq) + ((lane & 3) << 4);
    } else {
      const int row = ldw * RPW + j * 8 + lr;
      goffq[j] = static_cast<uint32_t>(min(n0 + row, N - 1)) * static_cast<uint32_t>(ldq) + (((lane & 7) ^ swz8(row)) << 4);
    }
  }
  auto issue_a = [&](int kt, int stage) {  // 4 loads
    const uint8_t* gk = A + kt * BK;
    uint8_t* dst = smem + stage * A_STAGE + ldw * 32 * BK;
#pragma unroll
    for (int j = 0; j < 4; ++j) QWIX_GLDS16(gk + goffa[j], dst + j * 1024);
  };
  auto issue_raw = [&](int ss) {  // int4: superslab ss (elements 256 ss ..), NQ loads; int8: slab ss, one load
    if constexpr (W8) {
      QWIX_GLDS16(Q + ss * 64 + goffq[0], smem + R_BASE + (ss & 3) * R_STAGE + ldw * 1024);
    } else {
      const uint8_t* gq = Q + ss * 128;
      uint8_t* dst = smem + R_BASE + (ss & 1) * R_STAGE + ldw * RPW * 128;
#pragma unroll
      for (int j = 0; j < NQ; ++j) QWIX_GLDS16(gq + goffq[j], dst + j * 1024);
    }
  };

  // ---- converter: thread -> (weight row, NPT of the slab's 64 elements)
  const int ctid = tid & (NTHREADS - 1);
  const int crow = ctid / TPR, cpart = ctid % TPR;
  const char* const sptr = static_cast<const char*>(S) + static_cast<int64_t>(min(n0 + crow, N - 1)) * (SBF ? 2 : 4);
  const int64_t s_group_pitch = static_cast<int64_t>(N) * (SBF ? 2 : 4);
  // The scales of four slabs are requested at once, a superslab ahead, by untracked loads (valid once a later
  // end-of-slab wait has covered them); the pointer walks the groups slab by slab.
  const int slabs_per_group = group >> 6;
  const char* sc_ptr = sptr;
  const int8_t* zp_ptr = ZP ? Z + min(n0 + crow, N - 1) : nullptr;
  int sc_left = slabs_per_group;
  auto request_scales = [&](uint32_t (&dst)[4], int (&dstz)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (SBF)
        asm volatile("global_load_ushort %0, %1, off" : "=&v"(dst[j]) : "v"(sc_ptr) : "memory");
      else
        asm volatile("global_load_dword %0, %1, off" : "=&v"(dst[j]) : "v"(sc_ptr) : "memory");
      if constexpr (ZP) asm volatile("global_load_sbyte %0, %1, off" : "=&v"(dstz[j]) : "v"(zp_ptr) : "memory");
      if (--sc_left == 0) {
        sc_left = slabs_per_group;
        sc_ptr += s_group_pitch;
        if constexpr (ZP) zp_ptr += N;
      }
    }
  };
  auto pin_scales = [&](uint32_t (&v)[4], int (&vz)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      asm volatile("" : "+v"(v[j]));
      if constexpr (ZP) asm volatile("" : "+v"(vz[j]));
    }
  };
  constexpr int kSL = ZP ? 8 : 4;  // loads of one request_scales
  constexpr int NRAW = NPT * (W8 ? 8 : 4) / 32;  // dwords of raw weights per thread and slab
  int craw[NRAW];
  uint32_t cout[NPT / 2];
  auto convert_read = [&](int kt) {
    const uint8_t* src;
    if constexpr (W8) {  // the row's 64 bytes of this slab, NPT of them
      src = smem + R_BASE + (kt & 3) * R_STAGE + (crow / RPW) * 1024 + (crow % RPW) * 64 + cpart * NPT;
    } else {  // NPT / 2 bytes of the row's line: 32 bytes per slab, in two 16-byte chunks
      const int byte = cpart * (NPT / 2);  // of the slab's 32
      const int chunk = ((kt & 3) * 2 + (byte >> 4)) ^ swz8(crow);
      src = smem + R_BASE + ((kt >> 2) & 1) * R_STAGE + crow * 128 + (chunk << 4) + (byte & 15);
    }
    if constexpr (NRAW == 4) {
      const v4i v = *reinterpret_cast<const v4i*>(src);
#pragma unroll
      for (int e = 0; e < 4; ++e) craw[e] = v[e];
    } else if constexpr (NRAW == 2) {
      const qwix_v2i v = *reinterpret_cast<const qwix_v2i*>(src);
      craw[0] = v[0];
      craw[1] = v[1];
    } else {
      craw[0] = *reinterpret_cast<const int*>(src);
    }
  };
  // A nibble n holds q = (n ^ 8) - 8.  With the 8 folded into the multiply-add, q * scale = fma(n ^ 8, scale, -8 scale): every
  // term is exact in f32 (four bits times the eight of a bf16 scale), so the product is the one of float(q) * scale, and a
  // byte of the masked word converts in one instruction.
  auto convert_quarter = [&](int q4, float sc, int zp) {  // elements 4 q4 .. 4 q4 + 3 of this thread's NPT
    if (q4 >= NCQ) return;
    const int off = (W8 ? 128 : 8) + (ZP ? zp : 0);          // what the stored byte / nibble carries too much
    const float moff = -static_cast<float>(off) * sc;        // exact (see above)
    auto value = [&](uint32_t u) -> float {
      if constexpr (ZP && !SBF) return static_cast<float>(static_cast<int>(u) - off) * sc;
      return __builtin_fmaf(static_cast<float>(u), sc, moff);
    };
    float f0, f1, f2, f3;
    if constexpr (F8) {
      // two bytes per instruction: v_cvt_pk_f32_fp8 issues in 8 counter ticks, v_cvt_f32_fp8 in 12.5 for one byte
      const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(craw[q4], false), hi = __builtin_amdgcn_cvt_pk_f32_fp8(craw[q4], true);
      f0 = lo[0] * sc;
      f1 = lo[1] * sc;
      f2 = hi[0] * sc;
      f3 = hi[1] * sc;
    } else if constexpr (W8) {
      const uint32_t u = static_cast<uint32_t>(craw[q4]) ^ 0x80808080u;
      f0 = value(u & 0xFFu);
      f1 = value((u >> 8) & 0xFFu);
      f2 = value((u >> 16) & 0xFFu);
      f3 = value(u >> 24);
    } else {
      const uint32_t w = static_cast<uint32_t>(craw[q4 >> 1]) ^ 0x88888888u;
      uint32_t even = w & 0x0F0F0F0Fu, odd = (w >> 4) & 0x0F0F0F0Fu;
      // opaque to the optimizer: it would fold the masks into one bit-field extract per nibble in front of the byte
      // conversion (v_bfe_u32 + v_cvt_f32_ubyte0) instead of converting the masked words' bytes in place
      asm("" : "+v"(even));
      asm("" : "+v"(odd));
      const int b0 = (q4 & 1) * 16;
      f0 = value((even >> b0) & 0xFFu);
      f1 = value((odd >> b0) & 0xFFu);
      f2 = value((even >> (b0 + 8)) & 0xFFu);
      f3 = value((odd >> (b0 + 8)) & 0xFFu);
    }
    cout[2 * q4] = pack_bf16x2(f0, f1);
    cout[2 * q4 + 1] = pack_bf16x2(f2, f3);
  };
  auto convert_write = [&](int kt) {  // NPT bf16 values: one or two 16-byte chunks of the row's slab
    uint8_t* row = smem + C_BASE + (kt & 1) * C_STAGE + crow * 128;
#pragma unroll
    for (int c = 0; c < NPT / 8; ++c)
      *reinterpret_cast<v4i*>(row + (((cpart * (NPT / 8) + c) ^ swz8(crow)) << 4)) =
          v4i{(int)cout[4 * c], (int)cout[4 * c + 1], (int)cout[4 * c + 2], (int)cout[4 * c + 3]};
  };
  auto scale_value = [&](uint32_t bits) { return __uint_as_float(SBF ? bits << 16 : bits); };

  // ---- fragments
  const int a_row = (wm * 64 + (lane & 31)) * BK;
  const int b_row = C_BASE + (wn * WN + (lane & 31)) * BK;
  const int hx = lane >> 5, x7 = swz8(lane & 31);
  v4i fa[2][TM], fb[2][TN];
  auto read_frags = [&](int sta, int stc, int ks, int buf) {
    const int off = ((ks * 2 + hx) ^ x7) << 4;
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[buf][i] = *reinterpret_cast<const v4i*>(smem + sta * A_STAGE + a_row + i * 32 * BK + off);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[buf][j] = *reinterpret_cast<const v4i*>(smem + stc * C_STAGE + b_row + j * 32 * BK + off);
  };
  auto mfma_step = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fb[buf][j]),
                                                            __builtin_bit_cast(bf16x8, fa[buf][i]), acc[i][j], 0, 0, 0);
  };
  // End of a slab: this wavefront's LDS writes are done and its loads have landed, except the NEWEST `newest` of
  // them (vmcnt counts in issue order): the requests of the slab that ends are for two slabs ahead and stay in
  // flight across the barrier.  Then everybody's.
  auto end_of_slab = [&](auto newest) {
    constexpr int n = decltype(newest)::value;
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0070 | (n & 15) | ((n >> 4) << 14));  // vmcnt(n), lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  using std::integral_constant;

  const int KT = K / 64;  // a multiple of 4
  uint32_t sc_cur[4], sc_next[4] = {0, 0, 0, 0};
  int zp_cur[4] = {0, 0, 0, 0}, zp_next[4] = {0, 0, 0, 0};
  int sta = 0;  // LDS stage of the activations of the slab being multiplied: kt % 3
  // One slab, J = kt % 4: requests activations two slabs ahead (and, at J == 0, the packed weights and scales of
  // the next superslab), converts the weights of slab kt + 1 between the k-steps of slab kt.
  // role 0: a wavefront requests and multiplies; 1: multiplies only; 2: requests only
  constexpr auto requests_of = [](int j, bool last, int role) constexpr {  // load instructions issued in slab j of four
    const bool converts = role == 0 || (role == 2) == LC;
    const bool la = role != 1 && (!last || j < 4 - AL), ls = converts && !last && j == 0;
    const bool lw = role != 1 && (W8 ? (!last || j < 3 - AL) : (!last && j == 0));
    return (la ? 4 : 0) + (lw ? NQ : 0) + (ls ? kSL : 0);
  };
  auto slab = [&](int kt, auto J, auto LAST, auto ROLE) {
    constexpr int j = decltype(J)::value, role = decltype(ROLE)::value;
    constexpr bool last = decltype(LAST)::value;  // the last four slabs: nothing further to request after two
    constexpr bool requests = role != 1, multiplies = role != 2, converts = role == 0 || (role == 2) == LC;
    constexpr bool more = !(last && j == 3);
    constexpr bool loads_a = requests && (!last || j < 4 - AL), loads_s = converts && !last && j == 0;
    // int8: slab kt + AL + 1; int4: the next superslab
    constexpr bool loads_w = requests && (W8 ? (!last || j < 3 - AL) : (!last && j == 0));
    constexpr bool SPREAD = multiplies;  // a wavefront that also multiplies issues one activation load per k-step
    __builtin_amdgcn_sched_barrier(0);
    const int sta_req = sta == 0 ? AST - 1 : sta - 1;
    if constexpr (loads_a && !SPREAD) issue_a(kt + AL, sta_req);
    if constexpr (loads_w) issue_raw(W8 ? kt + AL + 1 : (kt >> 2) + 1);
    if constexpr (loads_s) request_scales(sc_next, zp_next);
    __builtin_amdgcn_sched_barrier(0);
    float sc = 0.f;
    int zc = 0;
    if constexpr (converts) {
      if constexpr (j == AL && !last) pin_scales(sc_next, zp_next);  // requested at j == 0, covered by the wait that ended j == AL - 1
      sc = scale_value(j == 3 ? sc_next[0] : sc_cur[(j + 1) & 3]);
      zc = j == 3 ? zp_next[0] : zp_cur[(j + 1) & 3];
      if constexpr (more) convert_read(kt + 1);
    }
    if constexpr (role == 2 && converts && more) {  // the whole conversion while the requests are under way
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) convert_quarter(q4, sc, zc);
    }
    if constexpr (multiplies) {
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) {
        if constexpr (loads_a && SPREAD)  // one of the four activation loads per k-step
          QWIX_GLDS16(A + (kt + AL) * BK + goffa[ks], smem + sta_req * A_STAGE + ldw * 32 * BK + ks * 1024);
        if (ks + 1 < NK) read_frags(sta, j & 1, ks + 1, (ks + 1) & 1);
        if constexpr (converts && more) convert_quarter(ks, sc, zc);
        mfma_step(ks & 1);
      }
    }
    if constexpr (converts && more) convert_write(kt + 1);
    // in flight across the barrier: the requests of this slab and of the AL - 2 before it
    constexpr int before = AL == 3 ? requests_of((j + 3) & 3, last && j > 0, role) : 0;
    end_of_slab(integral_constant<int, requests_of(j, last, role) + before>{});
    sta = sta == AST - 1 ? 0 : sta + 1;
    if constexpr (multiplies && more) read_frags(sta, (j + 1) & 1, 0, 0);
  };
  using I0 = integral_constant<int, 0>;
  using I1 = integral_constant<int, 1>;
  using I2 = integral_constant<int, 2>;
  using I3 = integral_constant<int, 3>;
  auto slabs = [&](auto ROLE) {  // every role passes the same K / 64 barriers
    int kt = 0;
    for (; kt + 4 < KT; kt += 4) {
      slab(kt, I0{}, std::false_type{}, ROLE);
      slab(kt + 1, I1{}, std::false_type{}, ROLE);
      slab(kt + 2, I2{}, std::false_type{}, ROLE);
      slab(kt + 3, I3{}, std::false_type{}, ROLE);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        sc_cur[e] = sc_next[e];
        zp_cur[e] = zp_next[e];
      }
    }
    slab(kt, I0{}, std::true_type{}, ROLE);
    slab(kt + 1, I1{}, std::true_type{}, ROLE);
    slab(kt + 2, I2{}, std::true_type{}, ROLE);
    slab(kt + 3, I3{}, std::true_type{}, ROLE);
  };

  // ---- prologue: packed weights of slabs 0..3 (int8: 0..AL), activations of slabs 0..AL - 1, scales; slab 0 converted.
  // Two barriers for every role.
  const bool converter = !SPEC || loader == LC;  // wave-uniform
  if (!SPEC || loader) {
    issue_raw(0);
    if constexpr (W8) {
#pragma unroll
      for (int i = 1; i <= AL; ++i) issue_raw(i);
    }
#pragma unroll
    for (int i = 0; i < AL; ++i) issue_a(i, i);
  }
  // every wavefront requests them: registers of loads in flight must not pass the join of a branch
  request_scales(sc_cur, zp_cur);
  end_of_slab(integral_constant<int, 0>{});
  pin_scales(sc_cur, zp_cur);
  if (converter) {
    convert_read(0);
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) convert_quarter(q4, scale_value(sc_cur[0]), zp_cur[0]);
    convert_write(0);
  }
  end_of_slab(integral_constant<int, 0>{});
  if constexpr (SPEC) {
    if (loader) {
      slabs(I2{});
      return;  // a wavefront that has ended no longer counts at the workgroup's barriers
    }
    read_frags(0, 0, 0, 0);
    slabs(I1{});
  } else {
    read_frags(0, 0, 0, 0);
    slabs(I0{});
  }

  float sav[TM];
  float sbv[TN][4][4];
#pragma unroll
  for (int i = 0; i < TM; ++i) sav[i] = 1.f;
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int qd = 0; qd < 4; ++qd)
#pragma unroll
      for (int r = 0; r < 4; ++r) sbv[j][qd][r] = 1.f;
  const Epilogue ep{nullptr, nullptr, 0, 0, OUT, 0, 0, 0, nullptr, nullptr};
  staged_epilogue<OUT, 0, TM, TN, NWAVES, LDS_BYTES, false>(acc, sav, sbv, ep, m0 + wm * 64, n0 + wn * WN, M, N, out, ldo,
                                                            smem, wave, lane);
}

}  // namespace
}  // namespace qwix

extern "C" int qwix_hip_ksum_i8(const void* q, int64_t ld, int64_t rows, int64_t K, int32_t* out, void* stream) {
  if (!q || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null argument");
  if (rows <= 0 || K <= 0 || rows > INT32_MAX || K > INT32_MAX || K % 16 || ld % 16 || ld < K || !aligned16(q))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "ksum_i8 needs K and ld multiples of 16 and a 16-byte aligned base "
                "(rows=%lld K=%lld ld=%lld)", (long long)rows, (long long)K, (long long)ld);
  ksum_i8_kernel<<<dim3(static_cast<unsigned>((rows + 3) / 4)), 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const int8_t*>(q), ld, static_cast<int>(rows), static_cast<int>(K), out);
  return check_launch("ksum_i8");
}

static int qgemm_impl(const void* a, int64_t lda, const void* b, int64_t ldb, int qtype, int64_t M, int64_t N, int64_t K,
                      const void* sa, int sa_dtype, const void* sb, int sb_dtype, int acc_dtype, const int32_t* zu,
                      const int32_t* zv, void* out, int out_dtype, int64_t ldo, void* stream, void* workspace = nullptr,
                      size_t workspace_bytes = 0);
static int splitk_plan(int64_t M, int64_t N, int64_t K, double other_us);
// Problems of up to this many 128 x 128 tiles take 64 x 64 tiles (four times the workgroups).  Measured, int8 and
// e4m3, bf16 result, weights in the second-level cache / from HBM: 256 x 4096 over K 1024 9.5 -> 5.6 / 12.1 -> 8.4 us,
// 1024^3 9.3 -> 5.4 / 11.7 -> 8.2, 512 x 4096 over K 4096 23.5 -> 16.2 / 34.9 -> 26.8, 1536 x 2048 over K 2048 (192
// tiles) 16.0 -> 12.6 / 18.3 -> 14.6; level from 256 tiles on (2048 x 2048 over K 1024: 10.6 / 10.4 us), behind at 512
// (4096 x 2048 over K 1024: 13.0 / 17.1 us).
#ifndef QWIX_SMALL_TILES
#define QWIX_SMALL_TILES 200
#endif
constexpr int64_t kSmallTiles = QWIX_SMALL_TILES;

// What the unsplit tiled kernel takes, in us (the figure a split of K has to beat), with weights that come from HBM
// as a model's do (copies in rotation, 600 MB): 64 x 64 tiles with four stages 3.5 us + 0.29 us per 128 of K and round
// of 256 workgroups (256 x 1024 over K 4096 12.7 us, 512 x 512 over K 8192 21.8 us, 512 x 4096 over K 4096 21.0 us),
// 0.58 us per slab with two stages, 128 x 128 tiles beyond.
static double tiled_model_us(int64_t M, int64_t N, int64_t K) {
  const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128), tiles64 = ((M + 63) / 64) * ((N + 63) / 64);
  const double slabs = static_cast<double>(K / 128);
  if (M < 64 && N * K >= (int64_t{8} << 20)) return 5.0 + 0.55 * slabs;  // the one-tile-row kernel's range
  if (tiles128 <= kSmallTiles && tiles64 <= 512) return 3.5 + 0.29 * slabs * (tiles64 <= 256 ? 1.0 : tiles64 / 256.0);
  if (tiles128 <= kSmallTiles) return 3.5 + 0.58 * slabs;
  return 5.0 + 0.55 * slabs;
}

static bool streams_weights(int64_t M, int64_t N, int64_t K, bool one_tile_row = false);

// Dtype chain of the reference epilogue: int32 adopts the first scale's dtype (through f32); a
// float accumulator starts in acc_dtype; each multiply happens in the promotion of both sides.
static Epilogue make_epilogue(int qtype, const void* sa, int sa_dtype, const void* sb, int sb_dtype, int acc_dtype,
                              const int32_t* zu, const int32_t* zv, int out_dtype) {
  Epilogue ep{sa, sb, sa_dtype, sb_dtype, out_dtype, 0, 0, 0, zu, zv};
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
  return ep;
}

// Argument checks shared by the dense and the ragged entry points.
static int check_gemm_args(const void* a, int64_t lda, const void* b, int64_t ldb, int qtype, int64_t M, int64_t N,
                           int64_t K, const void* sa, int sa_dtype, const void* sb, int sb_dtype, int acc_dtype,
                           const void* out, int out_dtype, int64_t ldo) {
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
  return QWIX_OK;
}

extern "C" int qwix_hip_qgemm_fused_act(const void* x, int x_dtype, int64_t ldx, const void* b, int64_t ldb,
                                        int64_t M, int64_t N, int64_t K, const void* sb, int sb_dtype, void* out,
                                        int out_dtype, int64_t ldo, void* stream) {
  if (!x || !b || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null x/b/out");
  if (x_dtype != QWIX_BF16 && x_dtype != QWIX_F32) return fail(QWIX_ERR_INVALID_ARGUMENT, "activations must be bf16 or f32");
  if ((sb && sb_dtype != QWIX_BF16 && sb_dtype != QWIX_F32) || (out_dtype != QWIX_BF16 && out_dtype != QWIX_F32))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "scale and output dtypes must be f32 or bf16");
  const int es = x_dtype == QWIX_BF16 ? 2 : 4;
  // One 128-wide K block per wavefront: beyond K = 2048 the arithmetic of re-quantizing the rows in every
  // workgroup costs more than the launch of a separate quantize kernel saves (measured: K = 1024 runs in half
  // the time of the two launches, K = 4096 in the same time).
  constexpr int64_t kMaxK = 128 * kSkinnyWaves;
  if (M <= 0 || M > 32 || N <= 0 || N > INT32_MAX || K <= 0 || K % 128 || K > kMaxK)
    return fail(QWIX_ERR_UNSUPPORTED, "fused activation quantize needs 1..32 rows and K a multiple of 128 up to %lld "
                "(M=%lld K=%lld)", (long long)kMaxK, (long long)M, (long long)K);
  if (ldx < K || (ldx * es) % 16 || ldb < K || ldb % 16 || !aligned16(x) || !aligned16(b) || ldo < N ||
      32 * ldx * es >= (int64_t{1} << 31) || 64 * ldb >= (int64_t{1} << 31))
    return fail(QWIX_ERR_UNSUPPORTED, "bad leading dimensions or alignment (ldx=%lld ldb=%lld ldo=%lld)", (long long)ldx,
                (long long)ldb, (long long)ldo);
  // the activation scale is computed in the activations' dtype, like the stand-alone quantize does
  const Epilogue ep = make_epilogue(QWIX_INT8, x, x_dtype, sb, sb_dtype, 0, nullptr, nullptr, out_dtype);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (x_dtype == QWIX_BF16) return launch_skinny_fused<BF16, 1>(x, ldx, b, ldb, M, N, K, ep, out, ldo, st);
  return launch_skinny_fused<F32, 1>(x, ldx, b, ldb, M, N, K, ep, out, ldo, st);
}

extern "C" int qwix_hip_qgemm_ragged(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t b_group_stride,
                                     int qtype, int64_t M, int64_t N, int64_t K, const int32_t* group_sizes,
                                     int64_t G, const void* sa, int sa_dtype, const void* sb, int sb_dtype,
                                     int64_t sb_group_stride, int acc_dtype, void* out, int out_dtype, int64_t ldo,
                                     void* stream) {
  if (const int rc = check_gemm_args(a, lda, b, ldb, qtype, M, N, K, sa, sa_dtype, sb, sb_dtype, acc_dtype, out,
                                     out_dtype, ldo))
    return rc;
  if (!group_sizes || G <= 0 || G > 65536)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "ragged qgemm needs 1..65536 group sizes (G=%lld)", (long long)G);
  if (b_group_stride % 16 || b_group_stride < 0 || sb_group_stride < 0 || (sb_group_stride % 4 != 0 && N % 4 == 0))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad group strides (b: %lld bytes, sb: %lld elements)",
                (long long)b_group_stride, (long long)sb_group_stride);
  if (M * lda >= (int64_t{1} << 31) || N * ldb >= (int64_t{1} << 31) ||
      (M / 128 + G + 1) * ((N + 127) / 128) >= (int64_t{1} << 31))
    return fail(QWIX_ERR_UNSUPPORTED, "ragged qgemm: operand too large for 32-bit offsets (M*lda=%lld N*ldb=%lld)",
                (long long)(M * lda), (long long)(N * ldb));
  const Epilogue ep = make_epilogue(qtype, sa, sa_dtype, sb, sb_dtype, acc_dtype, nullptr, nullptr, out_dtype);
  const Ragged rg{group_sizes, static_cast<int>(G), b_group_stride, sb_group_stride};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (K % 128 == 0 && M <= 16 * G && G + 1 <= 65535 && 64 * ldb < (int64_t{1} << 31)) {
    // at most 16 rows per group on average (decode): stream every group's weight once instead of tiling
    // (measured, 64 groups x 2048 x 4096: 146 -> 119 us; at 32 rows per group a second pass over the weights loses)
    if (qtype == QWIX_INT8) return launch_ragged_skinny<QWIX_INT8>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
    return launch_ragged_skinny<QWIX_E4M3>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
  }
  if (K % 128 == 0) {
    // 256-row tiles pay off once the average group is several tiles tall; 128-row tiles waste fewer rows
    // at the ragged end of each group.
    const bool big = M / G >= 768 && ((M + 255) / 256) * ((N + 255) / 256) >= 192;
    // 17 to 48 rows per group on average: 64-row tiles with the deep weight prefetch (64 groups x 32 rows, K 2048,
    // N 4096: 131.7 against 144.8 us; from 64 rows per group on the 128-row tile wins again, 174 against 160 us)
    if (M <= 48 * G && out_dtype != QWIX_I32 &&
        (M / 64 + G + 1) * ((N + 127) / 128) < (int64_t{1} << 31)) {
      if (qtype == QWIX_INT8) {
        if (out_dtype == QWIX_BF16) return launch_ragged_mid<QWIX_INT8, QWIX_BF16>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
        return launch_ragged_mid<QWIX_INT8, QWIX_F32>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
      }
      if (out_dtype == QWIX_BF16) return launch_ragged_mid<QWIX_E4M3, QWIX_BF16>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
      return launch_ragged_mid<QWIX_E4M3, QWIX_F32>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
    }
    if (big && K >= 256 && out_dtype != QWIX_I32) {
      if (qtype == QWIX_INT8) {
        if (out_dtype == QWIX_BF16) return launch_ragged_pp<QWIX_INT8, QWIX_BF16>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
        return launch_ragged_pp<QWIX_INT8, QWIX_F32>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
      }
      if (out_dtype == QWIX_BF16) return launch_ragged_pp<QWIX_E4M3, QWIX_BF16>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
      return launch_ragged_pp<QWIX_E4M3, QWIX_F32>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
    }
    if (qtype == QWIX_INT8) {
      if (big) return dispatch_ragged_dma<QWIX_INT8, 256, 256, 2, 4>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
      return dispatch_ragged_dma<QWIX_INT8, 128, 128, 2, 2>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
    }
    if (big) return dispatch_ragged_dma<QWIX_E4M3, 256, 256, 2, 4>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
    return dispatch_ragged_dma<QWIX_E4M3, 128, 128, 2, 2>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
  }
  if (qtype == QWIX_INT8) return launch_ragged<QWIX_INT8>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
  return launch_ragged<QWIX_E4M3>(a, lda, b, ldb, rg, M, N, K, ep, out, ldo, st);
}

// Workspace of qwix_hip_qgemm_dynamic_act: the quantized rows, their scales, what the quantize kernel itself needs
// for rows too long for one workgroup, and the GEMM's split-K partials; each part 256-byte aligned.
static size_t dyn_align(size_t v) { return (v + 255) & ~size_t{255}; }
extern "C" size_t qwix_hip_qgemm_dynamic_act_workspace_bytes(int64_t M, int64_t N, int64_t K, int x_dtype) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const size_t es = x_dtype == QWIX_BF16 ? 2 : 4;
  return dyn_align(static_cast<size_t>(M) * K) + dyn_align(static_cast<size_t>(M) * es) +
         dyn_align(qwix_hip_quantize_workspace_bytes(M, K, 1, K, QWIX_ABSMAX)) +
         dyn_align(qwix_hip_qgemm_workspace_bytes(M, N, K));
}

extern "C" int qwix_hip_qgemm_dynamic_act(const void* x, int x_dtype, int64_t ldx, const void* b, int64_t ldb, int qtype,
                                          int64_t M, int64_t N, int64_t K, const void* sb, int sb_dtype, int acc_dtype,
                                          void* out, int out_dtype, int64_t ldo, void* workspace,
                                          size_t workspace_bytes, void* stream) {
  if (!x || !b || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null x/b/out");
  if (x_dtype != QWIX_BF16 && x_dtype != QWIX_F32) return fail(QWIX_ERR_INVALID_ARGUMENT, "activations must be bf16 or f32");
  if (qtype != QWIX_INT8 && qtype != QWIX_E4M3)
    return fail(QWIX_ERR_UNSUPPORTED, "dynamic activation quantization to int8 or e4m3 (got qtype %d)", qtype);
  if (M <= 0 || N <= 0 || K <= 0) return fail(QWIX_ERR_INVALID_ARGUMENT, "bad shape M=%lld N=%lld K=%lld", (long long)M,
                                             (long long)N, (long long)K);
  // decode-size int8 calls: one launch (the rows are quantized in the GEMM's prologue)
  if (qtype == QWIX_INT8 && M <= 32 && K % 128 == 0 && K <= 128 * kSkinnyWaves && sb != nullptr)
    return qwix_hip_qgemm_fused_act(x, x_dtype, ldx, b, ldb, M, N, K, sb, sb_dtype, out, out_dtype, ldo, stream);
  // otherwise: the quantize kernel, then the GEMM, on the caller's scratch memory
  if (ldx != K) return fail(QWIX_ERR_UNSUPPORTED, "the two-launch route needs dense activation rows (ldx=%lld K=%lld)",
                            (long long)ldx, (long long)K);
  const size_t need = qwix_hip_qgemm_dynamic_act_workspace_bytes(M, N, K, x_dtype);
  if (!workspace || workspace_bytes < need || !aligned16(workspace))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "workspace of %zu bytes required, got %zu", need, workspace_bytes);
  const size_t es = x_dtype == QWIX_BF16 ? 2 : 4;
  uint8_t* q = static_cast<uint8_t*>(workspace);
  uint8_t* sa = q + dyn_align(static_cast<size_t>(M) * K);
  uint8_t* qws = sa + dyn_align(static_cast<size_t>(M) * es);
  const size_t qws_bytes = qwix_hip_quantize_workspace_bytes(M, K, 1, K, QWIX_ABSMAX);
  uint8_t* gws = qws + dyn_align(qws_bytes);
  const size_t gws_bytes = qwix_hip_qgemm_workspace_bytes(M, N, K);
  if (int e = qwix_hip_quantize(x, x_dtype, M, K, 1, K, qtype, QWIX_ABSMAX, 0.f, QWIX_LAYOUT_NATURAL, q, sa, nullptr,
                                qws_bytes ? qws : nullptr, qws_bytes, stream))
    return e;
  return qgemm_impl(q, K, b, ldb, qtype, M, N, K, sa, x_dtype, sb, sb_dtype, acc_dtype, nullptr, nullptr, out, out_dtype,
                    ldo, stream, gws_bytes ? gws : nullptr, gws_bytes);
}

extern "C" int qwix_hip_gemm_bf16(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
                                  void* out, int out_dtype, int64_t ldo, void* stream) {
  if (!a || !b || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null a/b/out");
  if (M <= 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || 2 * K > INT32_MAX)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad GEMM shape M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                (long long)K);
  if (out_dtype != QWIX_BF16 && out_dtype != QWIX_F32) return fail(QWIX_ERR_INVALID_ARGUMENT, "bad out dtype %d", out_dtype);
  // rows are walked in 128-byte slabs that go to LDS directly
  if (K % 64 || lda % 8 || ldb % 8 || lda < K || ldb < K || !aligned16(a) || !aligned16(b))
    return fail(QWIX_ERR_UNSUPPORTED, "bf16 GEMM needs K a multiple of 64, row pitches multiples of 8 elements and "
                "16-byte aligned operands (K=%lld lda=%lld ldb=%lld)", (long long)K, (long long)lda, (long long)ldb);
  if (ldo < N || !aligned16(out) || (N % 4 == 0 && ldo % 4 != 0))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad output leading dimension %lld for N=%lld", (long long)ldo, (long long)N);
  const int64_t ldab = 2 * lda, ldbb = 2 * ldb, kb = 2 * K;  // the tile bodies count bytes
  if (M * ldab >= (int64_t{1} << 31) || N * ldbb >= (int64_t{1} << 31))
    return fail(QWIX_ERR_UNSUPPORTED, "operands beyond 2 GiB are not supported by the bf16 GEMM");
  const Epilogue ep{nullptr, nullptr, 0, 0, out_dtype, 0, 0, 0, nullptr, nullptr};
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool big = ((M + 255) / 256) * ((N + 255) / 256) >= 192;
  if (out_dtype == QWIX_BF16) {
    if (big && kb >= 256) return launch_pp<kOpBf16, QWIX_BF16, 0>(a, ldab, b, ldbb, M, N, kb, ep, out, ldo, st);
    if (big) return launch_dma<kOpBf16, 256, 256, 2, 4, QWIX_BF16, 0>(a, ldab, b, ldbb, M, N, kb, ep, out, ldo, st);
    return launch_dma<kOpBf16, 128, 128, 2, 2, QWIX_BF16, 0>(a, ldab, b, ldbb, M, N, kb, ep, out, ldo, st);
  }
  if (big && kb >= 256) return launch_pp<kOpBf16, QWIX_F32, 0>(a, ldab, b, ldbb, M, N, kb, ep, out, ldo, st);
  if (big) return launch_dma<kOpBf16, 256, 256, 2, 4, QWIX_F32, 0>(a, ldab, b, ldbb, M, N, kb, ep, out, ldo, st);
  return launch_dma<kOpBf16, 128, 128, 2, 2, QWIX_F32, 0>(a, ldab, b, ldbb, M, N, kb, ep, out, ldo, st);
}

template <bool IS_INT>
__global__ void __launch_bounds__(256)
    splitk_reduce_kernel(const uint8_t* __restrict__ ws, int splits, int M, int N, Epilogue ep, uint8_t* __restrict__ out,
                         int64_t ldo);  // defined with the split-K kernels of the quantized GEMM below

// The K split of qwix_hip_gemm_bf16_wq_ws: 0 = none.  The tile kernel walks K in 64-element slabs of about 0.37 us
// each, however few workgroups there are; while they cover at most half of the CUs, K is cut into equal ranges (whole
// 256-element superslabs; whole scale groups, or equal parts of one; at least 1024 elements) for up to one workgroup
// per CU.
static int wq_splits(int64_t M, int64_t N, int64_t K, int64_t group) {
  if (M <= 0 || N <= 0 || K <= 0 || group <= 0 || K % 256 || group % 64 || K % group) return 0;
  const bool low = M <= 128;
  const bool narrow = ((M + 255) / 256) * ((N + 127) / 128) <= 128;
  const int64_t tiles = ((M + (low ? 127 : 255)) / (low ? 128 : 256)) * ((N + (low || narrow ? 63 : 127)) / (low || narrow ? 64 : 128));
  if (tiles > 128) return 0;
  // a range is whole superslabs, and whole scale groups or a whole part of one (never across a group's end)
  int best = 0;
  for (int64_t sp = 2; sp * tiles <= 256 && sp * 1024 <= K; ++sp) {
    if (K % (sp * 256)) continue;
    const int64_t len = K / sp;
    if (len % group == 0 || group % len == 0) best = static_cast<int>(sp);
  }
  return best;
}

static int gemm_bf16_wq_impl(const void* a, int64_t lda, const void* q, int64_t ldq_bytes, int q_qtype, int64_t M,
                             int64_t N, int64_t K, int64_t group, const void* s, int s_dtype, const int8_t* zp,
                             void* out, int out_dtype, int64_t ldo, void* stream, void* workspace,
                             size_t workspace_bytes) {
  if (!a || !q || !s || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null a/q/s/out");
  if (q_qtype != QWIX_INT4 && q_qtype != QWIX_INT8 && q_qtype != QWIX_E4M3)
    return fail(QWIX_ERR_UNSUPPORTED, "weight qtype %d: int4, int8 or e4m3", q_qtype);
  if (q_qtype == QWIX_E4M3 && zp) return fail(QWIX_ERR_INVALID_ARGUMENT, "e4m3 weights have no zero point");
  if (M <= 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || 2 * K > INT32_MAX)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad GEMM shape M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                (long long)K);
  if ((out_dtype != QWIX_BF16 && out_dtype != QWIX_F32) || (s_dtype != QWIX_BF16 && s_dtype != QWIX_F32))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "scale and output dtypes must be f32 or bf16");
  // K in groups of four 64-element slabs (for int4 a 128-byte line of packed weights); a scale group covers whole slabs
  if (K % 256 || group <= 0 || group % 64 || K % group)
    return fail(QWIX_ERR_UNSUPPORTED, "K=%lld must be a multiple of 256 and group=%lld a multiple of 64 that divides K",
                (long long)K, (long long)group);
  const int64_t row_bytes = q_qtype == QWIX_INT4 ? K / 2 : K;
  if (lda % 8 || lda < K || ldq_bytes % 16 || ldq_bytes < row_bytes || !aligned16(a) || !aligned16(q))
    return fail(QWIX_ERR_UNSUPPORTED, "activation and weight rows must be 16-byte aligned (lda=%lld ldq=%lld)",
                (long long)lda, (long long)ldq_bytes);
  if (ldo < N || !aligned16(out) || (N % 4 == 0 && ldo % 4 != 0))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad output leading dimension %lld for N=%lld", (long long)ldo, (long long)N);
  if (M * lda * 2 >= (int64_t{1} << 31) || N * ldq_bytes >= (int64_t{1} << 31))
    return fail(QWIX_ERR_UNSUPPORTED, "operands beyond 2 GiB are not supported");
  // 64-column tiles while 128-column ones would occupy at most half of the CUs; 128-row tiles for up to 128 rows
  const bool narrow = ((M + 255) / 256) * ((N + 127) / 128) <= 128;
  const bool low = M <= 128;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // with a workspace that holds them: f32 partials of `splits` K ranges, added up (in range order) by a second kernel
  int splits = workspace ? wq_splits(M, N, K, group) : 0;
  if (splits > 0 && (workspace_bytes < static_cast<size_t>(splits) * M * N * 4 || !aligned16(workspace))) splits = 0;
  const int ksplit = splits > 0 ? static_cast<int>(K / splits) : 0;
  const int kern_out = splits > 0 ? QWIX_F32 : out_dtype;
  uint8_t* const kern_dst = static_cast<uint8_t*>(splits > 0 ? workspace : out);
  const int64_t kern_ldo = splits > 0 ? N : ldo;
#define QWIX_WQ_LAUNCH(OUTT, SBFF, BMM, BNN, BITS) \
  do {                                             \
    if (zp) QWIX_WQ_LAUNCH_Z(OUTT, SBFF, BMM, BNN, BITS, (BITS != 9)); else QWIX_WQ_LAUNCH_Z(OUTT, SBFF, BMM, BNN, BITS, false); \
  } while (0)
#define QWIX_WQ_LAUNCH_Z(OUTT, SBFF, BMM, BNN, BITS, ZPP)                                                            \
  do {                                                                                                               \
    auto kern = wgemm_wq_kernel<OUTT, SBFF, BMM, BNN, BITS, ZPP>;                                                    \
    /* activations 96 KB, converted weights 2 x BN x 128, raw weights 2 x BN x 128 (int8: 4 x 8 KB): <= 160 KB */    \
    constexpr size_t smem = (BMM == 128 ? 4 : 3) * BMM * 128 + 2 * BNN * 128 + (BITS >= 8 ? 4 * (BMM / 32) * 1024 : 2 * BNN * 128);      \
    const dim3 grid(static_cast<unsigned>(((M + BMM - 1) / BMM) * ((N + BNN - 1) / BNN)),                            \
                    static_cast<unsigned>(splits > 0 ? splits : 1));                                                 \
    static LdsGrant granted;                                                                                         \
    if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;                           \
    kern<<<grid, 512, smem, st>>>(static_cast<const uint8_t*>(a), 2 * lda, static_cast<const uint8_t*>(q), ldq_bytes, s, \
                                  zp, static_cast<int>(M), static_cast<int>(N), static_cast<int>(K),                 \
                                  static_cast<int>(group), kern_dst, kern_ldo, ksplit);                              \
  } while (0)
#define QWIX_WQ_TILE(OUTT, SBFF, BITS)                                                                               \
  do {                                                                                                               \
    if (low) QWIX_WQ_LAUNCH(OUTT, SBFF, 128, 64, BITS);                                                              \
    else if (narrow) QWIX_WQ_LAUNCH(OUTT, SBFF, 256, 64, BITS);                                                      \
    else QWIX_WQ_LAUNCH(OUTT, SBFF, 256, 128, BITS);                                                                 \
  } while (0)
#define QWIX_WQ_BITS(OUTT, SBFF)                                                                                     \
  do {                                                                                                               \
    if (q_qtype == QWIX_INT4) QWIX_WQ_TILE(OUTT, SBFF, 4);                                                           \
    else if (q_qtype == QWIX_INT8) QWIX_WQ_TILE(OUTT, SBFF, 8);                                                      \
    else QWIX_WQ_TILE(OUTT, SBFF, 9); /* e4m3 */                                                                     \
  } while (0)
  if (kern_out == QWIX_BF16) {
    if (s_dtype == QWIX_BF16) QWIX_WQ_BITS(QWIX_BF16, true); else QWIX_WQ_BITS(QWIX_BF16, false);
  } else {
    if (s_dtype == QWIX_BF16) QWIX_WQ_BITS(QWIX_F32, true); else QWIX_WQ_BITS(QWIX_F32, false);
  }
#undef QWIX_WQ_BITS
#undef QWIX_WQ_TILE
#undef QWIX_WQ_LAUNCH
#undef QWIX_WQ_LAUNCH_Z
  if (int e = check_launch("gemm_bf16_wq")) return e;
  if (splits > 0) {
    const Epilogue ep{nullptr, nullptr, 0, 0, out_dtype, 0, 0, 0, nullptr, nullptr};
    const int64_t threads = (M * N + 3) / 4;
    splitk_reduce_kernel<false><<<dim3(static_cast<unsigned>((threads + 255) / 256)), 256, 0, st>>>(
        static_cast<const uint8_t*>(workspace), splits, static_cast<int>(M), static_cast<int>(N), ep,
        static_cast<uint8_t*>(out), ldo);
    return check_launch("gemm_bf16_wq (split K)");
  }
  return 0;
}

extern "C" int qwix_hip_gemm_bf16_wq(const void* a, int64_t lda, const void* q, int64_t ldq_bytes, int q_qtype, int64_t M,
                                     int64_t N, int64_t K, int64_t group, const void* s, int s_dtype, const int8_t* zp,
                                     void* out, int out_dtype, int64_t ldo, void* stream) {
  return gemm_bf16_wq_impl(a, lda, q, ldq_bytes, q_qtype, M, N, K, group, s, s_dtype, zp, out, out_dtype, ldo, stream,
                           nullptr, 0);
}

extern "C" size_t qwix_hip_gemm_bf16_wq_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t group) {
  return static_cast<size_t>(wq_splits(M, N, K, group)) * static_cast<size_t>(M > 0 ? M : 0) * static_cast<size_t>(N > 0 ? N : 0) * 4;
}

extern "C" int qwix_hip_gemm_bf16_wq_ws(const void* a, int64_t lda, const void* q, int64_t ldq_bytes, int q_qtype,
                                        int64_t M, int64_t N, int64_t K, int64_t group, const void* s, int s_dtype,
                                        const int8_t* zp, void* out, int out_dtype, int64_t ldo, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  return gemm_bf16_wq_impl(a, lda, q, ldq_bytes, q_qtype, M, N, K, group, s, s_dtype, zp, out, out_dtype, ldo, stream,
                           workspace, workspace_bytes);
}

extern "C" int qwix_hip_qgemm(const void* a, int64_t lda, const void* b, int64_t ldb, int qtype, int64_t M,
                              int64_t N, int64_t K, const void* sa, int sa_dtype, const void* sb, int sb_dtype,
                              int acc_dtype, void* out, int out_dtype, int64_t ldo, void* stream) {
  return qgemm_impl(a, lda, b, ldb, qtype, M, N, K, sa, sa_dtype, sb, sb_dtype, acc_dtype, nullptr, nullptr, out,
                    out_dtype, ldo, stream);
}

extern "C" size_t qwix_hip_qgemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  // the split count qwix_hip_qgemm_ws would pick: the plan against the unsplit tiled kernel's model
  const int splits = streams_weights(M, N, K) ? 0 : splitk_plan(M, N, K, tiled_model_us(M, N, K));
  return splits > 0 ? static_cast<size_t>(splits) * M * N * 4 : 0;
}

extern "C" int qwix_hip_qgemm_ws(const void* a, int64_t lda, const void* b, int64_t ldb, int qtype, int64_t M,
                                 int64_t N, int64_t K, const void* sa, int sa_dtype, const void* sb, int sb_dtype,
                                 int acc_dtype, void* out, int out_dtype, int64_t ldo, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  return qgemm_impl(a, lda, b, ldb, qtype, M, N, K, sa, sa_dtype, sb, sb_dtype, acc_dtype, nullptr, nullptr, out,
                    out_dtype, ldo, stream, workspace, workspace_bytes);
}

extern "C" int qwix_hip_qgemm_zp(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N,
                                 int64_t K, const void* sa, int sa_dtype, const void* sb, int sb_dtype,
                                 const int32_t* zu, const int32_t* zv, void* out, int out_dtype, int64_t ldo,
                                 void* stream) {
  if (!zu || !zv) return fail(QWIX_ERR_INVALID_ARGUMENT, "null zero-point vectors");
  if (out_dtype != QWIX_F32 && out_dtype != QWIX_BF16)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "zero-point corrected output must be f32 or bf16");
  return qgemm_impl(a, lda, b, ldb, QWIX_INT8, M, N, K, sa, sa_dtype, sb, sb_dtype, 0, zu, zv, out, out_dtype, ldo,
                    stream);
}

extern "C" int qwix_hip_qgemm_batched(const void* a, int64_t lda, int64_t a_batch_stride, const void* b, int64_t ldb,
                                      int64_t b_batch_stride, int qtype, int64_t batch, int64_t M, int64_t N,
                                      int64_t K, const void* sa, int sa_dtype, int64_t sa_batch_stride,
                                      const void* sb, int sb_dtype, int64_t sb_batch_stride, int acc_dtype,
                                      void* out, int out_dtype, int64_t ldo, int64_t out_batch_stride,
                                      void* stream) {
  if (const int rc = check_gemm_args(a, lda, b, ldb, qtype, M, N, K, sa, sa_dtype, sb, sb_dtype, acc_dtype, out,
                                     out_dtype, ldo))
    return rc;
  if (batch <= 0 || batch > 65535)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "batched qgemm needs 1..65535 problems (batch=%lld)", (long long)batch);
  if (a_batch_stride % 16 || b_batch_stride % 16 || a_batch_stride < 0 || b_batch_stride < 0 || sa_batch_stride < 0 ||
      sb_batch_stride < 0 || out_batch_stride < 0 || (N % 4 == 0 && (sb_batch_stride % 4 || out_batch_stride % 4)))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad batch strides (a %lld b %lld bytes; sa %lld sb %lld out %lld elements)",
                (long long)a_batch_stride, (long long)b_batch_stride, (long long)sa_batch_stride,
                (long long)sb_batch_stride, (long long)out_batch_stride);
  if (M * lda >= (int64_t{1} << 31) || N * ldb >= (int64_t{1} << 31))
    return fail(QWIX_ERR_UNSUPPORTED, "batched qgemm: one problem must fit 32-bit offsets (M*lda=%lld N*ldb=%lld)",
                (long long)(M * lda), (long long)(N * ldb));
  const Epilogue ep = make_epilogue(qtype, sa, sa_dtype, sb, sb_dtype, acc_dtype, nullptr, nullptr, out_dtype);
  const Batched bs{a_batch_stride, b_batch_stride, sa_batch_stride, sb_batch_stride, out_batch_stride};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (qtype == QWIX_INT8) return launch_batched<QWIX_INT8>(a, lda, b, ldb, bs, batch, M, N, K, ep, out, ldo, st);
  return launch_batched<QWIX_E4M3>(a, lda, b, ldb, bs, batch, M, N, K, ep, out, ldo, st);
}

// ------------------------------------------------------------------------------------------------
// Split-K for problems whose 128 x 128 tiles occupy a fraction of the chip while K is long (a few hundred
// rows against a narrow weight): the grid gets a second dimension over ranges of K slabs, every workgroup
// writes its raw partial tile (int32, or f32 for e4m3) to a caller workspace [split][M][N], and a second
// kernel sums the splits and applies the epilogue.  Integer partials add exactly, so int8 results are the
// bits of the unsplit kernels.
template <int QT>
__global__ void __launch_bounds__(256)
    qgemm_splitk_kernel(const uint8_t* __restrict__ A, int64_t lda, const uint8_t* __restrict__ B, int64_t ldb, int M,
                        int N, int K, int slabs_per_split, uint8_t* __restrict__ ws) {
  int tile_m, tile_n;
  tile_coords((M + 127) / 128, (N + 127) / 128, &tile_m, &tile_n);
  const int k0 = blockIdx.y * slabs_per_split * 128;
  const int klen = min(K - k0, slabs_per_split * 128);  // > 0: the host sizes the grid that way
  const Epilogue raw{nullptr, nullptr, 0, 0, QT == QWIX_INT8 ? QWIX_I32 : QWIX_F32, 0, 0, 0, nullptr, nullptr};
  uint8_t* part = ws + static_cast<int64_t>(blockIdx.y) * M * N * 4;
  qgemm_dma_tile<QT, 128, 128, 2, 2, (QT == QWIX_INT8 ? QWIX_I32 : QWIX_F32), 0>(A + k0, lda, B + k0, ldb, tile_m * 128,
                                                                                tile_n * 128, M, N, klen, raw, part, N);
}

// out[m, n] = epilogue(sum over splits of ws[s][m][n]); four consecutive elements of the flattened (m, n) per thread.
template <bool IS_INT>
__global__ void __launch_bounds__(256)
    splitk_reduce_kernel(const uint8_t* __restrict__ ws, int splits, int M, int N, Epilogue ep, uint8_t* __restrict__ out,
                         int64_t ldo) {
  const int64_t total = static_cast<int64_t>(M) * N;
  const int64_t i0 = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  if (i0 >= total) return;
  const bool vec = (N & 3) == 0;  // then the four share a row and the loads are 16-byte aligned
  float v[4];
  // Eight partials are requested before the first is added: one trip to memory per eight splits, not per split.
  // They are added in split order (int32 sums do not depend on it; the f32 sums of e4m3 partials do).
  constexpr int kBatch = 8;
  if constexpr (IS_INT) {
    int a[4] = {0, 0, 0, 0};
    for (int s0 = 0; s0 < splits; s0 += kBatch) {
      if (vec) {
        int4 w[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
          w[j] = make_int4(0, 0, 0, 0);
          if (s0 + j < splits) w[j] = *reinterpret_cast<const int4*>(reinterpret_cast<const int*>(ws) + (s0 + j) * total + i0);
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) { a[0] += w[j].x; a[1] += w[j].y; a[2] += w[j].z; a[3] += w[j].w; }
      } else {
        for (int s = s0; s < min(splits, s0 + kBatch); ++s) {
          const int* p = reinterpret_cast<const int*>(ws) + s * total + i0;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (i0 + e < total) a[e] += p[e];
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = static_cast<float>(a[e]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = 0.f;
    for (int s0 = 0; s0 < splits; s0 += kBatch) {
      if (vec) {
        float4 w[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
          w[j] = make_float4(0.f, 0.f, 0.f, 0.f);
          if (s0 + j < splits) w[j] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(ws) + (s0 + j) * total + i0);
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
          if (s0 + j < splits) { v[0] += w[j].x; v[1] += w[j].y; v[2] += w[j].z; v[3] += w[j].w; }
        }
      } else {
        for (int s = s0; s < min(splits, s0 + kBatch); ++s) {
          const float* p = reinterpret_cast<const float*>(ws) + s * total + i0;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (i0 + e < total) v[e] += p[e];
        }
      }
    }
  }
  const bool r0 = ep.r0 != 0, r1 = ep.r1 != 0, r2 = ep.r2 != 0;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int64_t i = i0 + e;
    if (i >= total) break;
    const int m = static_cast<int>(i / N), n = static_cast<int>(i % N);
    float t = v[e];
    if (r0) t = round_bf16(t);
    if (ep.sa != nullptr) t *= load_scale(ep.sa, ep.sa_dtype, m);
    if (r1) t = round_bf16(t);
    if (ep.sb != nullptr) t *= load_scale(ep.sb, ep.sb_dtype, n);
    if (r2) t = round_bf16(t);
    if (ep.out_dtype == QWIX_BF16)
      reinterpret_cast<uint16_t*>(out)[static_cast<int64_t>(m) * ldo + n] = f32_to_bf16_bits(t);
    else
      reinterpret_cast<float*>(out)[static_cast<int64_t>(m) * ldo + n] = t;
  }
}

// The rule of qgemm_impl for taking the weight-streaming kernel (see there for the model).
static bool streams_weights(int64_t M, int64_t N, int64_t K, bool one_tile_row) {
  const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
  const double passes = static_cast<double>((M + 15) / 16);
  const double skinny_us = 4.0 + passes * (0.5 + static_cast<double>(N) * static_cast<double>(K) / 5.2e6);
  // The tiled kernels, with weights that come from HBM (measured with rotating weights, 32 rows: K 4096 35 us
  // whatever N up to 14336; K 8192, N 28672 71 us; K 4096, N 131072 148 us): about 0.95 us per 128-wide K slab
  // and round of two tiles per CU, and never faster than about 3.8 bytes/ns of weights.
  const double rounds = tiles128 <= 512 ? 1.0 : static_cast<double>(tiles128) / 512.0;
  const double slab_us = 0.95 * static_cast<double>(K / 128) * rounds;
  const double read_us = static_cast<double>(N) * static_cast<double>(K) / 3.8e6;
  const double tiled_us = 5.0 + (slab_us > read_us ? slab_us : read_us);
  if (M <= 16) {
    // One pass either way.  From about 100 MB of weights on, while one or two rounds of 64-column workgroups
    // cover N, the one-tile-row kernel streams them faster (16 rows, K 8192, N 28672: 47.4 against 53.0 us, the
    // rate of a plain device copy; K 4096, N 28672: 27.3 against 30.2 us); with more rounds it falls behind
    // (K 8192, N 57344: 126 against 100 us).
    return !(one_tile_row && N * K >= (int64_t{96} << 20) && N <= 32768);
  }
  if (M <= 32 && one_tile_row) {
    // The one-tile-row kernel is there for this call (qgemm_impl checks what it needs).  With 32 rows and
    // 64-column workgroups it was measured, weights from HBM, at K 4096, N 4096 / 14336 / 28672: 14.2 / 17.5 /
    // 29.5 us; K 8192, N 8192 / 28672: 23.9 / 51.8 us; K 2048, N 8192: 9.7 us (the two passes of the
    // weight-streaming kernel: 11.3 / 25.9 / 30.0, 33.4 / 54.1, 9.7 us): 0.29 us per slab of K while the
    // workgroups are few, 4.8 bytes/ns of weights once they fill the chip.
    // Single-wavefront workgroups (N up to 8192): 0.26 us per slab (K 4096, N 4096 / 6144: 13.1 / 13.0 us,
    // K 8192, N 8192: 22.2 us, K 14336, N 4096: 34.6 us against 11.6 / 14.5, 23.9, 28.9 us).
    const double slabs_us = (N <= 8192 ? 0.26 : 0.29) * static_cast<double>(K / 128);
    const double bytes_us = static_cast<double>(N) * static_cast<double>(K) / 4.8e6;
    return skinny_us < 5.0 + (slabs_us > bytes_us ? slabs_us : bytes_us);
  }
  if (M <= 64 && one_tile_row) {
    // 33 to 64 rows, the same comparison: 0.34 us per slab (K 4096 / 8192 / 14336, N 4096: 16.6 / 27.4 / 44.1
    // us, where three or four passes of the weight-streaming kernel took 19.6 / 31.9 / 52.6 us), 4 bytes/ns.
    const double slabs_us = 0.34 * static_cast<double>(K / 128);
    const double bytes_us = static_cast<double>(N) * static_cast<double>(K) / 4.0e6;
    return skinny_us < 5.8 + (slabs_us > bytes_us ? slabs_us : bytes_us);
  }
  if (M <= 32) return skinny_us < tiled_us;
  // more rows: against the tiled kernel this shape would get (64 x 64 tiles with four stages on small problems:
  // 256 rows over K 8192 against 1024 columns take 22 us there, 30.6 us in sixteen passes of the weight-streaming kernel)
  return M <= 256 && tiles128 <= 256 && skinny_us < tiled_model_us(M, N, K);
}

// Number of K ranges worth cutting the problem into (0: do not split).  Model, in microseconds, fitted to
// measurements (256 x 4096 x 1024: 21.6 unsplit, 15.4 in 8 ranges; 256 x 8192 x 2048: 39.4 and 21.1): a
// 128-wide K slab takes about 0.55, the two launches 9 together, and the partial tiles travel to the
// workspace and back at about 4 bytes/ns.  Splitting has to win by 15 % to be chosen.
static int splitk_plan(int64_t M, int64_t N, int64_t K, double other_us) {
  if (K % 128 != 0 || M <= 32) return 0;
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128), slabs = K / 128;
  if (tiles > 128 || slabs < 8) return 0;
  int best = 0;
  double best_us = 1e30;
  for (int s = 2; s <= 16 && s * 2 <= slabs && tiles * s <= 512; s *= 2) {
    const double per = static_cast<double>((slabs + s - 1) / s);
    const double waves = static_cast<double>((tiles * s + 255) / 256);
    const double us = 9.0 + 0.55 * per * waves + static_cast<double>(s) * M * N * 8.0 / 4.0e6;
    if (us < 0.85 * other_us && us < best_us) {
      best_us = us;
      best = s;
    }
  }
  return best;
}

template <int QT>
static int launch_splitk(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K, int splits,
                         const Epilogue& ep, void* out, int64_t ldo, void* ws, hipStream_t st) {
  constexpr size_t smem = 2 * (128 + 128) * 128;
  auto kern = qgemm_splitk_kernel<QT>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128), slabs = K / 128;
  const int per = static_cast<int>((slabs + splits - 1) / splits);
  const int used = static_cast<int>((slabs + per - 1) / per);  // every range holds at least one slab
  kern<<<dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(used)), 256, smem, st>>>(
      static_cast<const uint8_t*>(a), lda, static_cast<const uint8_t*>(b), ldb, static_cast<int>(M), static_cast<int>(N),
      static_cast<int>(K), per, static_cast<uint8_t*>(ws));
  const int64_t threads = (M * N + 3) / 4;
  splitk_reduce_kernel<QT == QWIX_INT8><<<dim3(static_cast<unsigned>((threads + 255) / 256)), 256, 0, st>>>(
      static_cast<const uint8_t*>(ws), used, static_cast<int>(M), static_cast<int>(N), ep, static_cast<uint8_t*>(out), ldo);
  return check_launch("qgemm (split K)");
}

static int qgemm_impl(const void* a, int64_t lda, const void* b, int64_t ldb, int qtype, int64_t M, int64_t N, int64_t K,
                      const void* sa, int sa_dtype, const void* sb, int sb_dtype, int acc_dtype, const int32_t* zu,
                      const int32_t* zv, void* out, int out_dtype, int64_t ldo, void* stream, void* workspace,
                      size_t workspace_bytes) {
  if (const int rc = check_gemm_args(a, lda, b, ldb, qtype, M, N, K, sa, sa_dtype, sb, sb_dtype, acc_dtype, out,
                                     out_dtype, ldo))
    return rc;
  const Epilogue ep = make_epilogue(qtype, sa, sa_dtype, sb, sb_dtype, acc_dtype, zu, zv, out_dtype);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Few rows: stream the weights instead of tiling.  Up to 16 rows always; up to 256 rows while a rough cost
  // model favours it (streams_weights): the skinny kernel makes one pass over the weights per 16 rows (about
  // 0.5 us + 5.2 bytes/ns each) after a 4 us start; the tiled kernels walk K in 128-wide slabs after 5 us,
  // however few of the chip's CUs their 128 x 128 tiles occupy.
  const double tiled_us = tiled_model_us(M, N, K);
  // what the one-tile-row kernel (launch_mid) needs
  // (65 to 128 rows: one workgroup per CU for its 96 or 128 KB of LDS stages, so only while one round of
  // workgroups covers N: 64-column ones up to N 16384, 128-column ones up to N 32768.  Measured against the
  // 128 x 128 tile, int8, weights from HBM, K 4096, N 4096 / 14336: 25.9 / 29.3 against 37.1 / 38.7 us; K 8192,
  // N 8192: 43.1 against 67.7 us; K 8192, N 28672: 68.9 against 77.0 us with 128-column workgroups, 90.4 with
  // two rounds of 64-column ones.)
  // 129 to 256 rows, N up to 8192: two tile rows of 128 side by side (four stages, two workgroups per CU) where
  // the 128 x 128 tiles would occupy a quarter of the chip: 256 rows, K 4096, N 4096: 24.6 against 36.5 us;
  // K 8192, N 8192: 43.8 against 65.0 us; K 14336, N 4096: 67.3 against 112.8 us; no gain from N 14336 on.
  const bool mid_ok = (M > 16 || (N * K >= (int64_t{96} << 20) && N <= 32768)) && (M <= 64 || (M <= 128 && (N + 127) / 128 <= 256) ||
                                 (M <= 256 && (N + 63) / 64 <= 128)) && K % 128 == 0 && out_dtype != QWIX_I32 &&
                      (zu == nullptr || qtype == QWIX_INT8) &&
                      N * K >= (int64_t{8} << 20) && M * lda < (int64_t{1} << 31) && N * ldb < (int64_t{1} << 31);
  const bool few_rows = streams_weights(M, N, K, mid_ok);
  const bool off31 = M * lda < (int64_t{1} << 31) && N * ldb < (int64_t{1} << 31);
  if (workspace != nullptr && zu == nullptr && out_dtype != QWIX_I32 && off31) {
    // only against the tiled kernels: where the weight-streaming kernel is chosen its own model has spoken
    const int splits = few_rows ? 0 : splitk_plan(M, N, K, tiled_us);
    if (splits > 0 && workspace_bytes >= static_cast<size_t>(splits) * M * N * 4 && aligned16(workspace)) {
      if (qtype == QWIX_INT8) return launch_splitk<QWIX_INT8>(a, lda, b, ldb, M, N, K, splits, ep, out, ldo, workspace, st);
      return launch_splitk<QWIX_E4M3>(a, lda, b, ldb, M, N, K, splits, ep, out, ldo, workspace, st);
    }
  }
  if (few_rows && K % 128 == 0 && M * lda < (int64_t{1} << 31) && 64 * ldb < (int64_t{1} << 31)) {
    if (qtype == QWIX_INT8) return launch_skinny<QWIX_INT8>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    return launch_skinny<QWIX_E4M3>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  }
  // 256 x 256 tiles once they fill most of the chip's 256 CUs; smaller problems use 128 x 128 tiles.
  const bool big = ((M + 255) / 256) * ((N + 255) / 256) >= 192;
  const bool off32 = M * lda < (int64_t{1} << 31) && N * ldb < (int64_t{1} << 31);  // 32-bit lane offsets
  if (K % 128 == 0 && off32) {  // direct-to-LDS pipeline
    // long K on a full chip: the ping-pong schedule (no raw-accumulator variant of it exists)
    if (big && K >= 256 && out_dtype != QWIX_I32) {
      if (qtype == QWIX_INT8) return dispatch_pp<QWIX_INT8>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      return dispatch_pp<QWIX_E4M3>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    }
    // 64 x 64 tiles with four slab stages, at most two per CU
    const bool small_deep = ((M + 127) / 128) * ((N + 127) / 128) <= kSmallTiles && ((M + 63) / 64) * ((N + 63) / 64) <= 512;
    // From 64 rows on those tiles take the shapes of the one-tile-row kernel faster (weights from HBM, 100 rows: K 4096,
    // N 4096 23.5 -> 12.9 us, K 14336, N 4096 68.3 -> 36.2, K 8192, N 8192 41.8 -> 23.5; 64 rows: 14.6 -> 13.2, 41.0 ->
    // 37.9, 25.5 -> 24.3; 256 rows, K 4096, N 4096: 22.5 -> 13.4; level at 48 rows, behind below).  Where they do not
    // apply (N 28672: 224 tiles of 128 x 128) the one-tile-row kernel stays ahead of 128 x 128 tiles (28.6 against 39.3 us
    // at 64 rows).
    if (mid_ok && !(small_deep && M >= 64)) {
      // up to 64 rows against a weight of megabytes (and too many rows, or too large a weight, for the
      // weight-streaming kernel): the tile that keeps three slabs of weights in flight per wavefront
      if (qtype == QWIX_INT8 && zu != nullptr) {  // zero-point correction in the epilogue
        if (out_dtype == QWIX_BF16) return launch_mid<QWIX_INT8, QWIX_BF16, 3>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
        return launch_mid<QWIX_INT8, QWIX_F32, 3>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      }
      // (the epilogue's rounding flags at compile time in the common case: bf16 scales, bf16 result)
      const bool all_round = ep.r0 && ep.r1 && ep.r2;
      if (qtype == QWIX_INT8) {
        if (out_dtype == QWIX_BF16 && all_round) return launch_mid<QWIX_INT8, QWIX_BF16, 1>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
        if (out_dtype == QWIX_BF16) return launch_mid<QWIX_INT8, QWIX_BF16>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
        return launch_mid<QWIX_INT8, QWIX_F32>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      }
      if (out_dtype == QWIX_BF16 && all_round) return launch_mid<QWIX_E4M3, QWIX_BF16, 1>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      if (out_dtype == QWIX_BF16) return launch_mid<QWIX_E4M3, QWIX_BF16>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      return launch_mid<QWIX_E4M3, QWIX_F32>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    }
    // 128 x 128 tiles that would occupy less than a third of the chip: 64 x 64 tiles, four times as many workgroups
    // (a layer of 256 tokens x 4096 features over K 1024 is 64 tiles of 128 x 128)
    const bool small = ((M + 127) / 128) * ((N + 127) / 128) <= kSmallTiles;
    // four slab stages (64 KB) while the 64 x 64 tiles are at most two per CU: weights from HBM, 256 x 1024 over
    // K 4096 21.8 -> 12.7 us, 512 x 512 over K 8192 40.7 -> 21.8, 512 x 4096 over K 4096 26.8 -> 21.0; with 768 tiles
    // (1536 x 2048 over K 2048) 14.6 -> 17.1 us, so those keep two stages
    const bool deep = ((M + 63) / 64) * ((N + 63) / 64) <= 512;
    // 128 x 128 tiles that are at most one per CU: three slab stages (96 KB).  Weights from HBM, 256 tiles: 1024 x 4096
    // over K 4096 34.8 -> 25.3 us, 2048 x 2048 over K 4096 31.8 -> 26.4, over K 1024 12.5 -> 11.3; with two tiles per CU
    // (512 tiles) the second workgroup hides more than the third stage does (4096 x 2048 over K 1024: 14.2 against 20.0 us)
    const bool one_round = ((M + 127) / 128) * ((N + 127) / 128) <= 256;
    if (qtype == QWIX_INT8) {
      if (big) return dispatch_dma<QWIX_INT8, 256, 256, 2, 4>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      if (small && deep) return dispatch_dma<QWIX_INT8, 64, 64, 2, 2, 4>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      if (small) return dispatch_dma<QWIX_INT8, 64, 64, 2, 2>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      if (one_round) return dispatch_dma<QWIX_INT8, 128, 128, 2, 2, 3>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
      return dispatch_dma<QWIX_INT8, 128, 128, 2, 2>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    }
    if (big) return dispatch_dma<QWIX_E4M3, 256, 256, 2, 4>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    if (small && deep) return dispatch_dma<QWIX_E4M3, 64, 64, 2, 2, 4>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    if (small) return dispatch_dma<QWIX_E4M3, 64, 64, 2, 2>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    if (one_round) return dispatch_dma<QWIX_E4M3, 128, 128, 2, 2, 3>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
    return dispatch_dma<QWIX_E4M3, 128, 128, 2, 2>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  }
  // register-staged kernel: any K that is a multiple of 16
  if (qtype == QWIX_INT8) return launch_qgemm<QWIX_INT8, 128, 128, 128>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
  return launch_qgemm<QWIX_E4M3, 128, 128, 128>(a, lda, b, ldb, M, N, K, ep, out, ldo, st);
}
