// What the matrix cores of the chip sustain with given operand BYTES and no memory traffic at all: the yardstick
// beside the nominal peak that the quantized GEMMs are priced against.
//
// One workgroup of 8 wavefronts per CU (two per SIMD, like the GEMM kernels).  Every lane loads four 16-byte "A"
// fragments and four 16-byte "B" fragments from the caller's operand arrays once, keeps them in registers, and then
// issues v_mfma_i32_32x32x32_i8 (or v_mfma_scale_f32_32x32x64_f8f6f4 with unit scales) back to back on eight
// accumulator tiles: per iteration 32 int8 MFMAs or 16 fp8 MFMAs, 2 097 152 operations per wavefront either way.
// The rate depends on the operand bytes: the matrix cores draw more power the more bits toggle in their multiplier
// arrays, and the board's power limit sets the clock.
#include "common.h"

namespace qwix {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kWorkgroups = 256, kThreads = 512;

template <bool FP8>
__global__ void __launch_bounds__(kThreads)
    mfma_ceiling_kernel(const uint8_t* __restrict__ a, uint32_t a_vecs, const uint8_t* __restrict__ b, uint32_t b_vecs,
                        int iters, int32_t* __restrict__ sink) {
  const uint32_t t = blockIdx.x * kThreads + threadIdx.x;
  v4i fa[4], fb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    fa[i] = *reinterpret_cast<const v4i*>(a + static_cast<size_t>((t * 4 + i) % a_vecs) * 16);
    fb[i] = *reinterpret_cast<const v4i*>(b + static_cast<size_t>((t * 4 + i) % b_vecs) * 16);
  }
  if constexpr (FP8) {
    v8i a8[2], b8[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      a8[i] = v8i{fa[2 * i][0], fa[2 * i][1], fa[2 * i][2], fa[2 * i][3], fa[2 * i + 1][0], fa[2 * i + 1][1], fa[2 * i + 1][2], fa[2 * i + 1][3]};
      b8[i] = v8i{fb[2 * i][0], fb[2 * i][1], fb[2 * i][2], fb[2 * i][3], fb[2 * i + 1][0], fb[2 * i + 1][1], fb[2 * i + 1][2], fb[2 * i + 1][3]};
    }
    v16f acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8[ks], b8[(ks + i) & 1], acc[i], 0, 0, 0, 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += acc[i][0];
    if (s == 12345.678f) sink[0] = 1;  // keeps the loop alive; practically never true
  } else {
    v16i acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][r] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks], fb[(ks + i) & 3], acc[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += acc[i][0];
    if (s == 0x7fffffff) sink[0] = s;
  }
}

}  // namespace
}  // namespace qwix

using namespace qwix;

extern "C" double qwix_hip_mfma_ceiling_ops(int64_t iters) {
  return static_cast<double>(kWorkgroups) * (kThreads / 64) * static_cast<double>(iters) * 32.0 * (2.0 * 32 * 32 * 32);
}

extern "C" int qwix_hip_mfma_ceiling(const void* a, size_t a_bytes, const void* b, size_t b_bytes, int qtype,
                                     int64_t iters, int32_t* sink, void* stream) {
  if (!a || !b || !sink) return fail(QWIX_ERR_INVALID_ARGUMENT, "null a/b/sink");
  if (qtype != QWIX_INT8 && qtype != QWIX_E4M3) return fail(QWIX_ERR_UNSUPPORTED, "qtype %d: int8 or e4m3", qtype);
  if (a_bytes < 16 || b_bytes < 16 || (a_bytes >> 4) > UINT32_MAX || (b_bytes >> 4) > UINT32_MAX || !aligned16(a) || !aligned16(b))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "operand arrays: 16-byte aligned, 16 bytes to 64 GiB");
  if (iters <= 0 || iters > INT32_MAX) return fail(QWIX_ERR_INVALID_ARGUMENT, "bad iteration count %lld", (long long)iters);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint32_t av = static_cast<uint32_t>(a_bytes >> 4), bv = static_cast<uint32_t>(b_bytes >> 4);
  if (qtype == QWIX_E4M3)
    mfma_ceiling_kernel<true><<<kWorkgroups, kThreads, 0, st>>>(static_cast<const uint8_t*>(a), av, static_cast<const uint8_t*>(b), bv,
                                                                static_cast<int>(iters), sink);
  else
    mfma_ceiling_kernel<false><<<kWorkgroups, kThreads, 0, st>>>(static_cast<const uint8_t*>(a), av, static_cast<const uint8_t*>(b), bv,
                                                                 static_cast<int>(iters), sink);
  return check_launch("mfma_ceiling");
}
