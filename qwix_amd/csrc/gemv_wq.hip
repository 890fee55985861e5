// Weight-only skinny GEMM (decode): bf16 activations x int4/int8 group-quantized weights.
//
//   out[m,n] = sum_g s[g,n] * sum_{k in g} x[m,k] * q[n,k]         M small (16 rows per pass)
//
// HBM-bound: the weight bytes are read exactly once, the activations stay in L2.  Even at M = 16
// the multiply-adds exceed what the vector ALUs can do in the time the weights stream in, so the
// products run on v_mfma_f32_16x16x32_bf16 with the weights converted to bf16 in registers:
//   int4: (nibble ^ 8) is OR-ed into the mantissa of bf16 128.0, giving 128 + (q + 8) exactly in
//         two bit-ops per pair; the offset is removed after the MFMA with the row sums of x, which
//         a second MFMA against an all-ones operand produces in the accumulator's own layout;
//   int8: sign-extend, convert, pack.
// A workgroup is 4 wavefronts that split K; each handles NT tiles of 16 output columns and the
// four partial sums meet in LDS.
#include "common.h"

namespace qwix {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

constexpr int NT = 2;

struct GemvArgs {
  const uint16_t* x; int64_t ldx;
  const uint8_t* q; int64_t ldb;
  int M, N, K, group;
  const void* s; int s_dtype;
  void* out; int out_dtype; int64_t ldo;
};

__device__ __forceinline__ bf16x8 as_bf16x8(v4u v) { return __builtin_bit_cast(bf16x8, v); }

template <int BQT>
__global__ void __launch_bounds__(256) gemv_wq_kernel(GemvArgs p) {
  constexpr bool W4 = (BQT == QWIX_INT4);
  __shared__ float red[4][NT][4][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, kq = lane >> 4;
  const int n_base = blockIdx.x * (16 * NT);
  const int m = blockIdx.y * 16 + col;  // row of x this lane feeds to the MFMA
  const int nblk = p.K / 128;
  const int per_wave = (nblk + 3) / 4;
  const int kb0 = wave * per_wave, kb1 = min(nblk, kb0 + per_wave);

  v4f outacc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) outacc[t] = v4f{0.f, 0.f, 0.f, 0.f};
  const v4u ones_u = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};

  for (int kb = kb0; kb < kb1; ++kb) {
    const int k0 = kb * 128 + kq * 32;
    // Four activation fragments of 8 consecutive k each.
    v4u xf[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      xf[j] = v4u{0, 0, 0, 0};
      if (m < p.M) xf[j] = *reinterpret_cast<const v4u*>(p.x + static_cast<int64_t>(m) * p.ldx + k0 + j * 8);
      if constexpr (W4) {  // element order (k0,k4,k1,k5,k2,k6,k3,k7): what the nibble widening yields
        const v4u d = xf[j];
        xf[j][0] = __builtin_amdgcn_perm(d[2], d[0], 0x05040100);
        xf[j][1] = __builtin_amdgcn_perm(d[2], d[0], 0x07060302);
        xf[j][2] = __builtin_amdgcn_perm(d[3], d[1], 0x05040100);
        xf[j][3] = __builtin_amdgcn_perm(d[3], d[1], 0x07060302);
      }
    }
    v4f rowsum = {0.f, 0.f, 0.f, 0.f};
    if constexpr (W4) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        rowsum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xf[j]), as_bf16x8(ones_u), rowsum, 0, 0, 0);
    }
    const int sg = (kb * 128) / p.group;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = n_base + t * 16 + col;
      v4f acc = {0.f, 0.f, 0.f, 0.f};
      float sc = 0.f;
      if (n < p.N) {
        sc = p.s_dtype == QWIX_BF16
                 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.s)[static_cast<int64_t>(sg) * p.N + n])
                 : reinterpret_cast<const float*>(p.s)[static_cast<int64_t>(sg) * p.N + n];
      }
      if constexpr (W4) {
        v4u pk = {0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u};  // zeros in two's complement
        if (n < p.N) pk = *reinterpret_cast<const v4u*>(p.q + static_cast<int64_t>(n) * p.ldb + k0 / 2);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const unsigned u = pk[j] ^ 0x88888888u;  // offset binary: nibble = q + 8
          v4u w;
          w[0] = (u & 0x000F000Fu) | 0x43004300u;          // (k0, k4) as bf16 128 + nibble
          w[1] = ((u >> 4) & 0x000F000Fu) | 0x43004300u;   // (k1, k5)
          w[2] = ((u >> 8) & 0x000F000Fu) | 0x43004300u;   // (k2, k6)
          w[3] = ((u >> 12) & 0x000F000Fu) | 0x43004300u;  // (k3, k7)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xf[j]), as_bf16x8(w), acc, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) outacc[t][r] += (acc[r] - 136.f * rowsum[r]) * sc;
      } else {
        v4u lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
        if (n < p.N) {
          lo = *reinterpret_cast<const v4u*>(p.q + static_cast<int64_t>(n) * p.ldb + k0);
          hi = *reinterpret_cast<const v4u*>(p.q + static_cast<int64_t>(n) * p.ldb + k0 + 16);
        }
        const unsigned words[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v4u w;
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const unsigned d = words[2 * j + h];
            const float f0 = static_cast<float>(static_cast<int>(d << 24) >> 24);
            const float f1 = static_cast<float>(static_cast<int>(d << 16) >> 24);
            const float f2 = static_cast<float>(static_cast<int>(d << 8) >> 24);
            const float f3 = static_cast<float>(static_cast<int>(d) >> 24);
            w[2 * h] = f32_to_bf16_bits(f0) | (static_cast<unsigned>(f32_to_bf16_bits(f1)) << 16);
            w[2 * h + 1] = f32_to_bf16_bits(f2) | (static_cast<unsigned>(f32_to_bf16_bits(f3)) << 16);
          }
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(xf[j]), as_bf16x8(w), acc, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) outacc[t][r] += acc[r] * sc;
      }
    }
  }

#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][t][r][lane] = outacc[t][r];
  __syncthreads();
  // result lane layout: column n = lane % 16, row m = 4 * (lane / 16) + r
  for (int idx = tid; idx < NT * 256; idx += 256) {
    const int t = idx >> 8, r = (idx >> 6) & 3, l = idx & 63;
    const float v = red[0][t][r][l] + red[1][t][r][l] + red[2][t][r][l] + red[3][t][r][l];
    const int mo = blockIdx.y * 16 + 4 * (l >> 4) + r, n = n_base + t * 16 + (l & 15);
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
  GemvArgs p;
  p.x = static_cast<const uint16_t*>(x); p.ldx = ldx;
  p.q = static_cast<const uint8_t*>(q); p.ldb = ldb_bytes;
  p.M = static_cast<int>(M); p.N = static_cast<int>(N); p.K = static_cast<int>(K); p.group = static_cast<int>(group);
  p.s = s; p.s_dtype = s_dtype;
  p.out = out; p.out_dtype = out_dtype; p.ldo = ldo;
  const dim3 grid(static_cast<unsigned>((N + 16 * NT - 1) / (16 * NT)), static_cast<unsigned>((M + 15) / 16));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (b_qtype == QWIX_INT4)
    gemv_wq_kernel<QWIX_INT4><<<grid, 256, 0, st>>>(p);
  else
    gemv_wq_kernel<QWIX_INT8><<<grid, 256, 0, st>>>(p);
  return check_launch("gemv_wq");
}
