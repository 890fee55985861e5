// Fast Walsh-Hadamard transform along rows, optionally fused with absmax quantization.
//
//   y[r, :] = ((x[r, :] * pre_sign) H_n) * post_sign * out_scale,   H_n Sylvester / natural order
//
// One workgroup per row.  The row is held in LDS as f32 (index i lives at i + i/8, which keeps the
// strided butterfly accesses spread over the banks); log2(n) butterfly stages run three at a time
// in registers (radix 8), so a row of 8192 makes 5 trips through LDS instead of 13.  All sums are
// f32; the result is rounded once to the array dtype, exactly where the reference rounds the
// output of its dense x @ H.  In the fused variant the rounded row is then quantized in place:
// absmax per row or per group, scale, divide, round, pack -- only qvalues and scales reach HBM.
#include "common.h"

namespace qwix {
namespace {

__device__ __forceinline__ int padi(int i) { return i + (i >> 3); }

template <int R>
__device__ __forceinline__ void radix_pass(float* buf, int n, int b, int tid) {
  const int groups = n >> R;
  for (int gid = tid; gid < groups; gid += 256) {
    const int low = gid & ((1 << b) - 1);
    const int i0 = ((gid >> b) << (b + R)) | low;
    float v[1 << R];
#pragma unroll
    for (int j = 0; j < (1 << R); ++j) v[j] = buf[padi(i0 + (j << b))];
#pragma unroll
    for (int s = 0; s < R; ++s) {
#pragma unroll
      for (int j = 0; j < (1 << R); ++j) {
        if ((j & (1 << s)) == 0) {
          const float a = v[j], c = v[j | (1 << s)];
          v[j] = a + c;
          v[j | (1 << s)] = a - c;
        }
      }
    }
#pragma unroll
    for (int j = 0; j < (1 << R); ++j) buf[padi(i0 + (j << b))] = v[j];
  }
}

// MODE 0: write y (dtype D).  MODE 1: quantize to QT with absmax over `tile` elements.
template <typename D, int MODE, int QT>
__global__ void __launch_bounds__(256)
    fwht_kernel(const void* __restrict__ x, int n, int logn, const void* __restrict__ pre,
                const void* __restrict__ post, float out_scale, int tile, void* __restrict__ y,
                void* __restrict__ scale) {
  extern __shared__ float buf[];
  __shared__ float red[4];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const int64_t base = row * n;

  for (int i = tid; i < n; i += 256) {
    float v = load1<D>(x, base + i);
    if (pre != nullptr) v *= load1<D>(pre, i);
    buf[padi(i)] = v;
  }
  __syncthreads();
  for (int b = 0; b < logn; b += 3) {
    const int r = min(3, logn - b);
    if (r == 3) radix_pass<3>(buf, n, b, tid);
    else if (r == 2) radix_pass<2>(buf, n, b, tid);
    else radix_pass<1>(buf, n, b, tid);
    __syncthreads();
  }

  auto finish = [&](int i) {
    float v = buf[padi(i)];
    if (post != nullptr) v *= load1<D>(post, i);
    v = rnd<D>(v);
    if (out_scale != 1.0f) v = rnd<D>(v * out_scale);
    return v;
  };

  if constexpr (MODE == 0) {
    for (int i = tid; i < n; i += 256) store1<D>(y, base + i, finish(i));
  } else {
    // chunks of 8 consecutive elements; chunk c -> group (8c / tile).
    const int chunks = n >> 3, cps = tile >> 3;  // chunks per scale group
    uint8_t* q = static_cast<uint8_t*>(y);
    float row_am = 0.f;
    if (cps > 64) {  // tile == n: the whole row shares one scale
      for (int cc = tid; cc < chunks; cc += 256) {
#pragma unroll
        for (int e = 0; e < 8; ++e) row_am = absmax_acc(row_am, finish(8 * cc + e));
      }
      row_am = wave_xor_max(row_am, 64);
      if ((tid & 63) == 0) red[tid >> 6] = row_am;
      __syncthreads();
      row_am = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    }
    for (int c0 = 0; c0 < chunks; c0 += 256) {
      const int c = c0 + tid;
      float v[8];
      float am = 0.f;
      if (c < chunks) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[e] = finish(8 * c + e);
          am = absmax_acc(am, v[e]);
        }
      }
      am = (cps <= 64) ? wave_xor_max(am, cps) : row_am;
      const float s = sym_scale<D, QT>(am);
      if (c < chunks) {
        const int64_t g = (static_cast<int64_t>(row) * n + 8 * c) / tile;
        if (cps > 64 ? (c == 0) : ((c % cps) == 0)) store1<D>(scale, g, s);
        const Divider<D, false> div(s);
        float t[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] = div(v[e]);
        // store_q equivalent for 8 values
        if constexpr (QT == QWIX_INT4) {
          uint32_t w = 0;
#pragma unroll
          for (int e = 0; e < 8; ++e) w |= static_cast<uint32_t>(to_int_q<QT>(t[e]) & 0xF) << (4 * e);
          *reinterpret_cast<uint32_t*>(q + (base + 8 * c) / 2) = w;
        } else if constexpr (QT == QWIX_INT8) {
          *reinterpret_cast<uint2*>(q + base + 8 * c) =
              make_uint2(pack4_i8(to_int_q<QT>(t[0]), to_int_q<QT>(t[1]), to_int_q<QT>(t[2]), to_int_q<QT>(t[3])),
                         pack4_i8(to_int_q<QT>(t[4]), to_int_q<QT>(t[5]), to_int_q<QT>(t[6]), to_int_q<QT>(t[7])));
        } else {
          *reinterpret_cast<uint2*>(q + base + 8 * c) =
              make_uint2(to_e4m3x2(t[0], t[1]) | (to_e4m3x2(t[2], t[3]) << 16),
                         to_e4m3x2(t[4], t[5]) | (to_e4m3x2(t[6], t[7]) << 16));
        }
      }
    }
  }
}

int check_fwht(const void* x, int64_t rows, int64_t n, int* logn) {
  if (!x || rows <= 0 || n < 2 || n > 16384) return fail(QWIX_ERR_INVALID_ARGUMENT, "fwht needs 2 <= n <= 16384 (n=%lld)", (long long)n);
  int l = 0;
  while ((int64_t{1} << l) < n) ++l;
  if ((int64_t{1} << l) != n)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "Expected reduction dimension size to be a power of 2, but got %lld", (long long)n);
  if (rows > INT32_MAX) return fail(QWIX_ERR_INVALID_ARGUMENT, "too many rows");
  *logn = l;
  return QWIX_OK;
}

template <typename K>
int set_smem(K kern, size_t smem) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     static_cast<int>(smem));
  if (e != hipSuccess) return fail(QWIX_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  return QWIX_OK;
}

}  // namespace
}  // namespace qwix

using namespace qwix;

extern "C" int qwix_hip_fwht(const void* x, int dtype, int64_t rows, int64_t n, const void* pre_sign,
                             const void* post_sign, float out_scale, void* y, void* stream) {
  int logn;
  if (int e = check_fwht(x, rows, n, &logn)) return e;
  if (!y) return fail(QWIX_ERR_INVALID_ARGUMENT, "null output");
  const size_t smem = static_cast<size_t>(n + n / 8 + 8) * sizeof(float);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == QWIX_BF16) {
    auto k = fwht_kernel<BF16, 0, QWIX_INT8>;
    if (int e = set_smem(k, smem)) return e;
    k<<<dim3(static_cast<unsigned>(rows)), 256, smem, st>>>(x, static_cast<int>(n), logn, pre_sign, post_sign, out_scale, 0, y, nullptr);
  } else if (dtype == QWIX_F32) {
    auto k = fwht_kernel<F32, 0, QWIX_INT8>;
    if (int e = set_smem(k, smem)) return e;
    k<<<dim3(static_cast<unsigned>(rows)), 256, smem, st>>>(x, static_cast<int>(n), logn, pre_sign, post_sign, out_scale, 0, y, nullptr);
  } else {
    return fail(QWIX_ERR_INVALID_ARGUMENT, "dtype %d is not f32/bf16", dtype);
  }
  return check_launch("fwht");
}

extern "C" int qwix_hip_fwht_quantize(const void* x, int dtype, int64_t rows, int64_t n, const void* pre_sign,
                                      const void* post_sign, float out_scale, int64_t tile, int qtype, void* qvalue,
                                      void* scale, void* stream) {
  int logn;
  if (int e = check_fwht(x, rows, n, &logn)) return e;
  if (!qvalue || !scale) return fail(QWIX_ERR_INVALID_ARGUMENT, "null output");
  if (n < 8 || tile < 8 || n % tile || (tile & (tile - 1)) || !(tile == n || tile <= 512))
    return fail(QWIX_ERR_UNSUPPORTED, "fused fwht+quantize needs n >= 8 and a power-of-two tile that is n or <= 512 "
                "(n=%lld tile=%lld); run qwix_hip_fwht then qwix_hip_quantize instead", (long long)n, (long long)tile);
  if (!aligned16(qvalue)) return fail(QWIX_ERR_INVALID_ARGUMENT, "qvalue must be 16-byte aligned");
  const size_t smem = static_cast<size_t>(n + n / 8 + 8) * sizeof(float);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(rows));
#define QWIX_FWHT_Q(DT, QT)                                                                                      \
  {                                                                                                                \
    auto k = fwht_kernel<DT, 1, QT>;                                                                               \
    if (int e = set_smem(k, smem)) return e;                                                                       \
    k<<<grid, 256, smem, st>>>(x, static_cast<int>(n), logn, pre_sign, post_sign, out_scale, static_cast<int>(tile), \
                               qvalue, scale);                                                                     \
  }
  if (dtype == QWIX_BF16) {
    if (qtype == QWIX_INT8) QWIX_FWHT_Q(BF16, QWIX_INT8)
    else if (qtype == QWIX_INT4) QWIX_FWHT_Q(BF16, QWIX_INT4)
    else if (qtype == QWIX_E4M3) QWIX_FWHT_Q(BF16, QWIX_E4M3)
    else return fail(QWIX_ERR_INVALID_ARGUMENT, "unknown qtype %d", qtype);
  } else if (dtype == QWIX_F32) {
    if (qtype == QWIX_INT8) QWIX_FWHT_Q(F32, QWIX_INT8)
    else if (qtype == QWIX_INT4) QWIX_FWHT_Q(F32, QWIX_INT4)
    else if (qtype == QWIX_E4M3) QWIX_FWHT_Q(F32, QWIX_E4M3)
    else return fail(QWIX_ERR_INVALID_ARGUMENT, "unknown qtype %d", qtype);
  } else {
    return fail(QWIX_ERR_INVALID_ARGUMENT, "dtype %d is not f32/bf16", dtype);
  }
#undef QWIX_FWHT_Q
  return check_launch("fwht_quantize");
}
