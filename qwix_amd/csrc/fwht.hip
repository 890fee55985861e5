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

// ------------------------------------------------------------------------------------------------
// Rows of 4096 / 8192 / 16384 elements: 32 elements per thread, n / 32 threads per row, and the
// log2(n) butterfly stages run in three register passes with only two trips through LDS.
//
//   pass 1  registers = index bits {0,1,2} and the two top bits; a thread loads 4 x 8 consecutive elements
//   pass 2  registers = index bits 3..7
//   pass 3  registers = the remaining bits 8..log2(n)-3, padded with the lowest index bits (which are
//           already transformed), so that a thread ends up with runs of 2, 4 or 8 consecutive elements
//
// Between passes the row is exchanged through LDS at address p + p/32, where p is a bit permutation
// of the element index with the writer's five low lane bits in p[0:4] and the reader's in p[5:9]:
// a writing half-wave covers 32 consecutive words, a reading half-wave 32 words of stride 33, both
// free of bank conflicts, and the register part of every address is a compile-time constant.
// All sums are f32 and the result is rounded once to the array dtype, as in the generic kernel.
template <int B>
struct RegFwht {
  static constexpr int kThreads = 1 << (B - 5);
  static constexpr int kAct3 = B - 10;      // butterfly bits of pass 3
  static constexpr int kPas = 5 - kAct3;    // low index bits that fill its registers
  static constexpr int kRun = 1 << kPas;    // consecutive elements a thread finishes with

  // element index from (thread, register) in each pass
  static __host__ __device__ constexpr int t1(int t) { return t << 3; }
  static __host__ __device__ constexpr int r1(int r) { return (r & 7) | ((r >> 3) << (B - 2)); }
  static __host__ __device__ constexpr int t2(int t) { return (t & 7) | ((t >> 3) << 8); }
  static __host__ __device__ constexpr int r2(int r) { return r << 3; }
  static __host__ __device__ constexpr int t3(int t) {
    return ((t & 31) << 3) | (((t >> 5) & ((1 << (3 - kPas)) - 1)) << kPas) | ((t >> (8 - kPas)) << (8 + kAct3));
  }
  static __host__ __device__ constexpr int r3(int r) { return (r & (kRun - 1)) | ((r >> kPas) << 8); }
  // LDS word address of element i in the two exchanges
  static __host__ __device__ constexpr int pad(int p) { return p + (p >> 5); }
  static __host__ __device__ constexpr int x1(int i) { return pad(((i >> 3) & 31) | ((i & 7) << 5) | (i & ~0xFF)); }
  static __host__ __device__ constexpr int x2(int i) {
    return pad((i & 7) | (((i >> 8) & 3) << 3) | (((i >> 3) & 31) << 5) | (i & ~0x3FF));
  }
};

template <int LO, int HI>
__device__ __forceinline__ void butterflies(float (&v)[32]) {
#pragma unroll
  for (int s = LO; s < HI; ++s)
#pragma unroll
    for (int j = 0; j < 32; ++j)
      if ((j & (1 << s)) == 0) {
        const float a = v[j], c = v[j | (1 << s)];
        v[j] = a + c;
        v[j | (1 << s)] = a - c;
      }
}

template <typename D>
__device__ __forceinline__ void load8(const void* p, int64_t i, float (&o)[8]) {
  if constexpr (D::kTag == QWIX_BF16) {
    const uint4 w = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p) + i);
    const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o[2 * e] = __uint_as_float(u[e] << 16);
      o[2 * e + 1] = __uint_as_float(u[e] & 0xFFFF0000u);
    }
  } else {
    const float4 a = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i);
    const float4 b = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i + 4);
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
}

template <int BYTES>
__device__ __forceinline__ void store_bytes(void* dst, const uint32_t (&w)[4]) {
  if constexpr (BYTES == 1) *reinterpret_cast<uint8_t*>(dst) = static_cast<uint8_t>(w[0]);
  else if constexpr (BYTES == 2) *reinterpret_cast<uint16_t*>(dst) = static_cast<uint16_t>(w[0]);
  else if constexpr (BYTES == 4) *reinterpret_cast<uint32_t*>(dst) = w[0];
  else if constexpr (BYTES == 8) nt_store8(reinterpret_cast<uint2*>(dst), make_uint2(w[0], w[1]));
  else {
    static_assert(BYTES % 16 == 0, "unsupported store width");
    nt_store16(reinterpret_cast<uint4*>(dst), make_uint4(w[0], w[1], w[2], w[3]));
  }
}

// Quantizes one run of consecutive finished elements with scale s and stores it.  |v| <= absmax, so
// the quotients are bounded and the two-op clamp-and-round converter applies.
template <typename D, int QT, int RUN>
__device__ __forceinline__ void quantize_run(const float* v, float s, uint8_t* q, int64_t i) {
  const Divider<D, false, QT == QWIX_E4M3> div(s);
  float t[RUN];
#pragma unroll
  for (int e = 0; e < RUN; ++e) t[e] = div(v[e]);
  uint32_t w[4] = {0, 0, 0, 0};
  if constexpr (QT == QWIX_INT4) {
#pragma unroll
    for (int e = 0; e < RUN; ++e) w[0] |= (rne_bits_clamped(t[e], -8.f, 7.f) & 0xFu) << (4 * e);
    store_bytes<RUN / 2>(q + i / 2, w);
  } else if constexpr (QT == QWIX_INT8) {
    if constexpr (RUN >= 4) {
#pragma unroll
      for (int e = 0; e < RUN; e += 4)
        w[e / 4] = pack4_low_bytes(rne_bits_clamped(t[e], -128.f, 127.f), rne_bits_clamped(t[e + 1], -128.f, 127.f),
                                   rne_bits_clamped(t[e + 2], -128.f, 127.f), rne_bits_clamped(t[e + 3], -128.f, 127.f));
    } else {
#pragma unroll
      for (int e = 0; e < RUN; ++e) w[0] |= (rne_bits_clamped(t[e], -128.f, 127.f) & 0xFFu) << (8 * e);
    }
    store_bytes<RUN>(q + i, w);
  } else {
#pragma unroll
    for (int e = 0; e < RUN; e += 2) w[e / 4] |= to_e4m3x2(t[e], t[e + 1]) << (16 * ((e >> 1) & 1));
    store_bytes<RUN>(q + i, w);
  }
}

// MODE 0: write y (dtype D).  MODE 1: quantize to QT with one absmax scale per 2^ltile elements
// (ltile == B: per row).
template <typename D, int MODE, int QT, int B>
__global__ void __launch_bounds__(RegFwht<B>::kThreads)
    fwht_reg_kernel(const void* __restrict__ x, const void* __restrict__ pre, const void* __restrict__ post,
                    float out_scale, int ltile, void* __restrict__ y, void* __restrict__ scale) {
  using P = RegFwht<B>;
  constexpr int n = 1 << B, NWAVE = P::kThreads / 64, RUN = P::kRun;
  extern __shared__ float buf[];
  __shared__ float red[NWAVE];
  const int tid = threadIdx.x;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * n;
  float v[32];

  // ---- pass 1
  {
    const int i0 = P::t1(tid);
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      float t[8];
      load8<D>(x, base + i0 + P::r1(8 * h), t);
      if (pre != nullptr) {
        float sg[8];
        load8<D>(pre, i0 + P::r1(8 * h), sg);
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] *= sg[e];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) v[8 * h + e] = t[e];
    }
    butterflies<0, 5>(v);
    float* w = buf + P::x1(i0);
#pragma unroll
    for (int r = 0; r < 32; ++r) w[P::x1(P::r1(r))] = v[r];
  }
  __syncthreads();
  // ---- pass 2
  {
    const int i0 = P::t2(tid);
    const float* rd = buf + P::x1(i0);
#pragma unroll
    for (int r = 0; r < 32; ++r) v[r] = rd[P::x1(P::r2(r))];
    butterflies<0, 5>(v);
    __syncthreads();  // every thread has read its part before the row is overwritten
    float* w = buf + P::x2(i0);
#pragma unroll
    for (int r = 0; r < 32; ++r) w[P::x2(P::r2(r))] = v[r];
  }
  __syncthreads();
  // ---- pass 3
  const int i3 = P::t3(tid);
  {
    const float* rd = buf + P::x2(i3);
#pragma unroll
    for (int r = 0; r < 32; ++r) v[r] = rd[P::x2(P::r3(r))];
    butterflies<P::kPas, 5>(v);
  }
  // ---- sign, rounding to the array dtype, scale
  constexpr int NRUN = 32 / RUN;
#pragma unroll
  for (int a = 0; a < NRUN; ++a) {
    const int i = i3 + P::r3(a * RUN);
#pragma unroll
    for (int e = 0; e < RUN; ++e) {
      float t = v[a * RUN + e];
      if (post != nullptr) t *= load1<D>(post, i + e);
      t = rnd<D>(t);
      if (out_scale != 1.0f) t = rnd<D>(t * out_scale);
      v[a * RUN + e] = t;
    }
  }
  if constexpr (MODE == 0) {
#pragma unroll
    for (int a = 0; a < NRUN; ++a) {
      const int64_t i = base + i3 + P::r3(a * RUN);
      if constexpr (D::kTag == QWIX_BF16) {
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < RUN; e += 2)
          w[e / 2] = f32_to_bf16_bits(v[a * RUN + e]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[a * RUN + e + 1])) << 16);
        store_bytes<RUN * 2>(reinterpret_cast<uint16_t*>(y) + i, w);
      } else {
#pragma unroll
        for (int e0 = 0; e0 < RUN; e0 += 4) {
          uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
          for (int e = 0; e < 4 && e0 + e < RUN; ++e) w[e] = __float_as_uint(v[a * RUN + e0 + e]);
          store_bytes<(RUN >= 4 ? 16 : RUN * 4)>(reinterpret_cast<float*>(y) + i + e0, w);
        }
      }
    }
  } else {
    uint8_t* q = static_cast<uint8_t*>(y);
    if (ltile == B) {
      float am = 0.f;
#pragma unroll
      for (int r = 0; r < 32; ++r) am = absmax_acc(am, v[r]);
      am = wave_xor_max(am, 64);
      if ((tid & 63) == 0) red[tid >> 6] = am;
      __syncthreads();
      am = red[0];
#pragma unroll
      for (int w = 1; w < NWAVE; ++w) am = fmaxf(am, red[w]);
      const float s = sym_scale<D, QT>(am);
      if (tid == 0) store1<D>(scale, blockIdx.x, s);
#pragma unroll
      for (int a = 0; a < NRUN; ++a) quantize_run<D, QT, RUN>(&v[a * RUN], s, q, base + i3 + P::r3(a * RUN));
    } else {
      // One LDS word per scale group, merged with integer atomic max: the bit patterns of
      // non-negative floats order like the floats, and a maximum does not depend on the order.
      unsigned* tmax = reinterpret_cast<unsigned*>(buf);
      __syncthreads();  // the row in LDS is no longer needed
      for (int i = tid; i < (n >> ltile); i += P::kThreads) tmax[i] = 0u;
      __syncthreads();
#pragma unroll
      for (int a = 0; a < NRUN; ++a) {
        float am = 0.f;
#pragma unroll
        for (int e = 0; e < RUN; ++e) am = absmax_acc(am, v[a * RUN + e]);
        atomicMax(&tmax[(i3 + P::r3(a * RUN)) >> ltile], __float_as_uint(am));
      }
      __syncthreads();
#pragma unroll
      for (int a = 0; a < NRUN; ++a) {
        const int i = i3 + P::r3(a * RUN);
        const float s = sym_scale<D, QT>(__uint_as_float(tmax[i >> ltile]));
        if ((i & ((1 << ltile) - 1)) == 0) store1<D>(scale, (base + i) >> ltile, s);
        quantize_run<D, QT, RUN>(&v[a * RUN], s, q, base + i);
      }
    }
  }
}

template <typename D, int MODE, int QT, int B>
int launch_fwht_reg(const void* x, int64_t rows, const void* pre, const void* post, float out_scale, int ltile,
                    void* y, void* scale, hipStream_t st) {
  constexpr int n = 1 << B;
  constexpr size_t smem = static_cast<size_t>(n + n / 32 + 32) * sizeof(float);
  auto kern = fwht_reg_kernel<D, MODE, QT, B>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  kern<<<dim3(static_cast<unsigned>(rows)), RegFwht<B>::kThreads, smem, st>>>(x, pre, post, out_scale, ltile, y, scale);
  return check_launch("fwht (register passes)");
}

template <typename D, int MODE, int QT>
int dispatch_fwht_reg(int logn, const void* x, int64_t rows, const void* pre, const void* post, float out_scale,
                      int ltile, void* y, void* scale, hipStream_t st) {
  switch (logn) {
    case 12: return launch_fwht_reg<D, MODE, QT, 12>(x, rows, pre, post, out_scale, ltile, y, scale, st);
    case 13: return launch_fwht_reg<D, MODE, QT, 13>(x, rows, pre, post, out_scale, ltile, y, scale, st);
    default: return launch_fwht_reg<D, MODE, QT, 14>(x, rows, pre, post, out_scale, ltile, y, scale, st);
  }
}

// The register-pass kernel reads and writes rows with 16-byte accesses.
inline bool reg_path_ok(int logn, const void* x, const void* pre, const void* y) {
  return logn >= 12 && logn <= 14 && aligned16(x) && aligned16(y) && (pre == nullptr || aligned16(pre));
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
  if (reg_path_ok(logn, x, pre_sign, y) && (dtype == QWIX_BF16 || dtype == QWIX_F32)) {
    if (dtype == QWIX_BF16)
      return dispatch_fwht_reg<BF16, 0, QWIX_INT8>(logn, x, rows, pre_sign, post_sign, out_scale, logn, y, nullptr, st);
    return dispatch_fwht_reg<F32, 0, QWIX_INT8>(logn, x, rows, pre_sign, post_sign, out_scale, logn, y, nullptr, st);
  }
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
  int ltile = 0;
  while ((int64_t{1} << ltile) < tile) ++ltile;
  if (reg_path_ok(logn, x, pre_sign, qvalue) && (dtype == QWIX_BF16 || dtype == QWIX_F32) &&
      (qtype == QWIX_INT8 || qtype == QWIX_INT4 || qtype == QWIX_E4M3)) {
#define QWIX_FWHT_R(DT, QT) return dispatch_fwht_reg<DT, 1, QT>(logn, x, rows, pre_sign, post_sign, out_scale, ltile, qvalue, scale, st)
    if (dtype == QWIX_BF16) {
      if (qtype == QWIX_INT8) QWIX_FWHT_R(BF16, QWIX_INT8);
      if (qtype == QWIX_INT4) QWIX_FWHT_R(BF16, QWIX_INT4);
      QWIX_FWHT_R(BF16, QWIX_E4M3);
    }
    if (qtype == QWIX_INT8) QWIX_FWHT_R(F32, QWIX_INT8);
    if (qtype == QWIX_INT4) QWIX_FWHT_R(F32, QWIX_INT4);
    QWIX_FWHT_R(F32, QWIX_E4M3);
#undef QWIX_FWHT_R
  }
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
