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
#include <algorithm>

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

// ------------------------------------------------------------------------------------------------
// bf16 rows of 8192 elements: seven of the thirteen butterfly levels on the matrix cores.
//
// H_8192 is a Kronecker product over the 13 index bits and the factors commute, so any seven bits may be transformed
// first, as one multiplication by H_128 = [(-1)^popcount(k & n)], and the other six by butterflies.  The first
// factor sees the bf16 inputs themselves: the products with +-1 are exact and v_mfma_f32_32x32x16_bf16 adds them in
// f32, which is what a butterfly network in f32 does too (sums of small integers stay exact either way).  One
// WAVEFRONT owns a row, 128 elements per lane, and nothing goes through LDS but the constant matrix:
//
//   element index bits   i[12:10] = j    i[9] = mb    i[8] = h    i[7:3] = ml    i[2:0] = e
//   load (mb, j)         lane l = 32 h + ml reads the 16 bytes at (j, mb, l): 1 KB contiguous per instruction
//   MFMA operand A       rows m = ml (two blocks mb), k = j + 8 h + 16 kk: the eight loads of a lane, transposed in
//                        registers (16-bit interleaves), give for each e the eight j of one k-step kk(e)
//   MFMA operand B       H_128 fragments (k-step, column block nb) from a table in LDS
//   MFMA result          lane l holds column n = (l & 31) + 32 nb of H_128's output, i.e. index bits
//                        i[12:10] = l[2:0], i[8] = l[3], i[2] = l[4], i[1:0] = nb, and rows m = 8 (r / 4) + 4 h + r % 4:
//                        i[4:3] = r[1:0], i[5] = h, i[7:6] = r[3:2], i[9] = mb
//   butterflies          over the six m bits: r[0..3] and mb inside the lane, h by one v_permlane32_swap per pair of
//                        registers (mb = 0, mb = 1), after which the lane half stands for i[9] and the pair for i[5]
//   finish               a lane ends with runs of four consecutive elements (i[1:0]); two rounds of v_permlane16_swap
//                        on the packed results (over i[3], then i[4]) turn them into runs of sixteen
//
// The sign vector in front of the transform is applied as an XOR of sign bits on the packed inputs.
struct HFragTable {
  uint32_t w[8 * 4 * 64 * 4];  // [k-step][column block][lane][4 dwords = 8 bf16]
};
constexpr HFragTable make_hfrag_table() {
  HFragTable t{};
  for (int kk = 0; kk < 8; ++kk)
    for (int nb = 0; nb < 4; ++nb)
      for (int l = 0; l < 64; ++l)
        for (int d = 0; d < 4; ++d) {
          uint32_t word = 0;
          for (int half = 0; half < 2; ++half) {
            const int k = 16 * kk + 8 * (l >> 5) + 2 * d + half, n = 32 * nb + (l & 31);
            int par = 0;
            for (int b = 0; b < 7; ++b) par ^= ((k & n) >> b) & 1;
            word |= static_cast<uint32_t>(par ? 0xBF80u : 0x3F80u) << (16 * half);
          }
          t.w[((kk * 4 + nb) * 64 + l) * 4 + d] = word;
        }
  return t;
}
__device__ const HFragTable kHFrag = make_hfrag_table();

typedef __bf16 fw_bf16x8 __attribute__((ext_vector_type(8)));
typedef float fw_v16f __attribute__((ext_vector_type(16)));
typedef int fw_v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t dword_of(const uint4& v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }

// Swaps A's lanes 16-31 / 48-63 with B's lanes 0-15 / 32-47.
__device__ __forceinline__ void swap_rows16(uint32_t& a, uint32_t& b) {
  const auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
  a = r[0];
  b = r[1];
}

// MODE 0: write y (bf16).  MODE 1: quantize to QT, one absmax scale per 2^ltile elements (ltile == 13: per row).
template <int MODE, int QT, bool PRE, bool POST>
__global__ void __launch_bounds__(512)
    fwht_mfma_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ pre, const uint16_t* __restrict__ post,
                     float out_scale, int ltile, int rows, void* __restrict__ y, void* __restrict__ scale) {
  constexpr int B = 13, n = 1 << B;
  constexpr int EB = (MODE == 0) ? 16 : (QT == QWIX_INT4 ? 4 : 8);  // bits per stored element
  constexpr int ROW_BYTES = n * EB / 8;
  extern __shared__ __attribute__((aligned(1024))) uint8_t fw_smem[];
  uint32_t* htab = reinterpret_cast<uint32_t*>(fw_smem);                  // 32 KB: the H_128 fragments
  uint8_t* stage = fw_smem + 32768 + (threadIdx.x >> 6) * ROW_BYTES;      // this wavefront's finished row
  const int tid = threadIdx.x;
  const int nwaves = gridDim.x * 8;

  uint4 raw[2][8];
  // loads of a row: (mb, j) -> 16 bytes at element (j << 10) | (mb << 9) | (lane << 3)
  auto load_row = [&](int row) {
    int ln = tid & 63;
    asm volatile("" : "+v"(ln));  // opaque: the addresses are rebuilt here instead of living (spilled) across the loop
    const uint16_t* src = x + static_cast<int64_t>(row) * n + (ln << 3);
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int j = 0; j < 8; ++j) raw[mb][j] = nt_load16(reinterpret_cast<const uint4*>(src + ((j << 10) | (mb << 9))));
  };
  int row = blockIdx.x * 8 + (tid >> 6);
  if (row < rows) load_row(row);
  // the constant matrix, under the latency of the first row
  for (int i = tid; i < 8 * 4 * 64; i += 512)
    reinterpret_cast<uint4*>(htab)[i] = reinterpret_cast<const uint4*>(kHFrag.w)[i];
  __syncthreads();
  for (; row < rows; row += nwaves) {
    const int64_t base = static_cast<int64_t>(row) * n;
    // Opaque per row: the per-lane addresses below are rebuilt for every row instead of being kept (and spilled)
    // across the whole loop.
    int lane = tid & 63;
    asm volatile("" : "+v"(lane));
    const int l4 = (lane >> 4) & 1, hh = lane >> 5;
    // after all exchanges: element index of this lane's (pair p, register r) run, without the run's own low bits
    const int lane_bits = (((lane >> 3) & 1) << 8) | (hh << 9) | ((lane & 7) << 10);
    if constexpr (PRE) {
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint4 sg = *reinterpret_cast<const uint4*>(pre + ((j << 10) | (mb << 9) | (lane << 3)));
          raw[mb][j].x ^= sg.x & 0x80008000u;
          raw[mb][j].y ^= sg.y & 0x80008000u;
          raw[mb][j].z ^= sg.z & 0x80008000u;
          raw[mb][j].w ^= sg.w & 0x80008000u;
        }
    }
    // ---- H_128 on the matrix cores: all four column blocks (nb = i[1:0]) of both row blocks
    auto run_index = [&](int p, int r) { return (l4 << 2) | ((r & 3) << 3) | (p << 5) | ((r >> 2) << 6) | lane_bits; };
    uint32_t pk[2][2][16];  // [pair p][half][r]: the finished elements i[1:0] = 2 half, 2 half + 1 as packed bf16
    fw_v16f acc[2][4];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][nb][r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
      // k-step kk multiplies element e of every 16-byte load: k[4] = i[2], k[5] = i[0], k[6] = i[1]
      constexpr int kSel[2] = {0x05040100, 0x07060302};  // low halves / high halves of two dwords
      const int e = ((kk & 1) << 2) | (((kk >> 2) & 1) << 1) | ((kk >> 1) & 1);
      fw_v4i a[2];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t lo = dword_of(raw[mb][2 * d], e >> 1), hi = dword_of(raw[mb][2 * d + 1], e >> 1);
          a[mb][d] = static_cast<int>(__builtin_amdgcn_perm(hi, lo, kSel[e & 1]));
        }
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        const fw_v4i b = *reinterpret_cast<const fw_v4i*>(htab + ((kk * 4 + nb) * 64 + lane) * 4);
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(fw_bf16x8, a[mb]),
                                                                __builtin_bit_cast(fw_bf16x8, b), acc[mb][nb], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // The inputs are used up: request the next row of this wavefront now, under the butterflies and the finish.
    if (row + nwaves < rows) load_row(row + nwaves);
    __builtin_amdgcn_sched_barrier(0);
    // ---- the rest in two halves (nb = 0, 1 and nb = 2, 3): less is alive at a time
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      // ---- butterflies over the register bits r[0..3] and mb
      float v[2][2][16];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nl = 0; nl < 2; ++nl)
#pragma unroll
          for (int r = 0; r < 16; ++r) v[mb][nl][r] = acc[mb][2 * half + nl][r];
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int nl = 0; nl < 2; ++nl)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if ((r & (1 << s)) == 0) {
                const float a0 = v[mb][nl][r], c0 = v[mb][nl][r | (1 << s)];
                v[mb][nl][r] = a0 + c0;
                v[mb][nl][r | (1 << s)] = a0 - c0;
              }
      // mb inside the lane, then the bit held by the lane half (h = i[5]): trade it for i[9].  After the swap the lower
      // half of the wavefront holds both h of mb = 0 and the upper half both h of mb = 1; index 0 / 1 of the pair is i[5].
#pragma unroll
      for (int nl = 0; nl < 2; ++nl)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float m0 = v[0][nl][r] + v[1][nl][r], m1 = v[0][nl][r] - v[1][nl][r];
          const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(m0), __float_as_uint(m1), false, false);
          const float a0 = __uint_as_float(sw[0]), c0 = __uint_as_float(sw[1]);
          v[0][nl][r] = a0 + c0;
          v[1][nl][r] = a0 - c0;
        }
      // v[p][nl][r] is element i = nl | half << 1 | l4 << 2 | r[1:0] << 3 | p << 5 | r[3:2] << 6 | lane_bits
      // ---- sign behind the transform, rounding to bf16, scale
#pragma unroll
      for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float t0 = v[p][0][r], t1 = v[p][1][r];
          if constexpr (POST) {
            const uint32_t w = *reinterpret_cast<const uint32_t*>(post + run_index(p, r) + 2 * half);
            t0 *= __uint_as_float(w << 16);
            t1 *= __uint_as_float(w & 0xFFFF0000u);
          }
          uint32_t w2 = pack_bf16x2(t0, t1);
          if (out_scale != 1.0f) w2 = pack_bf16x2(__uint_as_float(w2 << 16) * out_scale, __uint_as_float(w2 & 0xFFFF0000u) * out_scale);
          pk[p][half][r] = w2;
        }
      __builtin_amdgcn_sched_barrier(0);  // the halves one after the other: together they do not fit the register file
    }
    // ---- pack every run of four, then make runs of sixteen: word[p][r][..] -> out[p][r >> 2][..]
    constexpr int W = (MODE == 0) ? 2 : 1;          // dwords per run of four (int4: 16 bits in one dword)
    uint32_t word[2][16][W];
    if constexpr (MODE == 0) {
#pragma unroll
      for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          word[p][r][0] = pk[p][0][r];
          word[p][r][1] = pk[p][1][r];
        }
    } else {
      // |x| of bf16 orders like its low 15 bits
      typedef unsigned short fw_u16x2 __attribute__((ext_vector_type(2)));
      // quantizes the run (p, r) with scale s1 (r1 = its reciprocal) into word[p][r]
      auto quantize_run4 = [&](int p, int r, float s1, float r1) {
        Divider<BF16, false, false> div(1.f);  // zero quotients come out as +0; e4m3 takes its signs from the dividends
        div.s = s1;
        div.r = r1;
        float t[4];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          t[2 * hf] = __uint_as_float(pk[p][hf][r] << 16);
          t[2 * hf + 1] = __uint_as_float(pk[p][hf][r] & 0xFFFF0000u);
          div.pair_unsigned(t[2 * hf], t[2 * hf + 1]);
        }
        if constexpr (QT == QWIX_INT8) {
          word[p][r][0] = pack4_low_bytes(rne_bits_clamped(t[0], -128.f, 127.f), rne_bits_clamped(t[1], -128.f, 127.f),
                                          rne_bits_clamped(t[2], -128.f, 127.f), rne_bits_clamped(t[3], -128.f, 127.f));
        } else if constexpr (QT == QWIX_INT4) {
          word[p][r][0] = (rne_bits_clamped(t[0], -8.f, 7.f) & 0xFu) | ((rne_bits_clamped(t[1], -8.f, 7.f) & 0xFu) << 4) |
                          ((rne_bits_clamped(t[2], -8.f, 7.f) & 0xFu) << 8) | ((rne_bits_clamped(t[3], -8.f, 7.f) & 0xFu) << 12);
        } else {
          // a quotient carries the sign of its dividend, zero quotients included: the four sign bits come from there
          const uint32_t w = to_e4m3x2_bounded(t[0], t[1]) | (to_e4m3x2_bounded(t[2], t[3]) << 16);
          word[p][r][0] = (__builtin_amdgcn_perm(pk[p][1][r], pk[p][0][r], 0x07050301u) & 0x80808080u) | (w & 0x7F7F7F7Fu);
        }
      };
      __builtin_amdgcn_sched_barrier(0);
      if (ltile == B) {
        fw_u16x2 m = {0, 0};
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int r = 0; r < 16; ++r) m = __builtin_elementwise_max(m, __builtin_bit_cast(fw_u16x2, pk[p][hf][r] & 0x7FFF7FFFu));
        const float am = wave_xor_max(bf16_bits_to_f32(m[0] > m[1] ? m[0] : m[1]), 64);
        const float s1 = sym_scale<BF16, QT>(am), r1 = __builtin_amdgcn_rcpf(s1);
        if (lane == 0) store1<BF16>(scale, row, s1);
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            quantize_run4(p, r, s1, r1);
            if (r & 1) __builtin_amdgcn_sched_barrier(0);  // two runs at a time: all 32 at once do not fit the registers
          }
      } else {
        float gm[2][16];
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const fw_u16x2 m = __builtin_elementwise_max(__builtin_bit_cast(fw_u16x2, pk[p][0][r] & 0x7FFF7FFFu),
                                                         __builtin_bit_cast(fw_u16x2, pk[p][1][r] & 0x7FFF7FFFu));
            gm[p][r] = bf16_bits_to_f32(m[0] > m[1] ? m[0] : m[1]);
          }
        // index bits below ltile, in the order they sit: i[2] = lane bit 4, i[3], i[4] = r[0], r[1], i[5] = p,
        // i[6], i[7] = r[2], r[3], i[8] = lane bit 3
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int r = 0; r < 16; ++r) gm[p][r] = fmaxf(gm[p][r], __shfl_xor(gm[p][r], 16, 64));
        auto over_r = [&](int bit) {
#pragma unroll
          for (int p = 0; p < 2; ++p)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if ((r & bit) == 0) {
                const float m = fmaxf(gm[p][r], gm[p][r | bit]);
                gm[p][r] = m;
                gm[p][r | bit] = m;
              }
        };
        if (ltile > 3) over_r(1);
        if (ltile > 4) over_r(2);
        if (ltile > 5) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float m = fmaxf(gm[0][r], gm[1][r]);
            gm[0][r] = m;
            gm[1][r] = m;
          }
        }
        if (ltile > 6) over_r(4);
        if (ltile > 7) over_r(8);
        if (ltile > 8) {
#pragma unroll
          for (int p = 0; p < 2; ++p)
#pragma unroll
            for (int r = 0; r < 16; ++r) gm[p][r] = fmaxf(gm[p][r], __shfl_xor(gm[p][r], 8, 64));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float s1 = sym_scale<BF16, QT>(gm[p][r]);
            const int i0 = run_index(p, r);
            if ((i0 & ((1 << ltile) - 1)) == 0) store1<BF16>(scale, (base + i0) >> ltile, s1);
            quantize_run4(p, r, s1, __builtin_amdgcn_rcpf(s1));
            if (r & 1) __builtin_amdgcn_sched_barrier(0);
          }
      }
    }
    // first exchange, over r[0] (i[3]): afterwards lane bit 4 stands for i[3] and the word order for i[2];
    // second exchange, over r[1] (i[4]): afterwards lane bit 4 stands for i[4].
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if ((r & 1) == 0)
#pragma unroll
          for (int w = 0; w < W; ++w) swap_rows16(word[p][r][w], word[p][r | 1][w]);
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if ((r & 2) == 0)
#pragma unroll
          for (int w = 0; w < W; ++w) swap_rows16(word[p][r][w], word[p][r | 2][w]);
    // out run (p, r >> 2): words in the order r = 4 q, 4 q + 1, 4 q + 2, 4 q + 3: sixteen consecutive elements at
    // i = l4 << 4 | p << 5 | q << 6 | lane_bits.  A lane's runs lie 32 bytes (int8) apart from its neighbour's and far
    // from everybody else's, so the row is put together in this wavefront's piece of LDS and leaves with whole
    // kilobytes per store instruction.  Inside every 256-byte block of the staged row the 16-byte chunks are XOR-ed
    // with a key taken from the block number, so that the sixteen lanes that write at the same time (same chunk
    // number, different blocks) hit different banks.
    const int l3 = (lane >> 3) & 1, l210 = lane & 7;
    const int wkey = (EB == 4) ? l210 : (l3 | (l210 << 1));
    asm volatile("" ::: "memory");
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int i = (l4 << 4) | (p << 5) | (q << 6) | lane_bits;
        const int o = i * EB / 8;                                  // byte offset in the row
        const int blk = o >> 8, c = (o >> 4) & 15;
        uint8_t* dst = stage + (blk << 8) + ((c ^ wkey) << 4) + (o & 15);
        if constexpr (MODE == 0) {
          *reinterpret_cast<uint4*>(dst) = make_uint4(word[p][4 * q][0], word[p][4 * q][1], word[p][4 * q + 1][0], word[p][4 * q + 1][1]);
          uint8_t* dst2 = stage + (blk << 8) + (((c + 1) ^ wkey) << 4);
          *reinterpret_cast<uint4*>(dst2) =
              make_uint4(word[p][4 * q + 2][0], word[p][4 * q + 2][1], word[p][4 * q + 3][0], word[p][4 * q + 3][1]);
        } else if constexpr (QT == QWIX_INT4) {
          *reinterpret_cast<uint2*>(dst) = make_uint2(word[p][4 * q][0] | (word[p][4 * q + 1][0] << 16),
                                                      word[p][4 * q + 2][0] | (word[p][4 * q + 3][0] << 16));
        } else {
          *reinterpret_cast<uint4*>(dst) = make_uint4(word[p][4 * q][0], word[p][4 * q + 1][0], word[p][4 * q + 2][0], word[p][4 * q + 3][0]);
        }
      }
    __builtin_amdgcn_wave_barrier();
    asm volatile("" ::: "memory");  // the reads below are of other lanes' writes: LDS serves one wavefront in order
    uint8_t* out = static_cast<uint8_t*>(y) + base * EB / 8;
#pragma unroll
    for (int k = 0; k < ROW_BYTES / 1024; ++k) {
      const int L = k * 1024 + lane * 16;
      const int blk = L >> 8, c = (L >> 4) & 15;
      // the key the writers of this block used: EB 8: blk = l3 + 2 hh + 4 l210; EB 16: blk = q[1] + 2 l3 + 4 hh + 8 l210;
      // EB 4: blk = hh + 2 l210 (there l3 is part of the chunk number)
      const int rkey = (EB == 8) ? ((blk & 1) | ((blk >> 2) << 1)) : (EB == 16) ? (((blk >> 1) & 1) | ((blk >> 3) << 1)) : (blk >> 1);
      const uint4 v16 = *reinterpret_cast<const uint4*>(stage + (blk << 8) + ((c ^ rkey) << 4));
      nt_store16(reinterpret_cast<uint4*>(out + L), v16);
    }
    asm volatile("" ::: "memory");
  }
}

template <int MODE, int QT, bool PRE, bool POST>
int launch_fwht_mfma2(const void* x, int64_t rows, const void* pre, const void* post, float out_scale, int ltile, void* y,
                      void* scale, hipStream_t st) {
  // eight wavefronts per workgroup (two per SIMD: one multiplies while the other adds), a row per wavefront and trip;
  // one workgroup per CU is all that fits, so the grid is at most that and the wavefronts walk the rows
  int cus = 0, dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  const int64_t groups = std::min<int64_t>((rows + 7) / 8, cus);
  constexpr size_t smem = 32768 + 8 * (size_t{8192} * ((MODE == 0) ? 16 : (QT == QWIX_INT4 ? 4 : 8)) / 8);
  auto kern = fwht_mfma_kernel<MODE, QT, PRE, POST>;
  static LdsGrant granted;
  if (int e_ = grant_lds(reinterpret_cast<const void*>(kern), smem, granted)) return e_;
  kern<<<dim3(static_cast<unsigned>(groups)), 512, smem, st>>>(
      static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(pre), static_cast<const uint16_t*>(post), out_scale,
      ltile, static_cast<int>(rows), y, scale);
  return check_launch("fwht (matrix cores)");
}

template <int MODE, int QT>
int launch_fwht_mfma(const void* x, int64_t rows, const void* pre, const void* post, float out_scale, int ltile, void* y,
                     void* scale, hipStream_t st) {
  if (pre != nullptr) {
    if (post != nullptr) return launch_fwht_mfma2<MODE, QT, true, true>(x, rows, pre, post, out_scale, ltile, y, scale, st);
    return launch_fwht_mfma2<MODE, QT, true, false>(x, rows, pre, post, out_scale, ltile, y, scale, st);
  }
  if (post != nullptr) return launch_fwht_mfma2<MODE, QT, false, true>(x, rows, pre, post, out_scale, ltile, y, scale, st);
  return launch_fwht_mfma2<MODE, QT, false, false>(x, rows, pre, post, out_scale, ltile, y, scale, st);
}

// bf16 rows of 8192 with 16-byte aligned operands; scale groups of 8 to 512 elements or the whole row.
inline bool mfma_path_ok(int dtype, int logn, const void* x, const void* pre, const void* post, const void* y) {
  return dtype == QWIX_BF16 && logn == 13 && aligned16(x) && aligned16(y) && (pre == nullptr || aligned16(pre)) &&
         (post == nullptr || (reinterpret_cast<uintptr_t>(post) & 7) == 0);
}

// The matrix-core kernel runs a row per wavefront, 2048 rows per trip of the chip; the register kernel runs a row per
// workgroup of four wavefronts.  Measured (rotate + quantize to int8): 16 / 256 / 1024 rows 12.9 / 13.3 / 15.4 us against
// 5.8 / 6.0 / 9.8 us, 2048 rows 16.5 against 18.7, 3072 rows (two trips, the second half empty) 26.9 against 24.8, 8192
// rows 51.8 against 57.2: the matrix-core kernel where whole trips of 2048 rows make it cheaper by this model.
inline bool mfma_rows_pay(int64_t rows) {
  const double trips = static_cast<double>((rows + 2047) / 2048);
  return 4.5 + 11.8 * trips < 5.0 + 0.0065 * static_cast<double>(rows);
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
  if (mfma_rows_pay(rows) && mfma_path_ok(dtype, logn, x, pre_sign, post_sign, y))
    return launch_fwht_mfma<0, QWIX_INT8>(x, rows, pre_sign, post_sign, out_scale, logn, y, nullptr, st);
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
  if (mfma_rows_pay(rows) && mfma_path_ok(dtype, logn, x, pre_sign, post_sign, qvalue) && (qtype == QWIX_INT8 || qtype == QWIX_INT4 || qtype == QWIX_E4M3)) {
    if (qtype == QWIX_INT8) return launch_fwht_mfma<1, QWIX_INT8>(x, rows, pre_sign, post_sign, out_scale, ltile, qvalue, scale, st);
    if (qtype == QWIX_INT4) return launch_fwht_mfma<1, QWIX_INT4>(x, rows, pre_sign, post_sign, out_scale, ltile, qvalue, scale, st);
    return launch_fwht_mfma<1, QWIX_E4M3>(x, rows, pre_sign, post_sign, out_scale, ltile, qvalue, scale, st);
  }
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
