// Device-side numerics shared by all kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>

#include "../../include/qwix_hip.h"

namespace qwix {

// ------------------------------------------------------------------ host: errors
inline char* err_buf() {
  static thread_local char buf[512] = {0};
  return buf;
}
inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(err_buf(), 512, fmt, ap);
  va_end(ap);
  return code;
}
inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(QWIX_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return QWIX_OK;
}
// Dynamic-LDS limit of a kernel (hipFuncAttributeMaxDynamicSharedMemorySize), raised when a launch needs more
// than was granted so far on the current device.  Safe to call from several threads: the attribute call is
// idempotent and the record of what was granted is atomic; the library keeps no other mutable state.
struct LdsGrant {
  static constexpr int kDevices = 64;
  std::atomic<size_t> bytes[kDevices];
};
inline int grant_lds(const void* kernel, size_t bytes, LdsGrant& g) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= LdsGrant::kDevices)
    return fail(QWIX_ERR_LAUNCH, "no current HIP device (index %d)", dev);
  size_t have = g.bytes[dev].load(std::memory_order_acquire);
  if (bytes <= have) return QWIX_OK;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
  if (e != hipSuccess) return fail(QWIX_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  while (have < bytes && !g.bytes[dev].compare_exchange_weak(have, bytes, std::memory_order_release)) {}
  return QWIX_OK;
}
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// ------------------------------------------------------------------ streaming accesses
// 16-byte load / store of data that this kernel touches exactly once (nontemporal: not kept in the caches).
typedef int qwix_v4i __attribute__((ext_vector_type(4)));
typedef int qwix_v2i __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 nt_load16(const uint4* p) {
  return __builtin_bit_cast(uint4, __builtin_nontemporal_load(reinterpret_cast<const qwix_v4i*>(p)));
}
__device__ __forceinline__ void nt_store16(uint4* p, uint4 v) {
  __builtin_nontemporal_store(__builtin_bit_cast(qwix_v4i, v), reinterpret_cast<qwix_v4i*>(p));
}
__device__ __forceinline__ void nt_store8(uint2* p, uint2 v) {
  __builtin_nontemporal_store(__builtin_bit_cast(qwix_v2i, v), reinterpret_cast<qwix_v2i*>(p));
}

// ------------------------------------------------------------------ LDS layout
// Swizzle key of a 128-byte row in LDS: 16-byte chunk c of row r sits at chunk position c ^ swz128(r).  The LDS
// serves a ds_read_b128 sixteen lanes at a time out of 64 banks (256 bytes): sixteen consecutive rows must land
// in sixteen different 16-byte bank groups.  Row parity already selects the upper or lower 128 bytes, so the key
// is taken from the next three bits of the row number.
__device__ __forceinline__ int swz128(int row) { return (row >> 1) & 7; }

// ------------------------------------------------------------------ dtype tags
struct F32 {
  using storage = float;
  static constexpr int kTag = QWIX_F32;
  static constexpr int kVec = 4;  // elements per 16-byte vector
};
struct BF16 {
  using storage = uint16_t;
  static constexpr int kTag = QWIX_BF16;
  static constexpr int kVec = 8;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float x) {
  __bf16 b = static_cast<__bf16>(x);  // RNE
  return __builtin_bit_cast(uint16_t, b);
}
// Two f32 -> two bf16 (RNE) in one v_cvt_pk_bf16_f32: a in the low half, b in the high half.
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// Round an f32 result to bf16 precision but keep it in an f32 register.
__device__ __forceinline__ float round_bf16(float x) {
  return bf16_bits_to_f32(f32_to_bf16_bits(x));
}

// Two values at once: one convert for the pair.
__device__ __forceinline__ void round_bf16_pair(float& a, float& b) {
  const uint32_t w = pack_bf16x2(a, b);
  a = __uint_as_float(w << 16);
  b = __uint_as_float(w & 0xFFFF0000u);
}

template <typename D>
__device__ __forceinline__ float rnd(float x) {
  if constexpr (D::kTag == QWIX_BF16) return round_bf16(x);
  return x;
}
template <typename D>
__device__ __forceinline__ float load1(const void* p, int64_t i) {
  if constexpr (D::kTag == QWIX_BF16)
    return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[i]);
  else
    return reinterpret_cast<const float*>(p)[i];
}
template <typename D>
__device__ __forceinline__ void store1(void* p, int64_t i, float v) {
  if constexpr (D::kTag == QWIX_BF16)
    reinterpret_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
  else
    reinterpret_cast<float*>(p)[i] = v;
}

// One 16-byte vector of D -> kVec floats.
template <typename D>
__device__ __forceinline__ void unpack16(const uint4& v, float* f) {
  if constexpr (D::kTag == QWIX_BF16) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
    }
  } else {
    f[0] = __uint_as_float(v.x);
    f[1] = __uint_as_float(v.y);
    f[2] = __uint_as_float(v.z);
    f[3] = __uint_as_float(v.w);
  }
}

// ------------------------------------------------------------------ qtype traits
template <int QT>
struct QTraits;
template <>
struct QTraits<QWIX_INT8> {
  static constexpr float kSymBound = 127.5f, kMin = -128.f, kMax = 127.f;
};
template <>
struct QTraits<QWIX_INT4> {
  static constexpr float kSymBound = 7.5f, kMin = -8.f, kMax = 7.f;
};
template <>
struct QTraits<QWIX_E4M3> {
  static constexpr float kSymBound = 448.f, kMin = -448.f, kMax = 448.f;
};

constexpr float kTinySqrt = 0x1p-63f;  // sqrt(finfo.tiny) for f32 and bf16 alike

// Saturating float -> int32 of an already integral value; NaN -> 0.  The hardware convert has
// exactly these semantics, a C cast of an out-of-range float does not.
__device__ __forceinline__ int cvt_i32_sat(float r) {
  int q;
  asm("v_cvt_i32_f32 %0, %1" : "=v"(q) : "v"(r));
  return q;
}
template <int QT>
__device__ __forceinline__ int to_int_q(float v) {
  int q = cvt_i32_sat(__builtin_rintf(v));  // rintf = round half to even
  const int lo = static_cast<int>(QTraits<QT>::kMin), hi = static_cast<int>(QTraits<QT>::kMax);
  return min(max(q, lo), hi);
}
// Two clipped floats -> two OCP e4m3 bytes in the low 16 bits (RNE, subnormals kept).
__device__ __forceinline__ uint32_t to_e4m3x2(float a, float b) {
  // clip propagates NaN (the comparisons are false for NaN).
  a = a > 448.f ? 448.f : (a < -448.f ? -448.f : a);
  b = b > 448.f ? 448.f : (b < -448.f ? -448.f : b);
  return static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false)) & 0xFFFFu;
}
// The same for values that are not NaN: the clip is one v_med3 per value.
__device__ __forceinline__ uint32_t to_e4m3x2_bounded(float a, float b) {
  a = __builtin_amdgcn_fmed3f(a, -448.f, 448.f);
  b = __builtin_amdgcn_fmed3f(b, -448.f, 448.f);
  return static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false)) & 0xFFFFu;
}
__device__ __forceinline__ float e4m3_to_f32(uint32_t byte) {
  return __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(byte), 0);
}

// ------------------------------------------------------------------ scale math
// compute_scale_zero_point, symmetric branch: scale = D(absmax / bound), tiny guard.
template <typename D, int QT>
__device__ __forceinline__ float sym_scale(float absmax) {
  float s = rnd<D>(absmax / QTraits<QT>::kSymBound);
  return (s < kTinySqrt) ? 1.0f : s;
}
// asymmetric branch: scale = D(D(max-min)/(qmax-qmin)); zp = convert(D(qmin - D(min/scale))).
template <typename D, int QT>
__device__ __forceinline__ float asym_scale_zp(float mn, float mx, int* zp) {
  float s = rnd<D>(rnd<D>(mx - mn) / (QTraits<QT>::kMax - QTraits<QT>::kMin));
  s = (s < kTinySqrt) ? 1.0f : s;
  float z = rnd<D>(QTraits<QT>::kMin - rnd<D>(mn / s));
  *zp = to_int_q<QT>(z);
  return s;
}
template <typename D>
__device__ __forceinline__ float apply_factor(float v, float factor) {
  return factor > 0.f ? rnd<D>(v * rnd<D>(factor)) : v;
}

// x / s rounded to D.  f32: IEEE division.  bf16: both operands have 8-bit significands X and S (128 .. 255).  The
// quotient cannot lie on a bf16 rounding boundary (a boundary has an odd 9-bit significand Q >= 257, and
// X * 2^m = Q * S would make Q divide X), and its distance from the nearest one is at least 1 / (512 S) > 2^-17
// relative.  x * rcp(s) is within 2^-22 of the quotient (v_rcp_f32: 1 ulp, the product: half an ulp), so it rounds
// to the same bf16 as RNE_bf16(RNE_f32(x / s)) does: one multiply per element.  (Quotients in the bf16 subnormal range
// round to zero in every target type.)
// kSafe=false is for quotients known to be bounded (dynamic range: |x| <= absmax).
// kSignedZero keeps the sign of a zero quotient (matters for e4m3's -0 only).
template <typename D, bool kSafe = true, bool kSignedZero = true>
struct Divider {
  float s, r;
  __device__ __forceinline__ explicit Divider(float scale) : s(scale) {
    if constexpr (D::kTag == QWIX_BF16) r = __builtin_amdgcn_rcpf(scale);
  }
  // The quotient before its rounding to D (f32: the quotient itself).
  __device__ __forceinline__ float raw(float x) const {
    if constexpr (D::kTag == QWIX_BF16) {
      float q1 = x * r;
      if constexpr (kSafe) {
        const bool odd = !(__builtin_fabsf(q1) < 0x1p100f);
        if (__builtin_amdgcn_ballot_w64(odd) != 0) {
          if (odd) q1 = x / s;
        }
      }
      return q1;
    } else {
      return x / s;
    }
  }
  // Divides a pair; the bf16 rounding of both is one convert.  Zero quotients come out as +0.
  __device__ __forceinline__ void pair_unsigned(float& a, float& b) const {
    a = raw(a);
    b = raw(b);
    if constexpr (D::kTag == QWIX_BF16) round_bf16_pair(a, b);
  }
  __device__ __forceinline__ void pair(float& a, float& b) const {
    const float xa = a, xb = b;
    pair_unsigned(a, b);
    if constexpr (kSignedZero && D::kTag == QWIX_BF16) {
      a = __builtin_copysignf(a, xa);
      b = __builtin_copysignf(b, xb);
    }
  }
  __device__ __forceinline__ float operator()(float x) const {
    if constexpr (D::kTag == QWIX_BF16) {
      float q1 = x * r;
      // Overflowing or non-finite quotients (static scales only): take the IEEE path.  The test is made
      // wave-uniform first, so that the division sequence is branched over instead of being computed
      // for every element and selected away.
      if constexpr (kSafe) {
        const bool odd = !(__builtin_fabsf(q1) < 0x1p100f);
        if (__builtin_amdgcn_ballot_w64(odd) != 0) {
          if (odd) q1 = x / s;
        }
      }
      // The quotient always carries the sign of x (s > 0).
      if constexpr (kSignedZero) return __builtin_copysignf(round_bf16(q1), x);
      return round_bf16(q1);
    } else {
      return x / s;
    }
  }
};

// ------------------------------------------------------------------ wave helpers
__device__ __forceinline__ float wave_xor_max(float v, int width) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1)
    if (m < width) v = fmaxf(v, __shfl_xor(v, m, 64));
  return v;
}
__device__ __forceinline__ float wave_xor_min(float v, int width) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1)
    if (m < width) v = fminf(v, __shfl_xor(v, m, 64));
  return v;
}
// NaN-propagating max of |x|: fmaxf drops NaNs, so track them separately where it matters.
__device__ __forceinline__ float absmax_acc(float acc, float x) {
  return fmaxf(acc, __builtin_fabsf(x));
}

// Saturating round-half-even to a small integer in two float ops: clamp to [lo, hi] (one v_med3,
// +-inf included), then add 1.5 * 2^23: the add rounds to the nearest (even) integer and leaves its
// two's complement in the low mantissa bits.  NaN is not mapped to 0 here (unpinned either way).
__device__ __forceinline__ uint32_t rne_bits_clamped(float v, float lo, float hi) {
  return __float_as_uint(__builtin_amdgcn_fmed3f(v, lo, hi) + 12582912.0f);
}
__device__ __forceinline__ uint32_t pack4_low_bytes(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  return __builtin_amdgcn_perm(b, a, 0x0c0c0400u) | __builtin_amdgcn_perm(d, c, 0x04000c0cu);
}

// pack helpers
__device__ __forceinline__ uint32_t pack4_i8(int a, int b, int c, int d) {
  return (a & 0xFF) | ((b & 0xFF) << 8) | ((c & 0xFF) << 16) | (static_cast<uint32_t>(d) << 24);
}
__device__ __forceinline__ uint32_t pack2_i4(int lo, int hi) { return (lo & 0xF) | ((hi & 0xF) << 4); }

// ---- buffer loads: a wave-uniform descriptor plus a 32-bit per-lane byte offset plus a wave-uniform offset ----
// A descriptor without a bound of its own (the callers' offsets are in range by construction): raw, untyped.
__device__ __forceinline__ auto buffer_from(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7FFFFFFF, 0x00020000);
}

// 16 bytes per lane from a buffer straight into LDS (lane l lands at lds + 16 l).  The host pass of the compiler
// does not know the 16-byte form of this builtin (it checks against its own target), hence the guard: there is
// nothing to compile on that side.
template <typename R>
__device__ __forceinline__ void buffer_to_lds16(R rsrc, uint8_t* lds, unsigned voffset, int soffset) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(lds), 16, voffset, soffset, 0, 0);
#endif
}

}  // namespace qwix
