// Quantize / calibrate / dequantize kernels (HBM-bound) and their C entry points.
//
// Data model: the float array is the row-major 3-D view (outer, reduce, inner); one scale per
// (outer, reduce/tile, inner).  Two kernel families:
//   rows_*  inner == 1: every scale group is a contiguous segment of `tile` elements.  A group of
//           G = 2^g threads owns a segment, keeps it in registers (up to 8 x 16-byte loads per
//           thread), max-reduces with wave shuffles (+ LDS across waves), then divides, rounds
//           and stores packed bytes.  One read, one write.
//   cols_*  inner > 1: the reduced axis is strided.  Pass 1 reduces 128-row panels in registers
//           and merges panels with a 32-bit atomic max into a caller-provided workspace; pass 2
//           re-reads each panel, quantizes it, and writes either the natural layout or the
//           reduce-minor (transposed) layout the GEMM kernels consume.
#include <algorithm>
#include <cstdlib>
#include <mutex>

#include <type_traits>

#include "common.h"

namespace qwix {
namespace {

enum { MODE_QUANT = 0, MODE_CALIB = 1, MODE_GIVEN = 2 };

// Quantize N consecutive values (already divided / shifted) and store them packed.  BOUNDED selects
// the two-op clamp-and-round converter (vector paths); the scalar paths keep NaN -> 0.
template <int QT, int N, bool BOUNDED = false>
__device__ __forceinline__ void store_q(const float* v, uint8_t* q, int64_t elem, const uint32_t* bf16_signs = nullptr) {
  if constexpr (QT == QWIX_INT8) {
    uint32_t w[N / 4];
#pragma unroll
    for (int i = 0; i < N / 4; ++i) {
      if constexpr (BOUNDED)
        w[i] = pack4_low_bytes(rne_bits_clamped(v[4 * i], -128.f, 127.f), rne_bits_clamped(v[4 * i + 1], -128.f, 127.f),
                               rne_bits_clamped(v[4 * i + 2], -128.f, 127.f), rne_bits_clamped(v[4 * i + 3], -128.f, 127.f));
      else
        w[i] = pack4_i8(to_int_q<QT>(v[4 * i]), to_int_q<QT>(v[4 * i + 1]), to_int_q<QT>(v[4 * i + 2]),
                        to_int_q<QT>(v[4 * i + 3]));
    }
    if constexpr (N == 8)
      nt_store8(reinterpret_cast<uint2*>(q + elem), make_uint2(w[0], w[1]));
    else
      *reinterpret_cast<uint32_t*>(q + elem) = w[0];
  } else if constexpr (QT == QWIX_E4M3) {
    uint32_t w[N / 4];
#pragma unroll
    for (int i = 0; i < N / 4; ++i) {
      if constexpr (BOUNDED)
        w[i] = to_e4m3x2_bounded(v[4 * i], v[4 * i + 1]) | (to_e4m3x2_bounded(v[4 * i + 2], v[4 * i + 3]) << 16);
      else
        w[i] = to_e4m3x2(v[4 * i], v[4 * i + 1]) | (to_e4m3x2(v[4 * i + 2], v[4 * i + 3]) << 16);
      // bf16_signs: the packed bf16 words the values were divided from (two per output word).  A quotient
      // carries the sign of its dividend, zero quotients included: take the four sign bits from there.
      if (bf16_signs != nullptr)
        w[i] = (__builtin_amdgcn_perm(bf16_signs[2 * i + 1], bf16_signs[2 * i], 0x07050301u) & 0x80808080u) |
               (w[i] & 0x7F7F7F7Fu);
    }
    if constexpr (N == 8)
      nt_store8(reinterpret_cast<uint2*>(q + elem), make_uint2(w[0], w[1]));
    else
      *reinterpret_cast<uint32_t*>(q + elem) = w[0];
  } else {  // INT4: element `elem` is even; low nibble = even element.
    uint32_t w = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if constexpr (BOUNDED)
        w |= (rne_bits_clamped(v[i], -8.f, 7.f) & 0xFu) << (4 * i);
      else
        w |= static_cast<uint32_t>(to_int_q<QT>(v[i]) & 0xF) << (4 * i);
    }
    if constexpr (N == 8)
      *reinterpret_cast<uint32_t*>(q + elem / 2) = w;
    else
      *reinterpret_cast<uint16_t*>(q + elem / 2) = static_cast<uint16_t>(w);
  }
}

template <int QT>
__device__ __forceinline__ uint8_t q_byte(float v) {  // one value -> one byte (int4 unpacked)
  if constexpr (QT == QWIX_E4M3)
    return static_cast<uint8_t>(to_e4m3x2(v, 0.f) & 0xFF);
  else
    return static_cast<uint8_t>(to_int_q<QT>(v) & 0xFF);
}

// ------------------------------------------------------------------------------------ rows
// nseg segments of L = nvec * kVec contiguous elements.  log2g: threads per segment; NL: 16-byte
// loads per thread.  The segment stays in registers in its packed form between the reduction and the
// quantization (the empty asm keeps the compiler from re-issuing the loads instead), so HBM is read
// exactly once.  bf16 absmax runs on the packed halves: |x| ordered like its 15 low bits.
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

template <typename D, int QT, int CAL, int MODE, int NL>
__global__ void __launch_bounds__(256)
    rows_kernel(const uint8_t* __restrict__ x, int64_t nseg, int nvec, int log2g, float factor,
                uint8_t* __restrict__ q, void* __restrict__ scale, int8_t* __restrict__ zp,
                void* __restrict__ cal0, void* __restrict__ cal1, int per_scale, int per_shift) {
  constexpr int EV = D::kVec;
  constexpr bool ASYM = (CAL == QWIX_MINMAX);
  __shared__ float red[2][4];
  const int tid = threadIdx.x;
  const int g = 1 << log2g;
  const int64_t seg = (static_cast<int64_t>(blockIdx.x) << (8 - log2g)) + (tid >> log2g);
  const int lane = tid & (g - 1);
  const bool seg_ok = seg < nseg;
  const uint4* xv = reinterpret_cast<const uint4*>(x) + seg * nvec;

  uint4 raw[NL];
#pragma unroll
  for (int j = 0; j < NL; ++j) {
    const int v = lane + (j << log2g);
    raw[j] = make_uint4(0, 0, 0, 0);
    if (seg_ok && v < nvec) raw[j] = xv[v];
  }
#pragma unroll
  for (int j = 0; j < NL; ++j) asm volatile("" : "+v"(raw[j].x), "+v"(raw[j].y), "+v"(raw[j].z), "+v"(raw[j].w));

  float s = 1.f;
  int z = 0;
  if constexpr (MODE != MODE_GIVEN) {
    float mx = 0.f, mn = 0.f;  // minmax clips to include 0; absmax >= 0
    if constexpr (!ASYM && D::kTag == QWIX_BF16) {
      u16x2 m = {0, 0};
#pragma unroll
      for (int j = 0; j < NL; ++j) {
        const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2, w[e] & 0x7FFF7FFFu));
      }
      mx = bf16_bits_to_f32(m[0] > m[1] ? m[0] : m[1]);
    } else {
#pragma unroll
      for (int j = 0; j < NL; ++j) {
        float f[EV];
        unpack16<D>(raw[j], f);
#pragma unroll
        for (int e = 0; e < EV; ++e) {
          if constexpr (ASYM) {
            mx = fmaxf(mx, f[e]);
            mn = fminf(mn, f[e]);
          } else {
            mx = absmax_acc(mx, f[e]);
          }
        }
      }
    }
    mx = wave_xor_max(mx, g < 64 ? g : 64);
    if constexpr (ASYM) mn = wave_xor_min(mn, g < 64 ? g : 64);
    if (g > 64) {  // uniform branch: segments span 2 or 4 waves
      const int w = tid >> 6;
      if ((tid & 63) == 0) {
        red[0][w] = mx;
        red[1][w] = mn;
      }
      __syncthreads();
      const int w0 = (tid >> log2g) << (log2g - 6), nw = 1 << (log2g - 6);
      mx = red[0][w0];
      mn = red[1][w0];
      for (int i = 1; i < nw; ++i) {
        mx = fmaxf(mx, red[0][w0 + i]);
        mn = fminf(mn, red[1][w0 + i]);
      }
    }
    mx = apply_factor<D>(mx, factor);
    if constexpr (ASYM) mn = apply_factor<D>(mn, factor);
    if constexpr (MODE == MODE_CALIB) {
      if (seg_ok && lane == 0) {
        if constexpr (ASYM) {
          store1<D>(cal0, seg, mn);
          store1<D>(cal1, seg, mx);
        } else {
          store1<D>(cal0, seg, mx);
        }
      }
      return;
    }
    if constexpr (ASYM)
      s = asym_scale_zp<D, QT>(mn, mx, &z);
    else
      s = sym_scale<D, QT>(mx);
    if (seg_ok && lane == 0) {
      store1<D>(scale, seg, s);
      if constexpr (ASYM) zp[seg] = static_cast<int8_t>(z);
    }
  } else {
    if (seg_ok) {  // per_scale consecutive segments are pieces of one scale group
      int64_t si = seg;  // per_shift: log2(per_scale) if that is a power of two, else -1
      if (per_scale > 1)
        si = per_shift >= 0 ? (seg >> per_shift)
                            : (nseg <= 0xFFFFFFFFll ? static_cast<int64_t>(static_cast<uint32_t>(seg) / static_cast<uint32_t>(per_scale))
                                                    : seg / per_scale);
      s = load1<D>(scale, si);
      if constexpr (ASYM) z = zp[si];
    }
  }

  const float zf = static_cast<float>(z);
  // With a given scale a NaN input must stay NaN in e4m3; the one-op clip does not keep it.
  constexpr bool kBounded = !(MODE == MODE_GIVEN && QT == QWIX_E4M3);
  auto quantize_all = [&](auto safe_tag) {
    const Divider<D, decltype(safe_tag)::value, false> div(s);  // the sign of a zero quotient is restored below
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      const int v = lane + (j << log2g);
      if (seg_ok && v < nvec) {
        float t[EV];
        unpack16<D>(raw[j], t);
#pragma unroll
        for (int e = 0; e < EV; e += 2) {
          div.pair_unsigned(t[e], t[e + 1]);
          if constexpr (ASYM) {
            t[e] += zf;
            t[e + 1] += zf;
            if constexpr (D::kTag == QWIX_BF16) round_bf16_pair(t[e], t[e + 1]);
          }
        }
        if constexpr (QT == QWIX_E4M3 && D::kTag == QWIX_BF16) {
          const uint32_t signs[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
          store_q<QT, EV, kBounded>(t, q, (seg * nvec + v) * EV, signs);
        } else {
          store_q<QT, EV, kBounded>(t, q, (seg * nvec + v) * EV);
        }
      }
    }
  };
  if constexpr (MODE == MODE_GIVEN && D::kTag == QWIX_BF16) {
    // A given scale can be anything: quotients may overflow or be NaN, which the reciprocal-based division
    // does not reproduce.  One test per wavefront on the largest magnitude a thread holds decides whether
    // all of its elements can take the plain path (as they always can when the scale comes from absmax).
    u16x2 m = {0, 0};
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
      for (int e = 0; e < 4; ++e) m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2, w[e] & 0x7FFF7FFFu));
    }
    const float big = bf16_bits_to_f32(m[0] > m[1] ? m[0] : m[1]);  // NaN / inf inputs order above finite ones
    const bool odd = !(big * __builtin_fabsf(__builtin_amdgcn_rcpf(s)) < 0x1p100f);
    if (__builtin_amdgcn_ballot_w64(odd) == 0)
      quantize_all(std::false_type{});
    else
      quantize_all(std::true_type{});
  } else {
    quantize_all(std::integral_constant<bool, MODE == MODE_GIVEN>{});
  }
}

// Any segment length (also odd ones): one workgroup per segment, two strided scalar passes; the
// second pass re-reads what the first left in cache.  int4 needs an even L.
template <typename D, int QT, int CAL, int MODE>
__global__ void __launch_bounds__(256)
    rows_loop_kernel(const void* __restrict__ x, int64_t L, float factor, uint8_t* __restrict__ q,
                     void* __restrict__ scale, int8_t* __restrict__ zp, void* __restrict__ cal0,
                     void* __restrict__ cal1) {
  constexpr bool ASYM = (CAL == QWIX_MINMAX);
  __shared__ float red[2][4];
  const int tid = threadIdx.x;
  const int64_t seg = blockIdx.x;
  const int64_t base = seg * L;
  float s = 1.f;
  int z = 0;
  if constexpr (MODE != MODE_GIVEN) {
    float mx = 0.f, mn = 0.f;
    for (int64_t i = tid; i < L; i += 256) {
      const float v = load1<D>(x, base + i);
      if constexpr (ASYM) {
        mx = fmaxf(mx, v);
        mn = fminf(mn, v);
      } else {
        mx = absmax_acc(mx, v);
      }
    }
    mx = wave_xor_max(mx, 64);
    mn = wave_xor_min(mn, 64);
    if ((tid & 63) == 0) {
      red[0][tid >> 6] = mx;
      red[1][tid >> 6] = mn;
    }
    __syncthreads();
    mx = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
    mn = fminf(fminf(red[1][0], red[1][1]), fminf(red[1][2], red[1][3]));
    mx = apply_factor<D>(mx, factor);
    if constexpr (ASYM) mn = apply_factor<D>(mn, factor);
    if constexpr (MODE == MODE_CALIB) {
      if (tid == 0) {
        if constexpr (ASYM) {
          store1<D>(cal0, seg, mn);
          store1<D>(cal1, seg, mx);
        } else {
          store1<D>(cal0, seg, mx);
        }
      }
      return;
    }
    if constexpr (ASYM)
      s = asym_scale_zp<D, QT>(mn, mx, &z);
    else
      s = sym_scale<D, QT>(mx);
    if (tid == 0) {
      store1<D>(scale, seg, s);
      if constexpr (ASYM) zp[seg] = static_cast<int8_t>(z);
    }
  } else {
    s = load1<D>(scale, seg);
    if constexpr (ASYM) z = zp[seg];
  }
  const Divider<D, true> div(s);
  const float zf = static_cast<float>(z);
  auto one = [&](int64_t i) {
    float t = div(load1<D>(x, base + i));
    if constexpr (ASYM) t = rnd<D>(t + zf);
    return t;
  };
  if constexpr (QT == QWIX_INT4) {
    for (int64_t i = tid; i < L / 2; i += 256)
      q[(base >> 1) + i] = static_cast<uint8_t>(pack2_i4(to_int_q<QT>(one(2 * i)), to_int_q<QT>(one(2 * i + 1))));
  } else {
    for (int64_t i = tid; i < L; i += 256) q[base + i] = q_byte<QT>(one(i));
  }
}

// ------------------------------------------------------------------------------------ cols
// Panels of 128 rows x (16 * kVec) columns inside one tile.  Block index -> (outer, tile, chunk,
// column block).  ws: [plane][outer][ntiles][inner] f32 bit patterns, plane 0 = max (or absmax),
// plane 1 = -min.
struct ColGeom {
  int64_t outer, reduce, inner, tile, ntiles;
  int chunks_per_tile, col_blocks;
};

template <typename D>
__device__ __forceinline__ void col_decode(const ColGeom& gm, int64_t b, int64_t* o, int64_t* t,
                                           int* chunk, int64_t* c0) {
  const int64_t cb = b % gm.col_blocks;
  b /= gm.col_blocks;
  *chunk = static_cast<int>(b % gm.chunks_per_tile);
  b /= gm.chunks_per_tile;
  *t = b % gm.ntiles;
  *o = b / gm.ntiles;
  *c0 = (cb * 16 + (threadIdx.x & 15)) * D::kVec;
}

template <typename D, int CAL>
__global__ void __launch_bounds__(256)
    cols_absmax_kernel(const uint8_t* __restrict__ x, ColGeom gm, uint32_t* __restrict__ ws) {
  constexpr int EV = D::kVec;
  constexpr bool ASYM = (CAL == QWIX_MINMAX);
  __shared__ float red[2][4][16][EV];
  int64_t o, t, c0;
  int chunk;
  col_decode<D>(gm, blockIdx.x, &o, &t, &chunk, &c0);
  const int tid = threadIdx.x, tc = tid & 15, tr = tid >> 4;
  const bool col_ok = c0 < gm.inner;
  const int64_t row_end = (t + 1) * gm.tile;
  float mx[EV], mn[EV];
#pragma unroll
  for (int e = 0; e < EV; ++e) mx[e] = mn[e] = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int64_t r = t * gm.tile + chunk * 128 + tr + 16 * j;
    if (col_ok && r < row_end) {
      float f[EV];
      unpack16<D>(*reinterpret_cast<const uint4*>(
                      x + ((o * gm.reduce + r) * gm.inner + c0) * sizeof(typename D::storage)),
                  f);
#pragma unroll
      for (int e = 0; e < EV; ++e) {
        if constexpr (ASYM) {
          mx[e] = fmaxf(mx[e], f[e]);
          mn[e] = fminf(mn[e], f[e]);
        } else {
          mx[e] = absmax_acc(mx[e], f[e]);
        }
      }
    }
  }
  // lanes l and l^16, l^32 hold the same columns.
#pragma unroll
  for (int e = 0; e < EV; ++e) {
    mx[e] = fmaxf(mx[e], __shfl_xor(mx[e], 16, 64));
    mx[e] = fmaxf(mx[e], __shfl_xor(mx[e], 32, 64));
    if constexpr (ASYM) {
      mn[e] = fminf(mn[e], __shfl_xor(mn[e], 16, 64));
      mn[e] = fminf(mn[e], __shfl_xor(mn[e], 32, 64));
    }
  }
  if ((tid & 63) < 16) {
#pragma unroll
    for (int e = 0; e < EV; ++e) {
      red[0][tid >> 6][tc][e] = mx[e];
      red[1][tid >> 6][tc][e] = mn[e];
    }
  }
  __syncthreads();
  if (tid < 16 && col_ok) {
    const int64_t wbase = (o * gm.ntiles + t) * gm.inner + c0;
    const int64_t plane = gm.outer * gm.ntiles * gm.inner;
#pragma unroll
    for (int e = 0; e < EV; ++e) {
      float a = fmaxf(fmaxf(red[0][0][tc][e], red[0][1][tc][e]), fmaxf(red[0][2][tc][e], red[0][3][tc][e]));
      atomicMax(ws + wbase + e, __float_as_uint(a));  // a >= 0: bit patterns order like values
      if constexpr (ASYM) {
        float b = fminf(fminf(red[1][0][tc][e], red[1][1][tc][e]), fminf(red[1][2][tc][e], red[1][3][tc][e]));
        atomicMax(ws + plane + wbase + e, __float_as_uint(-b));
      }
    }
  }
}

// The same reduction for tall scale groups (tile >= 256 rows): a workgroup covers 256 rows x 64 vectors of
// columns, each wavefront reading whole 1 KiB row pieces, and issues one atomic per column for 256 rows
// instead of one for 128.
constexpr int kWideRows = 256;
template <typename D, int CAL>
__global__ void __launch_bounds__(256)
    cols_absmax_wide_kernel(const uint8_t* __restrict__ x, ColGeom gm, int wide_col_blocks, int wide_chunks,
                            uint32_t* __restrict__ ws) {
  constexpr int EV = D::kVec;
  constexpr bool ASYM = (CAL == QWIX_MINMAX);
  constexpr bool PACKED = !ASYM && D::kTag == QWIX_BF16;  // |x| of a bf16 pair orders like its low 15 bits
  __shared__ float red[ASYM ? 2 : 1][4][EV][64];
  int64_t b = blockIdx.x;
  const int64_t cb = b % wide_col_blocks;
  b /= wide_col_blocks;
  const int chunk = static_cast<int>(b % wide_chunks);
  b /= wide_chunks;
  const int64_t t = b % gm.ntiles, o = b / gm.ntiles;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int64_t c0 = (cb * 64 + lane) * EV;
  const bool col_ok = c0 < gm.inner;
  const int64_t row_end = (t + 1) * gm.tile;
  const int64_t row0 = t * gm.tile + static_cast<int64_t>(chunk) * kWideRows + w;  // rows row0 + 4 * i
  float mx[EV], mn[EV];
  u16x2 pm[4] = {{0, 0}, {0, 0}, {0, 0}, {0, 0}};
#pragma unroll
  for (int e = 0; e < EV; ++e) mx[e] = mn[e] = 0.f;
  const uint8_t* xp = x + ((o * gm.reduce + row0) * gm.inner + c0) * sizeof(typename D::storage);
  const int64_t step = 4 * gm.inner * sizeof(typename D::storage);
  for (int it = 0; it < kWideRows / 32; ++it) {
    uint4 raw[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      raw[j] = make_uint4(0, 0, 0, 0);
      if (col_ok && row0 + 4 * (it * 8 + j) < row_end) raw[j] = *reinterpret_cast<const uint4*>(xp + (it * 8 + j) * step);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr (PACKED) {
        const uint32_t wd[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
        for (int k = 0; k < 4; ++k)
          pm[k] = __builtin_elementwise_max(pm[k], __builtin_bit_cast(u16x2, wd[k] & 0x7FFF7FFFu));
      } else {
        float f[EV];
        unpack16<D>(raw[j], f);
#pragma unroll
        for (int e = 0; e < EV; ++e) {
          if constexpr (ASYM) {
            mx[e] = fmaxf(mx[e], f[e]);
            mn[e] = fminf(mn[e], f[e]);
          } else {
            mx[e] = absmax_acc(mx[e], f[e]);
          }
        }
      }
    }
  }
  if constexpr (PACKED) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      mx[2 * k] = bf16_bits_to_f32(pm[k][0]);
      mx[2 * k + 1] = bf16_bits_to_f32(pm[k][1]);
    }
  }
#pragma unroll
  for (int e = 0; e < EV; ++e) {
    red[0][w][e][lane] = mx[e];
    if constexpr (ASYM) red[1][w][e][lane] = mn[e];
  }
  __syncthreads();
  // 64 * EV columns, 256 threads
  const int64_t wbase = (o * gm.ntiles + t) * gm.inner + cb * 64 * EV;
  const int64_t plane = gm.outer * gm.ntiles * gm.inner;
  for (int c = tid; c < 64 * EV; c += 256) {
    if (cb * 64 * EV + c >= gm.inner) break;
    const int l = c / EV, e = c % EV;
    const float a = fmaxf(fmaxf(red[0][0][e][l], red[0][1][e][l]), fmaxf(red[0][2][e][l], red[0][3][e][l]));
    atomicMax(ws + wbase + c, __float_as_uint(a));  // a >= 0: bit patterns order like values
    if constexpr (ASYM) {
      const float m = fminf(fminf(red[1][0][e][l], red[1][1][e][l]), fminf(red[1][2][e][l], red[1][3][e][l]));
      atomicMax(ws + plane + wbase + c, __float_as_uint(-m));
    }
  }
}

// Long segments are calibrated in pieces (rows_kernel in calibration mode, one partial per piece); this
// kernel merges the `pieces` partials of a segment (one wavefront per segment) and either writes the
// calibration values (MODE_CALIB) or turns them into scale / zero point (MODE_QUANT).  The partials
// already carry the calibration factor: rounding is monotone, so max and factor commute.
template <typename D, int QT, int CAL, int MODE>
__global__ void __launch_bounds__(256)
    rows_merge_kernel(const void* __restrict__ p0, const void* __restrict__ p1, int64_t nseg, int pieces,
                      void* __restrict__ scale, int8_t* __restrict__ zp, void* __restrict__ cal0,
                      void* __restrict__ cal1) {
  constexpr bool ASYM = (CAL == QWIX_MINMAX);
  const int64_t seg = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (seg >= nseg) return;
  float mx = 0.f, mn = 0.f;
  for (int i = lane; i < pieces; i += 64) {
    if constexpr (ASYM) {
      mn = fminf(mn, load1<D>(p0, seg * pieces + i));
      mx = fmaxf(mx, load1<D>(p1, seg * pieces + i));
    } else {
      mx = fmaxf(mx, load1<D>(p0, seg * pieces + i));
    }
  }
  mx = wave_xor_max(mx, 64);
  if constexpr (ASYM) mn = wave_xor_min(mn, 64);
  if (lane != 0) return;
  if constexpr (MODE == MODE_CALIB) {
    if constexpr (ASYM) {
      store1<D>(cal0, seg, mn);
      store1<D>(cal1, seg, mx);
    } else {
      store1<D>(cal0, seg, mx);
    }
  } else {
    int z = 0;
    float s;
    if constexpr (ASYM)
      s = asym_scale_zp<D, QT>(mn, mx, &z);
    else
      s = sym_scale<D, QT>(mx);
    store1<D>(scale, seg, s);
    if constexpr (ASYM) zp[seg] = static_cast<int8_t>(z);
  }
}

__global__ void fill_u32_kernel(uint32_t* p, int64_t n, uint32_t v) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// ws -> calibration arrays of dtype D (calibrate-only path).
template <typename D, int CAL>
__global__ void cols_finish_cal_kernel(const uint32_t* __restrict__ ws, int64_t n, float factor,
                                       void* __restrict__ out0, void* __restrict__ out1) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float mx = apply_factor<D>(__uint_as_float(ws[i]), factor);
  if constexpr (CAL == QWIX_MINMAX) {
    const float mn = apply_factor<D>(-__uint_as_float(ws[n + i]), factor);
    store1<D>(out0, i, mn);
    store1<D>(out1, i, mx);
  } else {
    store1<D>(out0, i, mx);
  }
}

// Pass 2.  SRC 0: scale from ws (written out by chunk 0); SRC 1: scale given; SRC 2: the whole
// scale group (at most 128 rows) lies inside this block, which then calibrates on its own registers:
// one read of the input, no workspace, no atomics.
template <typename D, int QT, int CAL, int LAYOUT, int SRC>
__global__ void __launch_bounds__(256)
    cols_quantize_kernel(const uint8_t* __restrict__ x, ColGeom gm, const uint32_t* __restrict__ ws,
                         float factor, uint8_t* __restrict__ q, void* __restrict__ scale,
                         int8_t* __restrict__ zp) {
  constexpr int EV = D::kVec;
  constexpr bool ASYM = (CAL == QWIX_MINMAX);
  __shared__ float red[SRC == 2 ? 2 : 1][SRC == 2 ? 4 : 1][SRC == 2 ? 16 : 1][EV];
  int64_t o, t, c0;
  int chunk;
  // After a calibration pass over the same array the blocks run in the opposite order: what that pass read
  // last is what the last-level cache still holds, so it is re-read first.
  col_decode<D>(gm, SRC == 0 ? gridDim.x - 1 - blockIdx.x : blockIdx.x, &o, &t, &chunk, &c0);
  const bool col_ok = c0 < gm.inner;  // idle threads stay for the barriers
  const int rb = threadIdx.x >> 4;
  const int64_t sidx = (o * gm.ntiles + t) * gm.inner + c0;
  const int64_t row_end = (t + 1) * gm.tile;
  const int64_t r0 = t * gm.tile + chunk * 128 + rb * 8;
  float v[8][EV];
  uint4 raw[8];
  // The loads are issued before the scales are fetched, so that the two round trips overlap.
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    raw[j] = make_uint4(0, 0, 0, 0);
    if (col_ok && r0 + j < row_end)
      raw[j] = *reinterpret_cast<const uint4*>(x + ((o * gm.reduce + r0 + j) * gm.inner + c0) * sizeof(typename D::storage));
  }
  auto load_rows = [&]() {
#pragma unroll
    for (int j = 0; j < 8; ++j) unpack16<D>(raw[j], v[j]);
  };
  float s[EV];
  int z[EV];
  if constexpr (SRC == 2) {
    load_rows();
    float mx[EV], mn[EV];
#pragma unroll
    for (int e = 0; e < EV; ++e) {
      mx[e] = mn[e] = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if constexpr (ASYM) {
          mx[e] = fmaxf(mx[e], v[j][e]);
          mn[e] = fminf(mn[e], v[j][e]);
        } else {
          mx[e] = absmax_acc(mx[e], v[j][e]);
        }
      }
      // lanes l, l^16, l^32 hold the same columns
      mx[e] = fmaxf(mx[e], __shfl_xor(mx[e], 16, 64));
      mx[e] = fmaxf(mx[e], __shfl_xor(mx[e], 32, 64));
      if constexpr (ASYM) {
        mn[e] = fminf(mn[e], __shfl_xor(mn[e], 16, 64));
        mn[e] = fminf(mn[e], __shfl_xor(mn[e], 32, 64));
      }
    }
    const int tc = threadIdx.x & 15;
    if ((threadIdx.x & 63) < 16) {
#pragma unroll
      for (int e = 0; e < EV; ++e) {
        red[0][threadIdx.x >> 6][tc][e] = mx[e];
        if constexpr (ASYM) red[1][threadIdx.x >> 6][tc][e] = mn[e];
      }
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < EV; ++e) {
      z[e] = 0;
      const float a = apply_factor<D>(
          fmaxf(fmaxf(red[0][0][tc][e], red[0][1][tc][e]), fmaxf(red[0][2][tc][e], red[0][3][tc][e])), factor);
      if constexpr (ASYM) {
        const float b = apply_factor<D>(
            fminf(fminf(red[1][0][tc][e], red[1][1][tc][e]), fminf(red[1][2][tc][e], red[1][3][tc][e])), factor);
        s[e] = asym_scale_zp<D, QT>(b, a, &z[e]);
      } else {
        s[e] = sym_scale<D, QT>(a);
      }
      if (rb == 0 && col_ok) {
        store1<D>(scale, sidx + e, s[e]);
        if constexpr (ASYM) zp[sidx + e] = static_cast<int8_t>(z[e]);
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < EV; ++e) {
      z[e] = 0;
      s[e] = 1.f;
      if (!col_ok) continue;
      if constexpr (SRC == 0) {
        const float mx = apply_factor<D>(__uint_as_float(ws[sidx + e]), factor);
        if constexpr (ASYM) {
          const int64_t plane = gm.outer * gm.ntiles * gm.inner;
          const float mn = apply_factor<D>(-__uint_as_float(ws[plane + sidx + e]), factor);
          s[e] = asym_scale_zp<D, QT>(mn, mx, &z[e]);
        } else {
          s[e] = sym_scale<D, QT>(mx);
        }
        if (chunk == 0 && rb == 0) {
          store1<D>(scale, sidx + e, s[e]);
          if constexpr (ASYM) zp[sidx + e] = static_cast<int8_t>(z[e]);
        }
      } else {
        s[e] = load1<D>(scale, sidx + e);
        if constexpr (ASYM) z[e] = zp[sidx + e];
      }
    }
    load_rows();
  }
#pragma unroll
  for (int e = 0; e < EV; ++e) {
    const Divider<D, SRC == 1, QT == QWIX_E4M3> div(s[e]);
    const float zf = static_cast<float>(z[e]);
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      div.pair(v[j][e], v[j + 1][e]);
      if constexpr (ASYM) {
        v[j][e] += zf;
        v[j + 1][e] += zf;
        if constexpr (D::kTag == QWIX_BF16) round_bf16_pair(v[j][e], v[j + 1][e]);
      }
    }
  }
  constexpr bool kBounded = !(SRC == 1 && QT == QWIX_E4M3);  // a given scale: NaN inputs stay NaN in e4m3
  if constexpr (LAYOUT == QWIX_LAYOUT_NATURAL) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (col_ok && r0 + j < row_end) store_q<QT, EV, kBounded>(v[j], q, (o * gm.reduce + r0 + j) * gm.inner + c0);
  } else {
    // (outer, inner, reduce): the block's 128 rows x 128 columns leave as 128 column pieces of 128 rows.
    // A thread's 8 rows of one column are 8 consecutive output bytes, but a direct store would scatter
    // 32-byte pieces over 128 output rows; staged through LDS the block writes whole 128-byte pieces.
    constexpr int ROW_EL = 128 + 16;                       // staged row pitch in elements (keeps 8-byte alignment)
    constexpr int EPB = (QT == QWIX_INT4) ? 2 : 1;         // elements per byte
    __shared__ __attribute__((aligned(16))) uint8_t stage[16 * EV * ROW_EL / EPB];
    const int tc = threadIdx.x & 15;
#pragma unroll
    for (int e = 0; e < EV; ++e) {
      float col[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) col[j] = v[j][e];
      store_q<QT, 8, kBounded>(col, stage, (tc * EV + e) * ROW_EL + rb * 8);
    }
    __syncthreads();
    // 16-byte pieces: piece p of column c covers rows 16*EPB*p .. of this block
    constexpr int PIECES = 128 / (16 * EPB);
    const int64_t row0 = t * gm.tile + chunk * 128;
    const int64_t cb0 = c0 - tc * EV;                      // first column of the block
    const bool vec = (gm.reduce % (16 * EPB) == 0) && (row0 % (16 * EPB) == 0);
    for (int i = threadIdx.x; i < 16 * EV * PIECES; i += 256) {
      const int c = i / PIECES, pc = i % PIECES;
      const int64_t col = cb0 + c, r = row0 + pc * 16 * EPB;
      if (col >= gm.inner || r >= row_end) continue;
      const uint8_t* src = stage + (c * ROW_EL + pc * 16 * EPB) / EPB;
      uint8_t* dst = q + ((o * gm.inner + col) * gm.reduce + r) / EPB;
      if (vec && r + 16 * EPB <= row_end) {
        nt_store16(reinterpret_cast<uint4*>(dst), *reinterpret_cast<const uint4*>(src));
      } else {
        const int nb = static_cast<int>((min(row_end, r + 16 * EPB) - r + EPB - 1) / EPB);
        for (int k = 0; k < nb; ++k) dst[k] = src[k];
      }
    }
  }
}

// ------------------------------------------------------------------------------------ generic 5-D
struct Geom5 {
  int64_t d[5];   // d0, r1, d2, r3, d4
  int64_t t1, t3; // tiles of r1 and r3
};
__device__ __forceinline__ int64_t scale_index5(const Geom5& g, int64_t i0, int64_t i1, int64_t i2,
                                                int64_t i3, int64_t i4) {
  const int64_t n1 = g.d[1] / g.t1, n3 = g.d[3] / g.t3;
  return (((i0 * n1 + i1 / g.t1) * g.d[2] + i2) * n3 + i3 / g.t3) * g.d[4] + i4;
}

template <typename D, int QT, int CAL>
__global__ void generic_scale_kernel(const void* __restrict__ x, Geom5 g, float factor,
                                     void* __restrict__ scale, int8_t* __restrict__ zp) {
  const int64_t n1 = g.d[1] / g.t1, n3 = g.d[3] / g.t3;
  const int64_t ns = g.d[0] * n1 * g.d[2] * n3 * g.d[4];
  int64_t si = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (si >= ns) return;
  int64_t r = si;
  const int64_t i4 = r % g.d[4]; r /= g.d[4];
  const int64_t j3 = r % n3; r /= n3;
  const int64_t i2 = r % g.d[2]; r /= g.d[2];
  const int64_t j1 = r % n1;
  const int64_t i0 = r / n1;
  float mx = 0.f, mn = 0.f;
  for (int64_t a = 0; a < g.t1; ++a)
    for (int64_t b = 0; b < g.t3; ++b) {
      const int64_t idx = ((((i0 * g.d[1]) + j1 * g.t1 + a) * g.d[2] + i2) * g.d[3] + j3 * g.t3 + b) * g.d[4] + i4;
      const float v = load1<D>(x, idx);
      if constexpr (CAL == QWIX_MINMAX) {
        mx = fmaxf(mx, v);
        mn = fminf(mn, v);
      } else {
        mx = absmax_acc(mx, v);
      }
    }
  mx = apply_factor<D>(mx, factor);
  if constexpr (CAL == QWIX_MINMAX) {
    mn = apply_factor<D>(mn, factor);
    int z;
    const float s = asym_scale_zp<D, QT>(mn, mx, &z);
    store1<D>(scale, si, s);
    zp[si] = static_cast<int8_t>(z);
  } else {
    store1<D>(scale, si, sym_scale<D, QT>(mx));
  }
}

// One thread per output byte (two elements for int4, along the innermost flattened axis).
template <typename D, int QT, int CAL>
__global__ void generic_quant_kernel(const void* __restrict__ x, Geom5 g, const void* __restrict__ scale,
                                     const int8_t* __restrict__ zp, uint8_t* __restrict__ q) {
  constexpr int PER = (QT == QWIX_INT4) ? 2 : 1;
  const int64_t n = g.d[0] * g.d[1] * g.d[2] * g.d[3] * g.d[4];
  const int64_t bi = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (bi * PER >= n) return;
  float t[PER];
#pragma unroll
  for (int p = 0; p < PER; ++p) {
    int64_t r = bi * PER + p;
    const int64_t i4 = r % g.d[4]; r /= g.d[4];
    const int64_t i3 = r % g.d[3]; r /= g.d[3];
    const int64_t i2 = r % g.d[2]; r /= g.d[2];
    const int64_t i1 = r % g.d[1];
    const int64_t i0 = r / g.d[1];
    const int64_t si = scale_index5(g, i0, i1, i2, i3, i4);
    const Divider<D, true> div(load1<D>(scale, si));
    t[p] = div(load1<D>(x, bi * PER + p));
    if constexpr (CAL == QWIX_MINMAX) t[p] = rnd<D>(t[p] + static_cast<float>(zp[si]));
  }
  if constexpr (QT == QWIX_INT4)
    q[bi] = static_cast<uint8_t>(pack2_i4(to_int_q<QT>(t[0]), to_int_q<QT>(t[1])));
  else
    q[bi] = q_byte<QT>(t[0]);
}

// ------------------------------------------------------------------------------------ 2-D blocks
// Scale groups that are t1 x t3 blocks of a matrix whose rows are `row_stride` elements apart (the 5-D
// geometry with d4 == 1): 2^log2g threads hold one block in registers, read row piece by row piece with
// 16-byte loads, so the array is read once and written once like the contiguous-segment kernel does.
struct BlockGeom {
  int64_t nblk;        // d0 * n1 * d2 * n3 = number of scales
  int64_t row_stride;  // d2 * r3 elements between consecutive rows of a block
  int64_t r1, r3;
  uint32_t n1, d2, n3; // blocks along r1, middle kept axis, blocks along r3
  uint32_t t1, t3;
  uint32_t vpr;        // 16-byte vectors per block row
  uint32_t vpr_magic;  // ceil(2^32 / vpr): v / vpr == (v * magic) >> 32 for v, vpr < 2^16 (unused when vpr == 1)
  int nvec, log2g;
};

template <typename D, int QT, int CAL, int NL>
__global__ void __launch_bounds__(256)
    blocks_kernel(const uint8_t* __restrict__ x, BlockGeom gm, float factor, uint8_t* __restrict__ q,
                  void* __restrict__ scale, int8_t* __restrict__ zp) {
  constexpr int EV = D::kVec;
  constexpr bool ASYM = (CAL == QWIX_MINMAX);
  __shared__ float red[2][4];
  const int tid = threadIdx.x;
  const int log2g = gm.log2g, g = 1 << log2g;
  const int64_t blk = (static_cast<int64_t>(blockIdx.x) << (8 - log2g)) + (tid >> log2g);
  const int lane = tid & (g - 1);
  const bool blk_ok = blk < gm.nblk;
  int64_t base = 0;  // first element of the block
  if (blk_ok) {
    const uint32_t b = static_cast<uint32_t>(blk);
    const uint32_t j3 = b % gm.n3, r = b / gm.n3;
    const uint32_t i2 = r % gm.d2, r2 = r / gm.d2;
    const uint32_t j1 = r2 % gm.n1, i0 = r2 / gm.n1;
    base = ((static_cast<int64_t>(i0) * gm.r1 + static_cast<int64_t>(j1) * gm.t1) * gm.d2 + i2) * gm.r3 +
           static_cast<int64_t>(j3) * gm.t3;
  }
  int64_t off[NL];  // element offset of each vector this thread owns
  uint4 raw[NL];
#pragma unroll
  for (int j = 0; j < NL; ++j) {
    const uint32_t v = lane + (j << log2g);
    const uint32_t row = gm.vpr == 1 ? v : static_cast<uint32_t>((static_cast<uint64_t>(v) * gm.vpr_magic) >> 32);
    off[j] = base + static_cast<int64_t>(row) * gm.row_stride + static_cast<int64_t>(v - row * gm.vpr) * EV;
    raw[j] = make_uint4(0, 0, 0, 0);
    if (blk_ok && static_cast<int>(v) < gm.nvec)
      raw[j] = *reinterpret_cast<const uint4*>(x + off[j] * sizeof(typename D::storage));
  }
#pragma unroll
  for (int j = 0; j < NL; ++j) asm volatile("" : "+v"(raw[j].x), "+v"(raw[j].y), "+v"(raw[j].z), "+v"(raw[j].w));

  float mx = 0.f, mn = 0.f;
  if constexpr (!ASYM && D::kTag == QWIX_BF16) {
    u16x2 m = {0, 0};
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
      for (int e = 0; e < 4; ++e) m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2, w[e] & 0x7FFF7FFFu));
    }
    mx = bf16_bits_to_f32(m[0] > m[1] ? m[0] : m[1]);
  } else {
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      float f[EV];
      unpack16<D>(raw[j], f);
#pragma unroll
      for (int e = 0; e < EV; ++e) {
        if constexpr (ASYM) {
          mx = fmaxf(mx, f[e]);
          mn = fminf(mn, f[e]);
        } else {
          mx = absmax_acc(mx, f[e]);
        }
      }
    }
  }
  mx = wave_xor_max(mx, g < 64 ? g : 64);
  if constexpr (ASYM) mn = wave_xor_min(mn, g < 64 ? g : 64);
  if (g > 64) {  // uniform branch: a block spans 2 or 4 wavefronts
    const int w = tid >> 6;
    if ((tid & 63) == 0) {
      red[0][w] = mx;
      red[1][w] = mn;
    }
    __syncthreads();
    const int w0 = (tid >> log2g) << (log2g - 6), nw = 1 << (log2g - 6);
    mx = red[0][w0];
    mn = red[1][w0];
    for (int i = 1; i < nw; ++i) {
      mx = fmaxf(mx, red[0][w0 + i]);
      mn = fminf(mn, red[1][w0 + i]);
    }
  }
  mx = apply_factor<D>(mx, factor);
  float s;
  int z = 0;
  if constexpr (ASYM) {
    mn = apply_factor<D>(mn, factor);
    s = asym_scale_zp<D, QT>(mn, mx, &z);
  } else {
    s = sym_scale<D, QT>(mx);
  }
  if (blk_ok && lane == 0) {
    store1<D>(scale, blk, s);
    if constexpr (ASYM) zp[blk] = static_cast<int8_t>(z);
  }
  const float zf = static_cast<float>(z);
  const Divider<D, false, false> div(s);  // the sign of a zero quotient is restored below
#pragma unroll
  for (int j = 0; j < NL; ++j) {
    const int v = lane + (j << log2g);
    if (blk_ok && v < gm.nvec) {
      float t[EV];
      unpack16<D>(raw[j], t);
#pragma unroll
      for (int e = 0; e < EV; e += 2) {
        div.pair_unsigned(t[e], t[e + 1]);
        if constexpr (ASYM) {
          t[e] += zf;
          t[e + 1] += zf;
          if constexpr (D::kTag == QWIX_BF16) round_bf16_pair(t[e], t[e + 1]);
        }
      }
      if constexpr (QT == QWIX_E4M3 && D::kTag == QWIX_BF16) {
        const uint32_t signs[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
        store_q<QT, EV, true>(t, q, off[j], signs);
      } else {
        store_q<QT, EV, true>(t, q, off[j]);
      }
    }
  }
}

// rms calibration (qarray.py:511-515): sqrt(mean(x^2)) * factor per scale group, every step rounded to the
// array dtype the way jnp does it (squares in D, the mean summed in f32 and cast to D, the root in D).  One
// wavefront per group over the 5-D geometry; a rarely used method, kept simple rather than coalesced.
template <typename D>
__global__ void __launch_bounds__(256)
    rms_kernel(const void* __restrict__ x, Geom5 g, float factor, void* __restrict__ out) {
  const int64_t n1 = g.d[1] / g.t1, n3 = g.d[3] / g.t3;
  const int64_t ns = g.d[0] * n1 * g.d[2] * n3 * g.d[4];
  const int64_t si = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (si >= ns) return;
  int64_t r = si;
  const int64_t i4 = r % g.d[4]; r /= g.d[4];
  const int64_t j3 = r % n3; r /= n3;
  const int64_t i2 = r % g.d[2]; r /= g.d[2];
  const int64_t j1 = r % n1;
  const int64_t i0 = r / n1;
  const int64_t count = g.t1 * g.t3;
  float sum = 0.f;
  for (int64_t e = lane; e < count; e += 64) {
    const int64_t a = e / g.t3, b = e % g.t3;
    const int64_t idx = ((((i0 * g.d[1]) + j1 * g.t1 + a) * g.d[2] + i2) * g.d[3] + j3 * g.t3 + b) * g.d[4] + i4;
    const float v = load1<D>(x, idx);
    sum += rnd<D>(v * v);
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, 64);
  if (lane != 0) return;
  const float mean = rnd<D>(sum / static_cast<float>(count));
  const float rms = rnd<D>(__builtin_sqrtf(mean));
  store1<D>(out, si, rnd<D>(rms * rnd<D>(factor)));
}

// ------------------------------------------------------------------------------------ misc
// Quantize with a given scale and noise before the rounding (stochastic rounding, numerics.py:191-195): integer
// qtypes only; the quotient (and the zero point added to it) is formed in the array dtype as always, then widened to
// f32, the caller's f32 noise added, and the sum rounded half to even and saturated.  Natural layout, one thread per
// pair of consecutive elements; a training-time path, not tuned.
template <typename D, int QT, bool ASYM>
__global__ void __launch_bounds__(256)
    noise_quantize_kernel(const void* __restrict__ x, int64_t pairs, int64_t reduce, int64_t inner, int64_t tile,
                          const void* __restrict__ scale, const int8_t* __restrict__ zp, const float* __restrict__ noise,
                          uint8_t* __restrict__ q) {
  const int64_t ntile = reduce / tile;
  for (int64_t pr = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; pr < pairs; pr += static_cast<int64_t>(gridDim.x) * 256) {
    int v[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int64_t i = 2 * pr + h;
      const int64_t c = i % inner, r = (i / inner) % reduce, o = i / (inner * reduce);
      const int64_t si = (o * ntile + r / tile) * inner + c;
      const Divider<D, true, true> div(load1<D>(scale, si));
      float t = div(load1<D>(x, i));
      if constexpr (ASYM) t = rnd<D>(t + static_cast<float>(zp[si]));
      v[h] = to_int_q<QT>(t + noise[i]);
    }
    if constexpr (QT == QWIX_INT4) {
      q[pr] = static_cast<uint8_t>(pack2_i4(v[0], v[1]));
    } else {
      q[2 * pr] = static_cast<uint8_t>(v[0] & 0xFF);
      q[2 * pr + 1] = static_cast<uint8_t>(v[1] & 0xFF);
    }
  }
}

template <typename D, int QT, int CAL>
__global__ void scale_zp_kernel(const void* __restrict__ c0, const void* __restrict__ c1, int64_t n,
                                void* __restrict__ scale, int8_t* __restrict__ zp) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if constexpr (CAL == QWIX_MINMAX) {
    int z;
    const float s = asym_scale_zp<D, QT>(load1<D>(c0, i), load1<D>(c1, i), &z);
    store1<D>(scale, i, s);
    zp[i] = static_cast<int8_t>(z);
  } else {
    store1<D>(scale, i, sym_scale<D, QT>(load1<D>(c0, i)));
  }
}

// out[(o, r, i)] = D(D(q - zp) * s).  One thread per element; layouts as documented.
template <typename D, int QT>
__global__ void dequant_kernel(const uint8_t* __restrict__ q, int layout, int64_t outer, int64_t reduce,
                               int64_t inner, int64_t tile, const void* __restrict__ scale,
                               const int8_t* __restrict__ zp, void* __restrict__ out) {
  const int64_t n = outer * reduce * inner;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const int64_t i = idx % inner, r = (idx / inner) % reduce, o = idx / (inner * reduce);
  const int64_t qi = layout == QWIX_LAYOUT_NATURAL ? idx : (o * inner + i) * reduce + r;
  float v;
  if constexpr (QT == QWIX_INT8) {
    v = static_cast<float>(reinterpret_cast<const int8_t*>(q)[qi]);
  } else if constexpr (QT == QWIX_E4M3) {
    v = e4m3_to_f32(q[qi]);
  } else {
    const int nib = (q[qi >> 1] >> ((qi & 1) * 4)) & 0xF;
    v = static_cast<float>((nib ^ 8) - 8);
  }
  const int64_t si = (o * (reduce / tile) + r / tile) * inner + i;
  v = rnd<D>(v);
  if (zp != nullptr) v = rnd<D>(v - rnd<D>(static_cast<float>(zp[si])));
  store1<D>(out, idx, rnd<D>(v * load1<D>(scale, si)));
}

// Quantized byte (or nibble) -> float, as dequant_kernel does it.
template <int QT>
__device__ __forceinline__ float q_to_f32(uint32_t b) {
  if constexpr (QT == QWIX_INT8) return static_cast<float>(static_cast<int>(b << 24) >> 24);
  else if constexpr (QT == QWIX_E4M3) return e4m3_to_f32(b & 0xFF);
  else return static_cast<float>(static_cast<int>((b & 0xF) ^ 8) - 8);
}

// Store 8 consecutive values of D at element index i (a multiple of 8).
template <typename D>
__device__ __forceinline__ void store8(void* out, int64_t i, const float* v) {
  if constexpr (D::kTag == QWIX_BF16) {
    uint4 w;
    w.x = f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16);
    w.y = f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16);
    w.z = f32_to_bf16_bits(v[4]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[5])) << 16);
    w.w = f32_to_bf16_bits(v[6]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[7])) << 16);
    *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(out) + i) = w;
  } else {
    float4* o = reinterpret_cast<float4*>(reinterpret_cast<float*>(out) + i);
    o[0] = make_float4(v[0], v[1], v[2], v[3]);
    o[1] = make_float4(v[4], v[5], v[6], v[7]);
  }
}

// Natural layout, 8 consecutive elements (along the innermost axis) per thread.  inner == 1: the 8 share a
// scale (tile % 8 == 0); inner > 1: they take 8 consecutive scales (inner % 8 == 0).
template <typename D, int QT>
__global__ void __launch_bounds__(256)
    dequant_vec_kernel(const uint8_t* __restrict__ q, int64_t outer, int64_t reduce, int64_t inner, int64_t tile,
                       const void* __restrict__ scale, const int8_t* __restrict__ zp, void* __restrict__ out) {
  const int64_t n = outer * reduce * inner;
  const int64_t idx = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 8;
  if (idx >= n) return;
  uint32_t b[8];
  if constexpr (QT == QWIX_INT4) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(q + idx / 2);
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] = (w >> (4 * e)) & 0xF;
  } else {
    const uint2 w = *reinterpret_cast<const uint2*>(q + idx);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      b[e] = (w.x >> (8 * e)) & 0xFF;
      b[4 + e] = (w.y >> (8 * e)) & 0xFF;
    }
  }
  float s[8], z[8];
  if (inner == 1) {
    const int64_t si = idx / tile;
    const float sv = load1<D>(scale, si);
    const float zv = zp ? rnd<D>(static_cast<float>(zp[si])) : 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      s[e] = sv;
      z[e] = zv;
    }
  } else {
    const int64_t i = idx % inner, rest = idx / inner, r = rest % reduce, o = rest / reduce;
    const int64_t si = (o * (reduce / tile) + r / tile) * inner + i;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      s[e] = load1<D>(scale, si + e);
      z[e] = zp ? rnd<D>(static_cast<float>(zp[si + e])) : 0.f;
    }
  }
  float v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float t = rnd<D>(q_to_f32<QT>(b[e]));
    if (zp != nullptr) t = rnd<D>(t - z[e]);
    v[e] = rnd<D>(t * s[e]);
  }
  store8<D>(out, idx, v);
}

// Reduce-minor in, reduce-minor out: element (o, i, r) of the (outer, inner, reduce) array; 8 consecutive r per
// thread share a scale (tile % 8 == 0).  The result is the K-contiguous float operand of the bf16 GEMM.
template <typename D, int QT, typename OD>
__global__ void __launch_bounds__(256)
    dequant_keep_rm_kernel(const uint8_t* __restrict__ q, int64_t outer, int64_t reduce, int64_t inner, int64_t tile,
                           const void* __restrict__ scale, const int8_t* __restrict__ zp, void* __restrict__ out) {
  const int64_t n = outer * reduce * inner;
  const int64_t idx = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 8;
  if (idx >= n) return;
  uint32_t b[8];
  if constexpr (QT == QWIX_INT4) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(q + idx / 2);
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] = (w >> (4 * e)) & 0xF;
  } else {
    const uint2 w = *reinterpret_cast<const uint2*>(q + idx);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      b[e] = (w.x >> (8 * e)) & 0xFF;
      b[4 + e] = (w.y >> (8 * e)) & 0xFF;
    }
  }
  const int64_t r = idx % reduce, rest = idx / reduce, i = rest % inner, o = rest / inner;
  const int64_t si = (o * (reduce / tile) + r / tile) * inner + i;
  const float sv = load1<D>(scale, si);
  const float zv = zp ? rnd<D>(static_cast<float>(zp[si])) : 0.f;
  float v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float t = rnd<D>(q_to_f32<QT>(b[e]));
    if (zp != nullptr) t = rnd<D>(t - zv);
    v[e] = rnd<D>(t * sv);
  }
  store8<OD>(out, idx, v);  // bf16 out of f32 values: one more rounding, what casting the f32 array gives
}

// Dequantize for the 5-D geometry (two reduced axis groups: block scales).  VEC = 8: eight consecutive elements
// of the innermost reduced axis share a scale (d4 == 1, t3 % 8 == 0); VEC = 1: anything.
template <typename D, int QT, int VEC>
__global__ void __launch_bounds__(256)
    generic_dequant_kernel(const uint8_t* __restrict__ q, Geom5 g, const void* __restrict__ scale,
                           const int8_t* __restrict__ zp, void* __restrict__ out) {
  const int64_t n = g.d[0] * g.d[1] * g.d[2] * g.d[3] * g.d[4];
  const int64_t idx = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * VEC;
  if (idx >= n) return;
  int64_t r = idx;
  const int64_t i4 = r % g.d[4]; r /= g.d[4];
  const int64_t i3 = r % g.d[3]; r /= g.d[3];
  const int64_t i2 = r % g.d[2]; r /= g.d[2];
  const int64_t i1 = r % g.d[1];
  const int64_t i0 = r / g.d[1];
  const int64_t si = scale_index5(g, i0, i1, i2, i3, i4);
  const float sv = load1<D>(scale, si);
  const float zv = zp ? rnd<D>(static_cast<float>(zp[si])) : 0.f;
  uint32_t b[VEC];
  if constexpr (VEC == 8) {
    if constexpr (QT == QWIX_INT4) {
      const uint32_t w = *reinterpret_cast<const uint32_t*>(q + idx / 2);
#pragma unroll
      for (int e = 0; e < 8; ++e) b[e] = (w >> (4 * e)) & 0xF;
    } else {
      const uint2 w = *reinterpret_cast<const uint2*>(q + idx);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        b[e] = (w.x >> (8 * e)) & 0xFF;
        b[4 + e] = (w.y >> (8 * e)) & 0xFF;
      }
    }
  } else {
    if constexpr (QT == QWIX_INT4) b[0] = (q[idx / 2] >> (4 * (idx & 1))) & 0xF;
    else b[0] = q[idx];
  }
  float v[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    float t = rnd<D>(q_to_f32<QT>(b[e]));
    if (zp != nullptr) t = rnd<D>(t - zv);
    v[e] = rnd<D>(t * sv);
  }
  if constexpr (VEC == 8) store8<D>(out, idx, v);
  else store1<D>(out, idx, v[0]);
}

// Reduce-minor layout (values stored (outer, inner, reduce), output (outer, reduce, inner)): a 64 x 64 tile is
// read along the reduced axis, turned in LDS, and written along the inner axis with its scales, 16 per thread.
template <typename D, int QT>
__global__ void __launch_bounds__(256)
    dequant_rm_kernel(const uint8_t* __restrict__ q, int64_t reduce, int64_t inner, int64_t tile,
                      const void* __restrict__ scale, const int8_t* __restrict__ zp, void* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) uint8_t turned[64][80];  // [r][i], rows padded to 80 bytes
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * 64, i0 = static_cast<int64_t>(blockIdx.y) * 64;
  const int64_t o = blockIdx.z;
  const int t = threadIdx.x;
  {  // 64 rows (i) x 64 values (r): 16 values per thread
    const int il = t >> 2, rc = (t & 3) * 16;
    const int64_t i = i0 + il, r = r0 + rc;
    uint32_t w[4] = {0, 0, 0, 0};
    if (i < inner && r < reduce) {
      const int64_t e = (o * inner + i) * reduce + r;
      if constexpr (QT == QWIX_INT4) {
        const uint2 p = *reinterpret_cast<const uint2*>(q + e / 2);
        w[0] = p.x;
        w[1] = p.y;
      } else {
        const uint4 p = *reinterpret_cast<const uint4*>(q + e);
        w[0] = p.x; w[1] = p.y; w[2] = p.z; w[3] = p.w;
      }
    }
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      uint32_t b;
      if constexpr (QT == QWIX_INT4) b = (w[k >> 3] >> (4 * (k & 7))) & 0xF;
      else b = (w[k >> 2] >> (8 * (k & 3))) & 0xFF;
      turned[rc + k][il] = static_cast<uint8_t>(b);
    }
  }
  __syncthreads();
  const int rl = t >> 2, ic = (t & 3) * 16;
  const int64_t r = r0 + rl, i = i0 + ic;
  if (r >= reduce || i >= inner) return;
  const uint4 pk = *reinterpret_cast<const uint4*>(&turned[rl][ic]);
  const uint32_t w[4] = {pk.x, pk.y, pk.z, pk.w};
  const int64_t si = (o * (reduce / tile) + r / tile) * inner + i;
  const int64_t oi = (o * reduce + r) * inner + i;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int k = 8 * h + e;
      float x = rnd<D>(q_to_f32<QT>((w[k >> 2] >> (8 * (k & 3))) & 0xFF));
      if (zp != nullptr) x = rnd<D>(x - rnd<D>(static_cast<float>(zp[si + k])));
      v[e] = rnd<D>(x * load1<D>(scale, si + k));
    }
    store8<D>(out, oi + 8 * h, v);
  }
}

// (rows, cols) elements -> (cols, rows); int4 repacks along the new minor axis.
template <int QT>
__global__ void __launch_bounds__(256)
    transpose_q_kernel(const uint8_t* __restrict__ src, int64_t rows, int64_t cols, uint8_t* __restrict__ dst) {
  __shared__ uint8_t tile[64][65];
  const int64_t r0 = static_cast<int64_t>(blockIdx.y) * 64, c0 = static_cast<int64_t>(blockIdx.x) * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
  for (int j = ty; j < 64; j += 4) {
    const int64_t r = r0 + j, c = c0 + tx;
    uint8_t v = 0;
    if (r < rows && c < cols) {
      if constexpr (QT == QWIX_INT4) {
        const int64_t e = r * cols + c;
        v = (src[e >> 1] >> ((e & 1) * 4)) & 0xF;
      } else {
        v = src[r * cols + c];
      }
    }
    tile[j][tx] = v;
  }
  __syncthreads();
  if constexpr (QT == QWIX_INT4) {
    // thread -> (new row = old col, pair of old rows)
    const int px = threadIdx.x & 31, py = threadIdx.x >> 5;  // 32 pairs x 8
    for (int j = py; j < 64; j += 8) {
      const int64_t nr = c0 + j, nc = r0 + 2 * px;
      if (nr < cols && nc < rows) {
        const uint8_t lo = tile[2 * px][j], hi = (nc + 1 < rows) ? tile[2 * px + 1][j] : 0;
        dst[(nr * rows + nc) >> 1] = static_cast<uint8_t>(lo | (hi << 4));
      }
    }
  } else {
    for (int j = ty; j < 64; j += 4) {
      const int64_t nr = c0 + j, nc = r0 + tx;
      if (nr < cols && nc < rows) dst[nr * rows + nc] = tile[tx][j];
    }
  }
}

// ------------------------------------------------------------------------------------ dispatch
inline int log2_ceil(int64_t v) {
  int l = 0;
  while ((int64_t{1} << l) < v) ++l;
  return l;
}

#define QWIX_DISPATCH_D(dtype, ...)                                         \
  if ((dtype) == QWIX_F32) { using D = F32; __VA_ARGS__ }                   \
  else if ((dtype) == QWIX_BF16) { using D = BF16; __VA_ARGS__ }            \
  else return fail(QWIX_ERR_INVALID_ARGUMENT, "dtype %d is not f32/bf16", (dtype));

#define QWIX_DISPATCH_QT_CAL(qtype, cal, ...)                                                   \
  if ((qtype) == QWIX_INT8 && (cal) == QWIX_ABSMAX) { constexpr int QT = QWIX_INT8, CAL = QWIX_ABSMAX; __VA_ARGS__ } \
  else if ((qtype) == QWIX_INT4 && (cal) == QWIX_ABSMAX) { constexpr int QT = QWIX_INT4, CAL = QWIX_ABSMAX; __VA_ARGS__ } \
  else if ((qtype) == QWIX_E4M3 && (cal) == QWIX_ABSMAX) { constexpr int QT = QWIX_E4M3, CAL = QWIX_ABSMAX; __VA_ARGS__ } \
  else if ((qtype) == QWIX_INT8 && (cal) == QWIX_MINMAX) { constexpr int QT = QWIX_INT8, CAL = QWIX_MINMAX; __VA_ARGS__ } \
  else if ((qtype) == QWIX_INT4 && (cal) == QWIX_MINMAX) { constexpr int QT = QWIX_INT4, CAL = QWIX_MINMAX; __VA_ARGS__ } \
  else return fail(QWIX_ERR_INVALID_ARGUMENT, "qtype %d / calibration %d unsupported (asymmetric needs int8/int4)", (qtype), (cal));

int check_geom(int64_t outer, int64_t reduce, int64_t inner, int64_t tile) {
  if (outer <= 0 || reduce <= 0 || inner <= 0 || tile <= 0)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "non-positive dimension (outer=%lld reduce=%lld inner=%lld tile=%lld)",
                (long long)outer, (long long)reduce, (long long)inner, (long long)tile);
  if (reduce % tile != 0)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "tile %lld does not divide the reduced axis %lld", (long long)tile,
                (long long)reduce);
  return QWIX_OK;
}

ColGeom make_col_geom(int64_t outer, int64_t reduce, int64_t inner, int64_t tile, int ev) {
  ColGeom g;
  g.outer = outer; g.reduce = reduce; g.inner = inner; g.tile = tile; g.ntiles = reduce / tile;
  g.chunks_per_tile = static_cast<int>((tile + 127) / 128);
  g.col_blocks = static_cast<int>((inner + 16 * ev - 1) / (16 * ev));
  return g;
}

// Pieces a long contiguous segment of L elements is cut into: the smallest count that divides L into
// pieces of at most 8192 elements that are multiples of 8 (one rule for both array dtypes, so that the
// workspace size does not depend on the dtype).  0: no such cut (the strided kernel takes the segment).
int64_t row_pieces(int64_t L) {
  constexpr int64_t kMaxPiece = 8192;
  if (L <= kMaxPiece || L % 8) return 0;
  for (int64_t r = (L + kMaxPiece - 1) / kMaxPiece; r <= (int64_t{1} << 20) && r * 8 <= L; ++r)
    if (L % r == 0 && (L / r) % 8 == 0) return r;
  return 0;
}

template <typename D, int QT, int CAL, int MODE>
void launch_rows(const void* x, int64_t nseg, int64_t L, float factor, void* q, void* scale, void* zp, void* c0,
                 void* c1, int per_scale, hipStream_t st) {
  const int nvec = static_cast<int>(L / D::kVec);
  constexpr int target = 4;  // 16-byte loads per thread
  int lg = log2_ceil((nvec + target - 1) / target);  // aim at `target` loads per thread, 8 at most
  while ((nvec + (1 << lg) - 1) >> lg > 8) ++lg;
  if (lg > 8) lg = 8;
  const int64_t blocks = (nseg + (256 >> lg) - 1) / (256 >> lg);
  const int loads = (nvec + (1 << lg) - 1) >> lg;
  const dim3 grid(static_cast<unsigned>(blocks));
  const uint8_t* xb = static_cast<const uint8_t*>(x);
  uint8_t* qb = static_cast<uint8_t*>(q);
  int8_t* zb = static_cast<int8_t*>(zp);
  const int sh = (per_scale & (per_scale - 1)) == 0 ? log2_ceil(per_scale) : -1;
  if (loads <= 2)
    rows_kernel<D, QT, CAL, MODE, 2><<<grid, 256, 0, st>>>(xb, nseg, nvec, lg, factor, qb, scale, zb, c0, c1, per_scale, sh);
  else if (loads <= 4)
    rows_kernel<D, QT, CAL, MODE, 4><<<grid, 256, 0, st>>>(xb, nseg, nvec, lg, factor, qb, scale, zb, c0, c1, per_scale, sh);
  else
    rows_kernel<D, QT, CAL, MODE, 8><<<grid, 256, 0, st>>>(xb, nseg, nvec, lg, factor, qb, scale, zb, c0, c1, per_scale, sh);
}

// mode: MODE_QUANT / MODE_CALIB / MODE_GIVEN.  ws: scratch for segments longer than one workgroup holds
// in registers (qwix_hip_quantize_workspace_bytes says how much); not needed when the scale is given.
template <int MODE>
int run_rows(const void* x, int dtype, int64_t nseg, int64_t L, int qtype, int cal, float factor,
             void* q, void* scale, void* zp, void* c0, void* c1, void* ws, size_t ws_bytes, hipStream_t st) {
  QWIX_DISPATCH_D(dtype, {
    QWIX_DISPATCH_QT_CAL(qtype, cal, {
      const bool aligned = aligned16(x) && (MODE == MODE_CALIB || (reinterpret_cast<uintptr_t>(q) & 7) == 0);
      const bool vec_ok = (L % D::kVec == 0) && aligned && (L / D::kVec <= 2048);
      const int64_t pieces = aligned ? row_pieces(L) : 0;
      if (vec_ok) {
        launch_rows<D, QT, CAL, MODE>(x, nseg, L, factor, q, scale, zp, c0, c1, 1, st);
      } else if (pieces > 0 && pieces <= INT32_MAX) {
        // long segments: calibrate piece by piece, merge, then quantize the pieces with the merged scale
        const int64_t n = nseg * pieces, piece = L / pieces;
        if constexpr (MODE != MODE_GIVEN) {
          const size_t need = static_cast<size_t>(n) * 4u * (CAL == QWIX_MINMAX ? 2u : 1u);
          if (!ws || ws_bytes < need)
            return fail(QWIX_ERR_INVALID_ARGUMENT, "workspace of %zu bytes required, got %zu", need, ws_bytes);
          void* p0 = ws;
          void* p1 = static_cast<uint8_t*>(ws) + static_cast<size_t>(n) * 4u;
          launch_rows<D, QT, CAL, MODE_CALIB>(x, n, piece, factor, nullptr, nullptr, nullptr, p0, p1, 1, st);
          rows_merge_kernel<D, QT, CAL, MODE><<<dim3(static_cast<unsigned>((nseg + 3) / 4)), 256, 0, st>>>(
              p0, p1, nseg, static_cast<int>(pieces), scale, static_cast<int8_t*>(zp), c0, c1);
        }
        if constexpr (MODE != MODE_CALIB)
          launch_rows<D, QT, CAL, MODE_GIVEN>(x, n, piece, 0.f, q, scale, zp, nullptr, nullptr,
                                              static_cast<int>(pieces), st);
      } else {
        if (QT == QWIX_INT4 && MODE != MODE_CALIB && (L & 1))
          return fail(QWIX_ERR_UNSUPPORTED, "int4 needs an even contiguous length, got %lld", (long long)L);
        rows_loop_kernel<D, QT, CAL, MODE><<<dim3(static_cast<unsigned>(nseg)), 256, 0, st>>>(
            x, L, factor, static_cast<uint8_t*>(q), scale, static_cast<int8_t*>(zp), c0, c1);
      }
    })
  })
  return check_launch("rows quantize");
}

int run_cols_absmax(const void* x, int dtype, const ColGeom& g, int cal, uint32_t* ws, hipStream_t st) {
  const int64_t n = g.outer * g.ntiles * g.inner * (cal == QWIX_MINMAX ? 2 : 1);
  fill_u32_kernel<<<dim3(static_cast<unsigned>((n + 255) / 256)), 256, 0, st>>>(ws, n, 0u);
  if (g.tile >= kWideRows) {
    const int ev = dtype == QWIX_BF16 ? 8 : 4;
    const int wcb = static_cast<int>((g.inner + 64 * ev - 1) / (64 * ev));
    const int wch = static_cast<int>((g.tile + kWideRows - 1) / kWideRows);
    const int64_t wblocks = g.outer * g.ntiles * wch * wcb;
    if (wblocks <= INT32_MAX) {
      QWIX_DISPATCH_D(dtype, {
        if (cal == QWIX_MINMAX)
          cols_absmax_wide_kernel<D, QWIX_MINMAX><<<dim3(static_cast<unsigned>(wblocks)), 256, 0, st>>>(
              static_cast<const uint8_t*>(x), g, wcb, wch, ws);
        else
          cols_absmax_wide_kernel<D, QWIX_ABSMAX><<<dim3(static_cast<unsigned>(wblocks)), 256, 0, st>>>(
              static_cast<const uint8_t*>(x), g, wcb, wch, ws);
      })
      return check_launch("cols absmax");
    }
  }
  const int64_t blocks = g.outer * g.ntiles * g.chunks_per_tile * g.col_blocks;
  QWIX_DISPATCH_D(dtype, {
    if (cal == QWIX_MINMAX)
      cols_absmax_kernel<D, QWIX_MINMAX><<<dim3(static_cast<unsigned>(blocks)), 256, 0, st>>>(
          static_cast<const uint8_t*>(x), g, ws);
    else
      cols_absmax_kernel<D, QWIX_ABSMAX><<<dim3(static_cast<unsigned>(blocks)), 256, 0, st>>>(
          static_cast<const uint8_t*>(x), g, ws);
  })
  return check_launch("cols absmax");
}

template <int SRC>
int run_cols_quantize(const void* x, int dtype, const ColGeom& g, int qtype, int cal, int layout,
                      const uint32_t* ws, float factor, void* q, void* scale, void* zp, hipStream_t st) {
  const int64_t blocks = g.outer * g.ntiles * g.chunks_per_tile * g.col_blocks;
  QWIX_DISPATCH_D(dtype, {
    QWIX_DISPATCH_QT_CAL(qtype, cal, {
      if (layout == QWIX_LAYOUT_NATURAL)
        cols_quantize_kernel<D, QT, CAL, QWIX_LAYOUT_NATURAL, SRC><<<dim3(static_cast<unsigned>(blocks)), 256, 0, st>>>(
            static_cast<const uint8_t*>(x), g, ws, factor, static_cast<uint8_t*>(q), scale, static_cast<int8_t*>(zp));
      else
        cols_quantize_kernel<D, QT, CAL, QWIX_LAYOUT_REDUCE_MINOR, SRC><<<dim3(static_cast<unsigned>(blocks)), 256, 0, st>>>(
            static_cast<const uint8_t*>(x), g, ws, factor, static_cast<uint8_t*>(q), scale, static_cast<int8_t*>(zp));
    })
  })
  return check_launch("cols quantize");
}

int check_cols(const void* x, int dtype, int64_t reduce, int64_t inner, int64_t tile, int layout,
               const void* q) {
  const int ev = dtype == QWIX_BF16 ? 8 : 4;
  if (q != nullptr && !aligned16(q)) return fail(QWIX_ERR_INVALID_ARGUMENT, "qvalue must be 16-byte aligned");
  if (inner % ev != 0 || !aligned16(x))
    return fail(QWIX_ERR_UNSUPPORTED,
                "strided-reduce quantize needs inner %% %d == 0 and a 16-byte aligned input (inner=%lld); "
                "use qwix_hip_quantize_generic", ev, (long long)inner);
  if (layout == QWIX_LAYOUT_REDUCE_MINOR && (reduce % 8 != 0 || tile % 8 != 0))
    return fail(QWIX_ERR_UNSUPPORTED, "reduce-minor layout needs reduce and tile to be multiples of 8 (%lld, %lld)",
                (long long)reduce, (long long)tile);
  if (layout != QWIX_LAYOUT_NATURAL && layout != QWIX_LAYOUT_REDUCE_MINOR)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "unknown layout %d", layout);
  return QWIX_OK;
}

}  // namespace
}  // namespace qwix

using namespace qwix;

// ------------------------------------------------------------------------------------ static scratch
// Calibration scratch of qwix_hip_quantize_static: one array per GPU, held from the moment the code
// object is loaded on that GPU until the process ends.  `quantize_scratch` is only a host-side handle of
// the symbol; the device address differs per GPU and comes from hipGetSymbolAddress, once per device.
constexpr size_t kStaticScratchBytes = size_t{1} << 20;
static __device__ __align__(256) unsigned char quantize_scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxScratchDevices = 64;
std::mutex scratch_mutex;
void* scratch_ptr[kMaxScratchDevices] = {nullptr};

// Device address of the current device's copy of quantize_scratch (looked up on the first call on
// that device, cached afterwards), or nullptr with the error text set.
void* static_scratch() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxScratchDevices) {
    fail(QWIX_ERR_LAUNCH, "no current HIP device (or device index %d >= %d)", dev, kMaxScratchDevices);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(quantize_scratch));
    if (e != hipSuccess || p == nullptr) {
      fail(QWIX_ERR_LAUNCH, "hipGetSymbolAddress(quantize_scratch) on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    scratch_ptr[dev] = p;
  }
  return scratch_ptr[dev];
}
}  // namespace

extern "C" {

int qwix_hip_abi_version(void) { return 1; }
const char* qwix_hip_last_error(void) { return err_buf(); }

size_t qwix_hip_quantize_workspace_bytes(int64_t outer, int64_t reduce, int64_t inner, int64_t tile,
                                         int calibration) {
  if (tile <= 0 || reduce % tile != 0) return 0;
  const size_t per = 4u * (calibration == QWIX_MINMAX ? 2u : 1u);
  if (inner <= 1)  // contiguous segments: partial calibration values of the pieces of long segments
    return static_cast<size_t>(outer * (reduce / tile) * row_pieces(tile)) * per;
  return static_cast<size_t>(outer * (reduce / tile) * inner) * per;
}

int qwix_hip_quantize(const void* x, int dtype, int64_t outer, int64_t reduce, int64_t inner, int64_t tile,
                      int qtype, int calibration, float calib_factor, int q_layout, void* qvalue, void* scale,
                      void* zero_point, void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_geom(outer, reduce, inner, tile)) return e;
  if (!x || !qvalue || !scale) return fail(QWIX_ERR_INVALID_ARGUMENT, "null x/qvalue/scale");
  if (calibration == QWIX_MINMAX && !zero_point)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "minmax calibration needs a zero_point output");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (inner == 1)  // both layouts coincide
    return run_rows<MODE_QUANT>(x, dtype, outer * (reduce / tile), tile, qtype, calibration, calib_factor, qvalue,
                                scale, zero_point, nullptr, nullptr, workspace, workspace_bytes, st);
  if (int e = check_cols(x, dtype, reduce, inner, tile, q_layout, qvalue)) return e;
  const ColGeom g = make_col_geom(outer, reduce, inner, tile, dtype == QWIX_BF16 ? 8 : 4);
  if (g.chunks_per_tile == 1)  // a scale group fits one block: calibrate and quantize in one pass, no workspace
    return run_cols_quantize<2>(x, dtype, g, qtype, calibration, q_layout, nullptr, calib_factor, qvalue, scale,
                                zero_point, st);
  const size_t need = qwix_hip_quantize_workspace_bytes(outer, reduce, inner, tile, calibration);
  if (!workspace || workspace_bytes < need)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "workspace of %zu bytes required, got %zu", need, workspace_bytes);
  if (int e = run_cols_absmax(x, dtype, g, calibration, static_cast<uint32_t*>(workspace), st)) return e;
  return run_cols_quantize<0>(x, dtype, g, qtype, calibration, q_layout, static_cast<const uint32_t*>(workspace),
                              calib_factor, qvalue, scale, zero_point, st);
}

size_t qwix_hip_quantize_static_max_bytes(void) { return kStaticScratchBytes; }

int qwix_hip_quantize_static(const void* x, int dtype, int64_t outer, int64_t reduce, int64_t inner, int64_t tile,
                             int qtype, int calibration, float calib_factor, int q_layout, void* qvalue,
                             void* scale, void* zero_point, void* stream) {
  if (int e = check_geom(outer, reduce, inner, tile)) return e;
  const size_t need = qwix_hip_quantize_workspace_bytes(outer, reduce, inner, tile, calibration);
  if (need > kStaticScratchBytes)
    return fail(QWIX_ERR_UNSUPPORTED,
                "this shape needs %zu bytes of calibration scratch, the static buffer holds %zu: call "
                "qwix_hip_quantize with a workspace instead", need, kStaticScratchBytes);
  void* ws = static_scratch();  // device address of this GPU's array; never the symbol itself
  if (ws == nullptr) return QWIX_ERR_LAUNCH;
  // The kernels behind qwix_hip_quantize clear what they accumulate into (a fill kernel on `stream`), so
  // what an earlier call left in the array does not matter.
  return qwix_hip_quantize(x, dtype, outer, reduce, inner, tile, qtype, calibration, calib_factor, q_layout, qvalue,
                           scale, zero_point, ws, kStaticScratchBytes, stream);
}

int qwix_hip_calibrate(const void* x, int dtype, int64_t outer, int64_t reduce, int64_t inner, int64_t tile,
                       int calibration, float calib_factor, void* out0, void* out1, void* workspace,
                       size_t workspace_bytes, void* stream) {
  if (int e = check_geom(outer, reduce, inner, tile)) return e;
  if (!x || !out0 || (calibration == QWIX_MINMAX && !out1))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "null input or output");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (inner == 1)
    return run_rows<MODE_CALIB>(x, dtype, outer * (reduce / tile), tile, QWIX_INT8, calibration, calib_factor,
                                nullptr, nullptr, nullptr, out0, out1, workspace, workspace_bytes, st);
  if (int e = check_cols(x, dtype, reduce, inner, tile, QWIX_LAYOUT_NATURAL, nullptr)) return e;
  const size_t need = qwix_hip_quantize_workspace_bytes(outer, reduce, inner, tile, calibration);
  if (!workspace || workspace_bytes < need)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "workspace of %zu bytes required, got %zu", need, workspace_bytes);
  const ColGeom g = make_col_geom(outer, reduce, inner, tile, dtype == QWIX_BF16 ? 8 : 4);
  if (int e = run_cols_absmax(x, dtype, g, calibration, static_cast<uint32_t*>(workspace), st)) return e;
  const int64_t n = outer * (reduce / tile) * inner;
  QWIX_DISPATCH_D(dtype, {
    if (calibration == QWIX_MINMAX)
      cols_finish_cal_kernel<D, QWIX_MINMAX><<<dim3(static_cast<unsigned>((n + 255) / 256)), 256, 0, st>>>(
          static_cast<const uint32_t*>(workspace), n, calib_factor, out0, out1);
    else
      cols_finish_cal_kernel<D, QWIX_ABSMAX><<<dim3(static_cast<unsigned>((n + 255) / 256)), 256, 0, st>>>(
          static_cast<const uint32_t*>(workspace), n, calib_factor, out0, out1);
  })
  return check_launch("finish calibration");
}

int qwix_hip_compute_scale_zero_point(const void* cal0, const void* cal1, int dtype, int64_t n, int qtype,
                                      int calibration, void* scale, void* zero_point, void* stream) {
  if (n <= 0 || !cal0 || !scale || (calibration == QWIX_MINMAX && (!cal1 || !zero_point)))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "bad arguments to compute_scale_zero_point");
  hipStream_t st = static_cast<hipStream_t>(stream);
  QWIX_DISPATCH_D(dtype, {
    QWIX_DISPATCH_QT_CAL(qtype, calibration, {
      scale_zp_kernel<D, QT, CAL><<<dim3(static_cast<unsigned>((n + 255) / 256)), 256, 0, st>>>(
          cal0, cal1, n, scale, static_cast<int8_t*>(zero_point));
    })
  })
  return check_launch("compute_scale_zero_point");
}

int qwix_hip_quantize_with_scale(const void* x, int dtype, int64_t outer, int64_t reduce, int64_t inner,
                                 int64_t tile, int qtype, const void* scale, const void* zero_point, int q_layout,
                                 void* qvalue, void* stream) {
  if (int e = check_geom(outer, reduce, inner, tile)) return e;
  if (!x || !qvalue || !scale) return fail(QWIX_ERR_INVALID_ARGUMENT, "null x/qvalue/scale");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int cal = zero_point ? QWIX_MINMAX : QWIX_ABSMAX;
  if (inner == 1)
    return run_rows<MODE_GIVEN>(x, dtype, outer * (reduce / tile), tile, qtype, cal, 0.f, qvalue,
                                const_cast<void*>(scale), const_cast<void*>(zero_point), nullptr, nullptr, nullptr, 0,
                                st);
  if (int e = check_cols(x, dtype, reduce, inner, tile, q_layout, qvalue)) return e;
  const ColGeom g = make_col_geom(outer, reduce, inner, tile, dtype == QWIX_BF16 ? 8 : 4);
  return run_cols_quantize<1>(x, dtype, g, qtype, cal, q_layout, nullptr, 0.f, qvalue, const_cast<void*>(scale),
                              const_cast<void*>(zero_point), st);
}

int qwix_hip_quantize_with_scale_noise(const void* x, int dtype, int64_t outer, int64_t reduce, int64_t inner,
                                       int64_t tile, int qtype, const void* scale, const void* zero_point,
                                       const float* noise, void* qvalue, void* stream) {
  if (int e = check_geom(outer, reduce, inner, tile)) return e;
  if (!x || !qvalue || !scale || !noise) return fail(QWIX_ERR_INVALID_ARGUMENT, "null x/qvalue/scale/noise");
  if (qtype != QWIX_INT8 && qtype != QWIX_INT4)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "noise is added before the rounding to an integer type only (qtype %d)", qtype);
  const int64_t n = outer * reduce * inner;
  if (n & 1) return fail(QWIX_ERR_UNSUPPORTED, "an even element count is needed");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t pairs = n / 2;
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((pairs + 255) / 256, 65536));
  uint8_t* qb = static_cast<uint8_t*>(qvalue);
  const int8_t* zb = static_cast<const int8_t*>(zero_point);
#define QWIX_NOISE(DT, QT)                                                                                          \
  do {                                                                                                              \
    if (zb) noise_quantize_kernel<DT, QT, true><<<blocks, 256, 0, st>>>(x, pairs, reduce, inner, tile, scale, zb, noise, qb); \
    else noise_quantize_kernel<DT, QT, false><<<blocks, 256, 0, st>>>(x, pairs, reduce, inner, tile, scale, zb, noise, qb);  \
  } while (0)
  if (dtype == QWIX_BF16) {
    if (qtype == QWIX_INT8) QWIX_NOISE(BF16, QWIX_INT8); else QWIX_NOISE(BF16, QWIX_INT4);
  } else if (dtype == QWIX_F32) {
    if (qtype == QWIX_INT8) QWIX_NOISE(F32, QWIX_INT8); else QWIX_NOISE(F32, QWIX_INT4);
  } else {
    return fail(QWIX_ERR_INVALID_ARGUMENT, "dtype %d is not f32/bf16", dtype);
  }
#undef QWIX_NOISE
  return check_launch("quantize_with_scale_noise");
}

int qwix_hip_quantize_generic(const void* x, int dtype, const int64_t dims[5], int64_t t1, int64_t t3, int qtype,
                              int calibration, float calib_factor, void* qvalue, void* scale, void* zero_point,
                              void* stream) {
  if (!x || !qvalue || !scale || !dims) return fail(QWIX_ERR_INVALID_ARGUMENT, "null argument");
  Geom5 g;
  int64_t n = 1;
  for (int i = 0; i < 5; ++i) {
    if (dims[i] <= 0) return fail(QWIX_ERR_INVALID_ARGUMENT, "dims[%d] = %lld", i, (long long)dims[i]);
    g.d[i] = dims[i];
    n *= dims[i];
  }
  if (t1 <= 0 || t3 <= 0 || dims[1] % t1 || dims[3] % t3)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "tiles (%lld, %lld) do not divide (%lld, %lld)", (long long)t1,
                (long long)t3, (long long)dims[1], (long long)dims[3]);
  if (qtype == QWIX_INT4 && (n & 1)) return fail(QWIX_ERR_UNSUPPORTED, "int4 needs an even element count");
  if (calibration == QWIX_MINMAX && !zero_point) return fail(QWIX_ERR_INVALID_ARGUMENT, "minmax needs zero_point");
  g.t1 = t1;
  g.t3 = t3;
  const int64_t ns = dims[0] * (dims[1] / t1) * dims[2] * (dims[3] / t3) * dims[4];
  const int64_t nb = qtype == QWIX_INT4 ? n / 2 : n;
  hipStream_t st = static_cast<hipStream_t>(stream);
  {  // blocks of 16-byte row pieces that fit one workgroup's registers: the single-pass kernel
    const int ev = dtype == QWIX_BF16 ? 8 : 4;
    const int64_t nvec = t3 % ev == 0 ? t1 * (t3 / ev) : 0;
    if (dims[4] == 1 && nvec >= 2 && nvec <= 256 * 16 && aligned16(x) && (reinterpret_cast<uintptr_t>(qvalue) & 7) == 0 &&
        ns <= 0xFFFFFFFFll && (dtype == QWIX_F32 || dtype == QWIX_BF16)) {
      BlockGeom bg;
      bg.nblk = ns;
      bg.row_stride = dims[2] * dims[3];
      bg.r1 = dims[1];
      bg.r3 = dims[3];
      bg.n1 = static_cast<uint32_t>(dims[1] / t1);
      bg.d2 = static_cast<uint32_t>(dims[2]);
      bg.n3 = static_cast<uint32_t>(dims[3] / t3);
      bg.t1 = static_cast<uint32_t>(t1);
      bg.t3 = static_cast<uint32_t>(t3);
      bg.vpr = static_cast<uint32_t>(t3 / ev);
      bg.vpr_magic = bg.vpr == 1 ? 0u : static_cast<uint32_t>(((uint64_t{1} << 32) + bg.vpr - 1) / bg.vpr);
      bg.nvec = static_cast<int>(nvec);
      int lg = log2_ceil((nvec + 3) / 4);  // aim at 4 loads per thread, as many as 16 for the largest blocks
      if (lg > 8) lg = 8;
      bg.log2g = lg;
      const int loads = static_cast<int>((nvec + (1 << lg) - 1) >> lg);
      const dim3 grid(static_cast<unsigned>((ns + (256 >> lg) - 1) / (256 >> lg)));
      const uint8_t* xb = static_cast<const uint8_t*>(x);
      uint8_t* qb = static_cast<uint8_t*>(qvalue);
      int8_t* zb = static_cast<int8_t*>(zero_point);
      QWIX_DISPATCH_D(dtype, {
        QWIX_DISPATCH_QT_CAL(qtype, calibration, {
          if (loads <= 4)
            blocks_kernel<D, QT, CAL, 4><<<grid, 256, 0, st>>>(xb, bg, calib_factor, qb, scale, zb);
          else if (loads <= 8)
            blocks_kernel<D, QT, CAL, 8><<<grid, 256, 0, st>>>(xb, bg, calib_factor, qb, scale, zb);
          else
            blocks_kernel<D, QT, CAL, 16><<<grid, 256, 0, st>>>(xb, bg, calib_factor, qb, scale, zb);
        })
      })
      return check_launch("block quantize");
    }
  }
  QWIX_DISPATCH_D(dtype, {
    QWIX_DISPATCH_QT_CAL(qtype, calibration, {
      generic_scale_kernel<D, QT, CAL><<<dim3(static_cast<unsigned>((ns + 255) / 256)), 256, 0, st>>>(
          x, g, calib_factor, scale, static_cast<int8_t*>(zero_point));
      generic_quant_kernel<D, QT, CAL><<<dim3(static_cast<unsigned>((nb + 255) / 256)), 256, 0, st>>>(
          x, g, scale, static_cast<const int8_t*>(zero_point), static_cast<uint8_t*>(qvalue));
    })
  })
  return check_launch("generic quantize");
}

int qwix_hip_calibrate_rms(const void* x, int dtype, const int64_t dims[5], int64_t t1, int64_t t3, float factor,
                           void* out, void* stream) {
  if (!x || !out || !dims) return fail(QWIX_ERR_INVALID_ARGUMENT, "null argument");
  if (!(factor > 0.f)) return fail(QWIX_ERR_INVALID_ARGUMENT, "rms calibration needs a positive scale factor");
  Geom5 g;
  for (int i = 0; i < 5; ++i) {
    if (dims[i] <= 0) return fail(QWIX_ERR_INVALID_ARGUMENT, "dims[%d] = %lld", i, (long long)dims[i]);
    g.d[i] = dims[i];
  }
  if (t1 <= 0 || t3 <= 0 || dims[1] % t1 || dims[3] % t3)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "tiles (%lld, %lld) do not divide (%lld, %lld)", (long long)t1,
                (long long)t3, (long long)dims[1], (long long)dims[3]);
  g.t1 = t1;
  g.t3 = t3;
  const int64_t ns = dims[0] * (dims[1] / t1) * dims[2] * (dims[3] / t3) * dims[4];
  if ((ns + 3) / 4 > INT32_MAX) return fail(QWIX_ERR_UNSUPPORTED, "too many scale groups");
  hipStream_t st = static_cast<hipStream_t>(stream);
  QWIX_DISPATCH_D(dtype, {
    rms_kernel<D><<<dim3(static_cast<unsigned>((ns + 3) / 4)), 256, 0, st>>>(x, g, factor, out);
  })
  return check_launch("rms calibration");
}

int qwix_hip_dequantize_generic(const void* qvalue, int qtype, const int64_t dims[5], int64_t t1, int64_t t3,
                                const void* scale, const void* zero_point, int dtype, void* out, void* stream) {
  if (!qvalue || !scale || !out || !dims) return fail(QWIX_ERR_INVALID_ARGUMENT, "null argument");
  Geom5 g;
  int64_t n = 1;
  for (int i = 0; i < 5; ++i) {
    if (dims[i] <= 0) return fail(QWIX_ERR_INVALID_ARGUMENT, "dims[%d] = %lld", i, (long long)dims[i]);
    g.d[i] = dims[i];
    n *= dims[i];
  }
  if (t1 <= 0 || t3 <= 0 || dims[1] % t1 || dims[3] % t3)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "tiles (%lld, %lld) do not divide (%lld, %lld)", (long long)t1,
                (long long)t3, (long long)dims[1], (long long)dims[3]);
  if (qtype == QWIX_INT4 && (n & 1)) return fail(QWIX_ERR_UNSUPPORTED, "int4 needs an even element count");
  g.t1 = t1;
  g.t3 = t3;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* q = static_cast<const uint8_t*>(qvalue);
  const int8_t* zp = static_cast<const int8_t*>(zero_point);
  const bool vec = dims[4] == 1 && t3 % 8 == 0 && (reinterpret_cast<uintptr_t>(qvalue) & 7) == 0 && aligned16(out);
  const int64_t threads = vec ? n / 8 : n;
  const dim3 grid(static_cast<unsigned>((threads + 255) / 256));
  if (threads + 255 >= (int64_t{256} << 31)) return fail(QWIX_ERR_UNSUPPORTED, "array too large");
#define QWIX_DEQ_GEN(QTT)                                                                            \
  if (vec) generic_dequant_kernel<D, QTT, 8><<<grid, 256, 0, st>>>(q, g, scale, zp, out);          \
  else generic_dequant_kernel<D, QTT, 1><<<grid, 256, 0, st>>>(q, g, scale, zp, out)
  QWIX_DISPATCH_D(dtype, {
    if (qtype == QWIX_INT8) { QWIX_DEQ_GEN(QWIX_INT8); }
    else if (qtype == QWIX_INT4) { QWIX_DEQ_GEN(QWIX_INT4); }
    else if (qtype == QWIX_E4M3) { QWIX_DEQ_GEN(QWIX_E4M3); }
    else return fail(QWIX_ERR_INVALID_ARGUMENT, "unknown qtype %d", qtype);
  })
#undef QWIX_DEQ_GEN
  return check_launch("generic dequantize");
}

int qwix_hip_dequantize(const void* qvalue, int qtype, int q_layout, int64_t outer, int64_t reduce, int64_t inner,
                        int64_t tile, const void* scale, const void* zero_point, int dtype, void* out,
                        void* stream) {
  if (int e = check_geom(outer, reduce, inner, tile)) return e;
  if (!qvalue || !scale || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null argument");
  if (q_layout != QWIX_LAYOUT_NATURAL && q_layout != QWIX_LAYOUT_REDUCE_MINOR)
    return fail(QWIX_ERR_INVALID_ARGUMENT, "unknown layout %d", q_layout);
  const int64_t n = outer * reduce * inner;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* q = static_cast<const uint8_t*>(qvalue);
  const int8_t* zp = static_cast<const int8_t*>(zero_point);
  const bool ptr_ok = aligned16(qvalue) && aligned16(out);
  // fast paths; the one-thread-per-element kernel below takes every other shape
  const bool natural = q_layout == QWIX_LAYOUT_NATURAL || inner == 1;
  if (natural && ptr_ok && n % 8 == 0 && (inner == 1 ? tile % 8 == 0 : inner % 8 == 0)) {
    const unsigned vb = static_cast<unsigned>((n / 8 + 255) / 256);
#define QWIX_DEQ_VEC(QTT) dequant_vec_kernel<D, QTT><<<vb, 256, 0, st>>>(q, outer, reduce, inner, tile, scale, zp, out)
    QWIX_DISPATCH_D(dtype, {
      if (qtype == QWIX_INT8) QWIX_DEQ_VEC(QWIX_INT8);
      else if (qtype == QWIX_INT4) QWIX_DEQ_VEC(QWIX_INT4);
      else if (qtype == QWIX_E4M3) QWIX_DEQ_VEC(QWIX_E4M3);
      else return fail(QWIX_ERR_INVALID_ARGUMENT, "unknown qtype %d", qtype);
    })
#undef QWIX_DEQ_VEC
    return check_launch("dequantize");
  }
  if (!natural && ptr_ok && inner % 16 == 0 && reduce % (qtype == QWIX_INT4 ? 32 : 16) == 0 && outer <= 65535 &&
      (inner + 63) / 64 <= 65535) {
    const dim3 grid(static_cast<unsigned>((reduce + 63) / 64), static_cast<unsigned>((inner + 63) / 64),
                    static_cast<unsigned>(outer));
#define QWIX_DEQ_RM(QTT) dequant_rm_kernel<D, QTT><<<grid, 256, 0, st>>>(q, reduce, inner, tile, scale, zp, out)
    QWIX_DISPATCH_D(dtype, {
      if (qtype == QWIX_INT8) QWIX_DEQ_RM(QWIX_INT8);
      else if (qtype == QWIX_INT4) QWIX_DEQ_RM(QWIX_INT4);
      else if (qtype == QWIX_E4M3) QWIX_DEQ_RM(QWIX_E4M3);
      else return fail(QWIX_ERR_INVALID_ARGUMENT, "unknown qtype %d", qtype);
    })
#undef QWIX_DEQ_RM
    return check_launch("dequantize");
  }
  QWIX_DISPATCH_D(dtype, {
    if (qtype == QWIX_INT8)
      dequant_kernel<D, QWIX_INT8><<<blocks, 256, 0, st>>>(q, q_layout, outer, reduce, inner, tile, scale, zp, out);
    else if (qtype == QWIX_INT4)
      dequant_kernel<D, QWIX_INT4><<<blocks, 256, 0, st>>>(q, q_layout, outer, reduce, inner, tile, scale, zp, out);
    else if (qtype == QWIX_E4M3)
      dequant_kernel<D, QWIX_E4M3><<<blocks, 256, 0, st>>>(q, q_layout, outer, reduce, inner, tile, scale, zp, out);
    else
      return fail(QWIX_ERR_INVALID_ARGUMENT, "unknown qtype %d", qtype);
  })
  return check_launch("dequantize");
}

int qwix_hip_dequantize_rm(const void* qvalue, int qtype, int64_t outer, int64_t reduce, int64_t inner, int64_t tile,
                           const void* scale, const void* zero_point, int dtype, void* out, int out_dtype,
                           void* stream) {
  if (out_dtype != dtype && !(dtype == QWIX_F32 && out_dtype == QWIX_BF16))
    return fail(QWIX_ERR_INVALID_ARGUMENT, "out_dtype must be the scale dtype, or bf16 for f32 scales");
  if (int e = check_geom(outer, reduce, inner, tile)) return e;
  if (!qvalue || !scale || !out) return fail(QWIX_ERR_INVALID_ARGUMENT, "null argument");
  if (reduce % 8 || tile % 8 || !aligned16(qvalue) || !aligned16(out))
    return fail(QWIX_ERR_UNSUPPORTED, "reduce-minor dequantize needs reduce and tile multiples of 8 and 16-byte aligned "
                "arrays (reduce=%lld tile=%lld)", (long long)reduce, (long long)tile);
  const int64_t n = outer * reduce * inner;
  const unsigned vb = static_cast<unsigned>((n / 8 + 255) / 256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* q = static_cast<const uint8_t*>(qvalue);
  const int8_t* zp = static_cast<const int8_t*>(zero_point);
#define QWIX_DEQ_KEEP(QTT)                                                                                       \
  do {                                                                                                           \
    if (out_dtype == dtype)                                                                                      \
      dequant_keep_rm_kernel<D, QTT, D><<<vb, 256, 0, st>>>(q, outer, reduce, inner, tile, scale, zp, out);      \
    else                                                                                                         \
      dequant_keep_rm_kernel<D, QTT, BF16><<<vb, 256, 0, st>>>(q, outer, reduce, inner, tile, scale, zp, out);   \
  } while (0)
  QWIX_DISPATCH_D(dtype, {
    if (qtype == QWIX_INT8) QWIX_DEQ_KEEP(QWIX_INT8);
    else if (qtype == QWIX_INT4) QWIX_DEQ_KEEP(QWIX_INT4);
    else if (qtype == QWIX_E4M3) QWIX_DEQ_KEEP(QWIX_E4M3);
    else return fail(QWIX_ERR_INVALID_ARGUMENT, "unknown qtype %d", qtype);
  })
#undef QWIX_DEQ_KEEP
  return check_launch("dequantize (reduce-minor)");
}

int qwix_hip_transpose_q(const void* src, int qtype, int64_t rows, int64_t cols, void* dst, void* stream) {
  if (!src || !dst || rows <= 0 || cols <= 0) return fail(QWIX_ERR_INVALID_ARGUMENT, "bad transpose arguments");
  if (qtype == QWIX_INT4 && ((rows & 1) || (cols & 1)))
    return fail(QWIX_ERR_UNSUPPORTED, "int4 transpose needs even rows and cols");
  const dim3 grid(static_cast<unsigned>((cols + 63) / 64), static_cast<unsigned>((rows + 63) / 64));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (qtype == QWIX_INT4)
    transpose_q_kernel<QWIX_INT4><<<grid, 256, 0, st>>>(static_cast<const uint8_t*>(src), rows, cols,
                                                        static_cast<uint8_t*>(dst));
  else
    transpose_q_kernel<QWIX_INT8><<<grid, 256, 0, st>>>(static_cast<const uint8_t*>(src), rows, cols,
                                                        static_cast<uint8_t*>(dst));
  return check_launch("transpose");
}

}  // extern "C"
