/*
 * qwix_hip.h -- C ABI of libqwix_hip.so: the MI355X (gfx950) kernels behind Qwix's
 * quantize + quantized dot_general path.
 *
 * Every entry point
 *   - takes raw DEVICE pointers, sizes and a hipStream_t (passed as void*),
 *   - only enqueues work on that stream (no hipMalloc/hipFree, no device sync),
 *   - returns QWIX_OK or an error code; qwix_hip_last_error() gives the text of
 *     the calling thread's last error,
 *   - is re-entrant; the only state the library keeps is, per kernel and device, the dynamic-LDS limit it has
 *     already raised (an atomic), and the per-device address of the scratch array of qwix_hip_quantize_static.
 * These are exactly the symbols a jax.ffi custom-call handler (or ctypes, or a
 * torch extension) binds; the reference functions they replace are cited per
 * entry (paths relative to the google/qwix tree).
 *
 * Conventions
 *   dtype   QWIX_F32 / QWIX_BF16                         (float arrays)
 *   qtype   QWIX_INT8 / QWIX_INT4 / QWIX_E4M3            (quantized values)
 *   int4    two values per byte along the physically contiguous axis; the element
 *           with the even index sits in the LOW nibble; two's complement.
 *   A float array of rank n that is quantized with one reduced (or tiled) axis is
 *   described as the row-major 3-D view (outer, reduce, inner); `tile` divides
 *   `reduce`; the scale is the row-major array (outer, reduce/tile, inner).
 *   Per-token activations:   outer=tokens, reduce=features, inner=1, tile=reduce.
 *   Per-channel (K,N) weight: outer=1, reduce=K, inner=N, tile=K.
 *   Sub-channel (K,N) weight: outer=1, reduce=K, inner=N, tile=128.
 */
#ifndef QWIX_HIP_H_
#define QWIX_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QWIX_API __attribute__((visibility("default")))

enum { QWIX_OK = 0, QWIX_ERR_INVALID_ARGUMENT = 1, QWIX_ERR_UNSUPPORTED = 2, QWIX_ERR_LAUNCH = 3 };
enum { QWIX_F32 = 0, QWIX_BF16 = 1, QWIX_I32 = 2 };
enum { QWIX_INT8 = 0, QWIX_INT4 = 1, QWIX_E4M3 = 2 };
enum { QWIX_ABSMAX = 0, QWIX_MINMAX = 1 };
/* Quantized-value layouts for the 3-D view (outer, reduce, inner). */
enum {
  QWIX_LAYOUT_NATURAL = 0,      /* (outer, reduce, inner) row-major, like the input        */
  QWIX_LAYOUT_REDUCE_MINOR = 1  /* (outer, inner, reduce) row-major: the reduced axis is    */
                                /* contiguous, which is what the GEMM kernels consume       */
};

/* Version / diagnostics. */
QWIX_API int qwix_hip_abi_version(void);
QWIX_API const char* qwix_hip_last_error(void);

/* ---------------------------------------------------------------------------------------
 * Quantize: calibrate -> scale(/zero point) -> divide -> round -> saturating cast, fused.
 * Replaces qarray.quantize (qwix/_src/core/qarray.py:638-644) = calibrate (:470-534) +
 * compute_scale_zero_point (:537-584) + quantize_with_scale_zero_point (:594-635) +
 * numerics.convert_to (qwix/_src/core/numerics.py:139-196).
 *   x           (outer, reduce, inner) of `dtype`
 *   calibration QWIX_ABSMAX or QWIX_MINMAX; calib_factor > 0 multiplies the range
 *               ("absmax,0.9"); pass 0 for none
 *   qvalue      out; int8/e4m3: 1 byte per element, int4: packed (see above)
 *   scale       out, `dtype`, (outer, reduce/tile, inner)
 *   zero_point  out for QWIX_MINMAX (int8 per scale element, also for int4), else NULL
 *   workspace   device scratch of qwix_hip_quantize_workspace_bytes(...) bytes (may be
 *               NULL when that is 0)
 */
QWIX_API size_t qwix_hip_quantize_workspace_bytes(int64_t outer, int64_t reduce, int64_t inner,
                                         int64_t tile, int calibration);
QWIX_API int qwix_hip_quantize(const void* x, int dtype, int64_t outer, int64_t reduce, int64_t inner,
                      int64_t tile, int qtype, int calibration, float calib_factor,
                      int q_layout, void* qvalue, void* scale, void* zero_point,
                      void* workspace, size_t workspace_bytes, void* stream);

/* qwix_hip_quantize for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments and results as qwix_hip_quantize without the workspace: the calibration scratch
 * (partial absmax / min / max values of scale groups that span several workgroups) lives in a
 * file-scope device array of qwix_hip_quantize_static_max_bytes() = 1 MiB that every GPU the library
 * runs on holds until the process ends.  Shapes whose qwix_hip_quantize_workspace_bytes(...) exceeds
 * that are refused with QWIX_ERR_UNSUPPORTED.  The call allocates nothing and frees nothing.  All calls
 * on one GPU share that GPU's array: calls that overlap on one GPU (different streams, or threads)
 * race; calls ordered on one stream do not (every call clears what it accumulates into).  The array used
 * is the one of the CURRENT device of the calling thread: the caller must have made the stream's device
 * current (hipSetDevice) before the call, as for any launch on that stream. */
QWIX_API size_t qwix_hip_quantize_static_max_bytes(void);
QWIX_API int qwix_hip_quantize_static(const void* x, int dtype, int64_t outer, int64_t reduce, int64_t inner,
                             int64_t tile, int qtype, int calibration, float calib_factor,
                             int q_layout, void* qvalue, void* scale, void* zero_point, void* stream);

/* calibrate alone (qarray.py:470-534): writes absmax (QWIX_ABSMAX: out0) or min/max
 * (QWIX_MINMAX: out0=min, out1=max), each `dtype`, shaped like the scale. */
QWIX_API int qwix_hip_calibrate(const void* x, int dtype, int64_t outer, int64_t reduce, int64_t inner,
                       int64_t tile, int calibration, float calib_factor, void* out0,
                       void* out1, void* workspace, size_t workspace_bytes, void* stream);

/* calibrate with the 'rms,s' method (qwix/_src/core/qarray.py:511-515): out[group] =
 * D(D(sqrt(D(mean(D(x^2))))) * D(s)) for every scale group of the 5-D geometry of
 * qwix_hip_quantize_generic (a single reduced group: dims = (outer, reduce, inner, 1, 1), t3 = 1).
 * The result is an 'absmax' calibration: qwix_hip_compute_scale_zero_point turns it into a scale.
 * The mean is summed in f32; the order of that sum is the one rounding XLA does not pin. */
QWIX_API int qwix_hip_calibrate_rms(const void* x, int dtype, const int64_t dims[5], int64_t t1, int64_t t3,
                           float factor, void* out, void* stream);

/* compute_scale_zero_point (qarray.py:537-584) on n calibration values. */
QWIX_API int qwix_hip_compute_scale_zero_point(const void* cal0, const void* cal1, int dtype, int64_t n,
                                      int qtype, int calibration, void* scale, void* zero_point,
                                      void* stream);

/* quantize_with_scale_zero_point (qarray.py:594-635) with a given scale (static range). */
QWIX_API int qwix_hip_quantize_with_scale(const void* x, int dtype, int64_t outer, int64_t reduce,
                                 int64_t inner, int64_t tile, int qtype, const void* scale,
                                 const void* zero_point, int q_layout, void* qvalue,
                                 void* stream);

/* The same with stochastic rounding (numerics.convert_to with a noise_fn, numerics.py:191-195; reached through
 * quantize_with_scale_zero_point(..., noise_fn), qarray.py:594-635): int8 / int4 only; the quotient (plus zero point)
 * is formed in the array dtype, widened to f32, noise[i] (f32, shaped and ordered like x) is added, and the sum is
 * rounded half to even and saturated.  Natural layout (int4: pairs along the contiguous axis). */
QWIX_API int qwix_hip_quantize_with_scale_noise(const void* x, int dtype, int64_t outer, int64_t reduce, int64_t inner,
                                       int64_t tile, int qtype, const void* scale, const void* zero_point,
                                       const float* noise, void* qvalue, void* stream);

/* Generic fallback for shapes the 3-D view cannot express (two tiled/reduced axes):
 * x is the row-major 5-D view (d0, r1, d2, r3, d4); tiles t1 | r1 and t3 | r3 are reduced;
 * scale is (d0, r1/t1, d2, r3/t3, d4).  Natural layout only.  Slow but complete. */
QWIX_API int qwix_hip_quantize_generic(const void* x, int dtype, const int64_t dims[5], int64_t t1,
                              int64_t t3, int qtype, int calibration, float calib_factor,
                              void* qvalue, void* scale, void* zero_point, void* stream);

/* dequantize (qarray.py:692-708): (q - zp) * scale in the scale dtype. */
QWIX_API int qwix_hip_dequantize(const void* qvalue, int qtype, int q_layout, int64_t outer,
                        int64_t reduce, int64_t inner, int64_t tile, const void* scale,
                        const void* zero_point, int dtype, void* out, void* stream);

/* dequantize for the 5-D geometry of qwix_hip_quantize_generic (two reduced axis groups, e.g. one
 * scale per t1 x t3 block; two_dim_scales_test.py:29-56 dequantizes such an array):
 * out[i] = D(D(q[i] - zp) * scale) with the scale / zero point of element i's block.  qvalue in the
 * natural layout, scale (and zero_point, may be NULL) as qwix_hip_quantize_generic writes them. */
QWIX_API int qwix_hip_dequantize_generic(const void* qvalue, int qtype, const int64_t dims[5], int64_t t1,
                                int64_t t3, const void* scale, const void* zero_point, int dtype,
                                void* out, void* stream);

/* Layout helper: (rows, cols) bytes -> (cols, rows) bytes; int4: repacks so the pairs run
 * along the new contiguous axis.  Used to bring a NATURAL qvalue to REDUCE_MINOR. */
QWIX_API int qwix_hip_transpose_q(const void* src, int qtype, int64_t rows, int64_t cols, void* dst,
                         void* stream);

/* ---------------------------------------------------------------------------------------
 * Quantized GEMM, dequantize-on-output.  Replaces _fast_dot_general
 * (qwix/_src/core/dot_general.py:135-261) for a 2-D contraction:
 *     out[m,n] = cast_R( (T(sum_k a[m,k] b[k,n]) * sa[m]) * sb[n] )
 *   a        (M,K) row-major, lda bytes-per-row >= K (K-contiguous)
 *   b        stored K-contiguous: b_nk[n*ldb + k]   (QWIX_LAYOUT_REDUCE_MINOR of a (K,N) weight)
 *   qtype    QWIX_INT8 (int32 accumulate, exact) or QWIX_E4M3 (f32 accumulate)
 *   sa, sb   per-row / per-column scales (sa_dtype / sb_dtype in {F32,BF16}); NULL = none
 *   out      (M,N) row-major of out_dtype in {F32,BF16}; QWIX_I32 returns the raw int32
 *            accumulators (int8 only; scales ignored)
 * Intermediate dtypes follow the reference: int32 -> f32 -> scale dtype, one rounding per
 * multiply, lhs scale first; e4m3: the f32 accumulator is rounded to acc_dtype first
 * (the reference's accumulator type = result type for non-integer operands).
 */
QWIX_API int qwix_hip_qgemm(const void* a, int64_t lda, const void* b, int64_t ldb, int qtype, int64_t M,
                   int64_t N, int64_t K, const void* sa, int sa_dtype, const void* sb,
                   int sb_dtype, int acc_dtype, void* out, int out_dtype, int64_t ldo,
                   void* stream);

/* qwix_hip_qgemm with scratch memory.  A few hundred rows against a narrow weight with a long K leave most
 * of the chip idle under 128 x 128 tiles; given a workspace the library may cut K into ranges that run as
 * separate workgroups and add the partial tiles up in a second kernel (int32 partials: bit-identical to
 * qwix_hip_qgemm for int8; e4m3 sums its f32 partials in range order).  qwix_hip_qgemm_workspace_bytes
 * returns how many bytes that takes for a shape, 0 where splitting never pays; a NULL or smaller workspace
 * makes the call behave exactly like qwix_hip_qgemm.  The workspace is 16-byte aligned device memory that
 * only this call uses until it has finished on `stream`.  Same reference function as qwix_hip_qgemm
 * (_fast_dot_general, qwix/_src/core/dot_general.py:135-261). */
QWIX_API size_t qwix_hip_qgemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
QWIX_API int qwix_hip_qgemm_ws(const void* a, int64_t lda, const void* b, int64_t ldb, int qtype, int64_t M,
                      int64_t N, int64_t K, const void* sa, int sa_dtype, const void* sb, int sb_dtype,
                      int acc_dtype, void* out, int out_dtype, int64_t ldo, void* workspace,
                      size_t workspace_bytes, void* stream);

/* Asymmetric (zero-point) operand on the quantized path.  Replaces the correction terms of
 * _fast_dot_general (qwix/_src/core/dot_general.py:228-253): the reference subtracts
 * dot(broadcast(zp_lhs), q_rhs) or dot(q_lhs, broadcast(zp_rhs)) from the int32 accumulator
 * before scaling.  With one zero point per row (lhs) or per column (rhs) that term is the outer
 * product zu[m] * zv[n]:
 *     lhs asymmetric:  zu = zero points of the rows of a,  zv[n] = sum_k b[n,k]
 *     rhs asymmetric:  zu[m] = sum_k a[m,k],               zv = zero points of the columns of b
 *     out[m,n] = cast_R( (T(sum_k a[m,k] b[n,k] - zu[m] * zv[n]) * sa[m]) * sb[n] )
 * int8 operands, int32 arithmetic (exact), otherwise as qwix_hip_qgemm. */
QWIX_API int qwix_hip_qgemm_zp(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N,
                      int64_t K, const void* sa, int sa_dtype, const void* sb, int sb_dtype,
                      const int32_t* zu, const int32_t* zv, void* out, int out_dtype, int64_t ldo,
                      void* stream);

/* Ragged quantized GEMM (mixture-of-experts).  Replaces _fast_ragged_dot_general
 * (qwix/_src/core/ragged_dot.py:123-226) for the dimension numbers of qwix.ragged_dot
 * (ragged_dot.py:24-29: lhs (M,K), rhs (G,K,N), lhs rows split into G consecutive groups):
 *     out[m,n] = cast_R( (T(sum_k a[m,k] * b_g[n,k]) * sa[m]) * sb_g[n] ),   g = group of row m,
 * with the same accumulator / rounding chain as qwix_hip_qgemm.  group_sizes (device memory, G
 * int32 values) is read by the kernel, never by the host: negative sizes count as 0, groups are
 * cut off at row M, and rows past the last group are written as zeros (what the masked sum of
 * lax.ragged_dot_general gives them).  b is G panels of (N,K) K-contiguous values,
 * b_group_stride bytes apart; sb holds one vector of N scales per group, sb_group_stride
 * elements apart (the expanded per-group scale of ragged_dot.py:32-57,205-217), or a single shared
 * vector when sb_group_stride is 0.  sa / sb may be null. */
QWIX_API int qwix_hip_qgemm_ragged(const void* a, int64_t lda, const void* b, int64_t ldb,
                          int64_t b_group_stride, int qtype, int64_t M, int64_t N, int64_t K,
                          const int32_t* group_sizes, int64_t G, const void* sa, int sa_dtype,
                          const void* sb, int sb_dtype, int64_t sb_group_stride, int acc_dtype,
                          void* out, int out_dtype, int64_t ldo, void* stream);

/* Batched quantized GEMM: `batch` independent problems of one shape in a single launch.  Replaces
 * the batch dimensions of _fast_dot_general (qwix/_src/core/dot_general.py:135-261: lhs_ba / rhs_ba
 * of dimension_numbers; the scale transposes of :79-90 put the batch axes first), e.g. the
 * 'bqd,bkd->bqk' contractions of attention.  Problem z uses a + z*a_batch_stride and
 * b + z*b_batch_stride (bytes), scale vectors sa + z*sa_batch_stride and sb + z*sb_batch_stride
 * (elements; 0 = one vector shared by all problems) and writes out + z*out_batch_stride (elements).
 * Everything else as qwix_hip_qgemm. */
QWIX_API int qwix_hip_qgemm_batched(const void* a, int64_t lda, int64_t a_batch_stride, const void* b,
                           int64_t ldb, int64_t b_batch_stride, int qtype, int64_t batch, int64_t M,
                           int64_t N, int64_t K, const void* sa, int sa_dtype, int64_t sa_batch_stride,
                           const void* sb, int sb_dtype, int64_t sb_batch_stride, int acc_dtype,
                           void* out, int out_dtype, int64_t ldo, int64_t out_batch_stride,
                           void* stream);

/* Decode-size w8a8 with the activation quantization folded into the GEMM: per-token absmax int8
 * quantization of x (quantize, qwix/_src/core/qarray.py:638-644, as PtqProvider applies it to the
 * lhs of dot_general, providers/boxed_param.py:416-455) followed by _fast_dot_general
 * (dot_general.py:135-261) in one launch; the counterpart, for M <= 32, of the Pallas kernel
 * qwix/contrib/kernels/lhs_fused_quantized_matmul.py.  Results are bit-identical to
 * qwix_hip_quantize + qwix_hip_qgemm:
 *     s[m] = D(max_k |x[m,k]| / 127.5) (1 if below 2^-63),  q = sat(rint(D(x / s))),
 *     out[m,n] = cast_R( (T(sum_k q[m,k] b[n,k]) * s[m]) * sb[n] ),   D = dtype of x.
 * x: (M, K) of x_dtype (QWIX_BF16 / QWIX_F32), row pitch ldx elements; b: (N, K) int8; M <= 32,
 * K % 128 == 0, K <= 2048: every workgroup re-derives the quantized rows it needs, which beats a
 * separate quantize launch only while K is short. */
QWIX_API int qwix_hip_qgemm_fused_act(const void* x, int x_dtype, int64_t ldx, const void* b, int64_t ldb,
                             int64_t M, int64_t N, int64_t K, const void* sb, int sb_dtype, void* out,
                             int out_dtype, int64_t ldo, void* stream);

/* Dynamic-range w8a8 in one call at any batch size: per-token absmax quantization of x to int8 or e4m3
 * (qarray.quantize, qwix/_src/core/qarray.py:638-644, as PtqProvider applies it to the lhs of dot_general,
 * providers/boxed_param.py:416-455) followed by _fast_dot_general (dot_general.py:135-261): the operation that
 * qwix/contrib/kernels/lhs_fused_quantized_matmul.py specifies, with the numerics of the two reference
 * functions (per-token scales over the whole of K, scale in the dtype of x).  Decode-size int8 calls run as
 * one launch (qwix_hip_qgemm_fused_act); every other shape runs the quantize kernel and then the GEMM on the
 * caller's scratch memory (qwix_hip_qgemm_dynamic_act_workspace_bytes(M, N, K, x_dtype) bytes, 16-byte aligned,
 * used only by this call until it has finished on `stream`), with dense rows (ldx == K).  Results are
 * bit-identical to qwix_hip_quantize + qwix_hip_qgemm.  At prefill sizes the two kernels stay separate on
 * purpose: with per-token scales every column tile of a row panel would redo the panel's quantization. */
QWIX_API size_t qwix_hip_qgemm_dynamic_act_workspace_bytes(int64_t M, int64_t N, int64_t K, int x_dtype);
QWIX_API int qwix_hip_qgemm_dynamic_act(const void* x, int x_dtype, int64_t ldx, const void* b, int64_t ldb, int qtype,
                               int64_t M, int64_t N, int64_t K, const void* sb, int sb_dtype, int acc_dtype,
                               void* out, int out_dtype, int64_t ldo, void* workspace,
                               size_t workspace_bytes, void* stream);

/* out[r] = sum_k q[r*ld + k] for int8 rows (K % 16 == 0): the K-sums qwix_hip_qgemm_zp needs
 * (the reference obtains them as a dot_general against the broadcast zero point,
 * dot_general.py:233-239,246-252). */
QWIX_API int qwix_hip_ksum_i8(const void* q, int64_t ld, int64_t rows, int64_t K, int32_t* out, void* stream);

/* Sub-channel GEMM (dot_general.py:186-203,255-260): K is split in groups of `group`
 * (multiple of 128); per-group int32 partials are scaled and summed:
 *     out[m,n] = cast_R( sum_g (T(acc_g[m,n]) * sa[m,g']) * sb[g,n] )
 *   a        int8 (M,K) K-contiguous
 *   b        int8 or int4 (b_qtype), K-contiguous rows: b_nk[n*ldb_bytes + ...]
 *   sa       (M, ga) with ga in {1, K/group}, row-major;  sb (K/group, N) row-major
 *   exact    1: every intermediate is rounded exactly as the reference does (bit-exact with
 *               the CPU oracle, slower); 0: f32 throughout (within rtol 1e-2)
 *   acc_out  optional (K/group, M, N) int32 raw partials for parity tests, else NULL
 * b_qtype QWIX_E4M3: a and b are both OCP e4m3 bytes; every group's dot is summed in f32 on the
 * matrix cores, delivered in out_dtype (float operands accumulate in the result type,
 * qarray.py:781-821), then scaled lhs first with one rounding per step and summed over the groups
 * in f32 (exact = 1: with the reference's roundings; 0: f32 throughout, one rounding of the sum;
 * acc_out must be NULL).
 */
QWIX_API int qwix_hip_qgemm_grouped(const void* a, int64_t lda, const void* b, int64_t ldb_bytes,
                           int b_qtype, int64_t M, int64_t N, int64_t K, int64_t group,
                           const void* sa, int sa_dtype, int64_t ga, const void* sb,
                           int sb_dtype, void* out, int out_dtype, int64_t ldo, int exact,
                           int32_t* acc_out, void* stream);

/* Hadamard rotation + activation quantize + sub-channel GEMM in one call: the functional content of
 * hadamard_quantize_multiply (qwix/contrib/kernels/fused_hadamard_quantized_matmul.py:349-414) with the numerics
 * of the unfused path (hadamard_rot.py:133-190, quantize, _fast_dot_general with tiled weights):
 *     xq, sa = quantize_int8( ((x * pre_sign) H_K) * post_sign * out_scale, tile = act_tile along K )
 *     out    = qwix_hip_qgemm_grouped(xq, b, sa, sb, exact = 0)
 * x (M, K) of x_dtype, dense rows; act_tile = K (one scale per token) or = group; b, sb, group, out as in
 * qwix_hip_qgemm_grouped.  workspace: qwix_hip_qgemm_hadamard_act_workspace_bytes(M, K, act_tile, x_dtype) bytes of
 * device memory, 16-byte aligned (the int8 rows and their scales; nothing is allocated).  Two kernels on the
 * stream; bit-identical to qwix_hip_fwht_quantize followed by qwix_hip_qgemm_grouped.  A workspace that is larger by
 * qwix_hip_qgemm_grouped_workspace_bytes(M, N, K, group, b_qtype) lets the GEMM cut K into ranges where that pays
 * (then: followed by qwix_hip_qgemm_grouped_ws on the surplus, three kernels). */
QWIX_API size_t qwix_hip_qgemm_hadamard_act_workspace_bytes(int64_t M, int64_t K, int64_t act_tile, int x_dtype);
QWIX_API int qwix_hip_qgemm_hadamard_act(const void* x, int x_dtype, int64_t M, int64_t N, int64_t K, const void* pre_sign,
                                const void* post_sign, float out_scale, int64_t act_tile, const void* b,
                                int64_t ldb_bytes, int b_qtype, int64_t group, const void* sb, int sb_dtype,
                                void* out, int out_dtype, int64_t ldo, void* workspace, size_t workspace_bytes,
                                void* stream);

/* qwix_hip_qgemm_grouped with K cut into ranges where its tiles are few (the same call of the reference:
 * _fast_dot_general with tiled scales, qwix/_src/core/dot_general.py:160-262): symmetric int8 x int8 / int4 operands, one
 * activation scale per row (ga == 1), more than 32 rows, exact == 0.  Every range's workgroups write the f32 sums of
 * their groups' scaled partials into `workspace` (qwix_hip_qgemm_grouped_workspace_bytes(M, N, K, group, b_qtype)
 * bytes, 16-byte aligned; 0 = this shape is not split); a second kernel adds them in range order, applies the
 * activation scale and rounds as the unsplit kernel's epilogue does.  The groups' f32 partials are then added in
 * another order than in qwix_hip_qgemm_grouped with exact == 0 (which itself is free in that order).  With workspace
 * NULL or too small, with exact != 0, zero points, per-group activation scales or acc_out: exactly
 * qwix_hip_qgemm_grouped. */
QWIX_API size_t qwix_hip_qgemm_grouped_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t group, int b_qtype);
QWIX_API int qwix_hip_qgemm_grouped_ws(const void* a, int64_t lda, const void* b, int64_t ldb_bytes, int b_qtype, int64_t M,
                              int64_t N, int64_t K, int64_t group, const void* sa, int sa_dtype, int64_t ga,
                              const void* sb, int sb_dtype, void* out, int out_dtype, int64_t ldo, int exact,
                              int32_t* acc_out, void* workspace, size_t workspace_bytes, void* stream);

/* Sub-channel GEMM with one asymmetric operand.  Replaces the zero-point terms of _fast_dot_general when a
 * contracting axis is tiled (qwix/_src/core/dot_general.py:196-203: the zero point is split with the tiles;
 * :228-253: the correction dot is subtracted from every tile's int32 partial before it is scaled):
 *     out[m,n] = cast_R( sum_g (T(acc_g[m,n] - zu[m,g] * zv[g,n]) * sa[m,g']) * sb[g,n] )
 *   lhs asymmetric:  zu = zero points of a (per row, or per row and group), zv[g,n] = sum of b[n, k in group g]
 *   rhs asymmetric:  zu[m,g] = sum of a[m, k in group g],  zv = zero points of b (per column, or per group and column)
 * zu[m,g] is read at zu[m * zu_row_stride + g * zu_group_stride], zv[g,n] at zv[n * zv_col_stride +
 * g * zv_group_stride] (int32, element strides; a group stride of 0 = one value for all groups).
 * qwix_hip_ksum_groups writes the K-sums.  acc_out, when given, receives the corrected partials.
 * Everything else as qwix_hip_qgemm_grouped. */
QWIX_API int qwix_hip_qgemm_grouped_zp(const void* a, int64_t lda, const void* b, int64_t ldb_bytes, int b_qtype,
                              int64_t M, int64_t N, int64_t K, int64_t group, const void* sa, int sa_dtype,
                              int64_t ga, const void* sb, int sb_dtype, const int32_t* zu,
                              int64_t zu_row_stride, int64_t zu_group_stride, const int32_t* zv,
                              int64_t zv_col_stride, int64_t zv_group_stride, void* out, int out_dtype,
                              int64_t ldo, int exact, int32_t* acc_out, void* stream);

/* out[r, g] = sum of the g-th group of `group` values of row r, for rows of int8 or packed int4 values
 * (ld_bytes apart, 16-byte aligned; group a multiple of 128 that divides K); out is (rows, K/group) int32.
 * The reference obtains these sums as a dot_general of the broadcast zero point against the quantized
 * values of the other operand (dot_general.py:233-239, 246-252). */
QWIX_API int qwix_hip_ksum_groups(const void* q, int qtype, int64_t ld_bytes, int64_t rows, int64_t K, int64_t group,
                         int32_t* out, void* stream);

/* bf16 x bf16 GEMM with f32 accumulation: the float contraction of the dequantize-first path
 * (_slow_dot_general, qwix/_src/core/dot_general.py:264-275: lax.dot_general on the dequantized operands) for
 * batches too large for qwix_hip_gemv_wq:  out[m,n] = cast( sum_k a[m,k] * b[n,k] ).
 *   a (M,K) and b (N,K) bf16, K-contiguous, lda / ldb in elements (multiples of 8), K % 64 == 0;
 *   out (M,N) of out_dtype in {F32, BF16}.
 * Same tile kernels as qwix_hip_qgemm (v_mfma_f32_32x32x16_bf16). */
QWIX_API int qwix_hip_gemm_bf16(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t M, int64_t N, int64_t K,
                       void* out, int out_dtype, int64_t ldo, void* stream);

/* The same contraction with the int4 / int8 weight dequantized inside the GEMM (prefill with weight-only
 * quantization: _slow_dot_general, qwix/_src/core/dot_general.py:264-275, = dequantize, qarray.py:692-708, then a
 * float dot): out[m, n] = sum_k a[m, k] * bf16((q[n, k] - zp[k / group, n]) * s[k / group, n]).  a: (M, K) bf16, row
 * pitch lda elements; q: (N, K) of q_qtype in {INT4 (packed), INT8, E4M3}, K-contiguous, row pitch ldq_bytes; s:
 * (K / group, N) in s_dtype (the product is formed in f32 and rounded to bf16 once); zp: int8 zero points laid out
 * like s, or NULL for symmetric (and e4m3) weights.  K % 256 == 0, group % 64 == 0.  Bit-identical to qwix_hip_dequantize_rm
 * (to bf16) followed by qwix_hip_gemm_bf16, without the dequantized copy of the weight. */
QWIX_API int qwix_hip_gemm_bf16_wq(const void* a, int64_t lda, const void* q, int64_t ldq_bytes, int q_qtype, int64_t M,
                          int64_t N, int64_t K, int64_t group, const void* s, int s_dtype, const int8_t* zp,
                          void* out, int out_dtype, int64_t ldo, void* stream);

/* qwix_hip_gemm_bf16_wq with K cut into ranges while its tiles would cover at most half of the CUs (the same call in
 * the reference: _slow_dot_general, qwix/_src/core/dot_general.py:264-275): every range's workgroups write f32
 * partials into `workspace` (qwix_hip_gemm_bf16_wq_workspace_bytes(M, N, K, group) bytes, 16-byte aligned; 0 = this
 * shape is not split) and a second kernel adds them in range order and rounds once to out_dtype.  The f32 sums are
 * then formed in another order than the unsplit kernel's, so results agree with qwix_hip_gemm_bf16_wq to f32
 * rounding of the accumulation, not bit for bit.  With workspace NULL or too small: exactly qwix_hip_gemm_bf16_wq. */
QWIX_API size_t qwix_hip_gemm_bf16_wq_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t group);
QWIX_API int qwix_hip_gemm_bf16_wq_ws(const void* a, int64_t lda, const void* q, int64_t ldq_bytes, int q_qtype, int64_t M,
                             int64_t N, int64_t K, int64_t group, const void* s, int s_dtype, const int8_t* zp,
                             void* out, int out_dtype, int64_t ldo, void* workspace, size_t workspace_bytes,
                             void* stream);

/* dequantize (qarray.py:692-708) of a REDUCE_MINOR qvalue that keeps that layout: out[(o, i, r)] =
 * D(D(q - zp) * scale[o, r / tile, i]) as a row-major (outer, inner, reduce) array, the K-contiguous operand
 * qwix_hip_gemm_bf16 reads.  D = `dtype` = the scale dtype; out_dtype is `dtype`, or QWIX_BF16 for f32 scales
 * (the f32 value rounded once more, as a cast of the dequantized array would).  reduce % 8 == 0, tile % 8 == 0. */
QWIX_API int qwix_hip_dequantize_rm(const void* qvalue, int qtype, int64_t outer, int64_t reduce, int64_t inner,
                           int64_t tile, const void* scale, const void* zero_point, int dtype, void* out,
                           int out_dtype, void* stream);

/* Weight-only skinny GEMM (the reference's _slow_dot_general, dot_general.py:264-275, with
 * the dequantize fused): out[m,n] = sum_k x[m,k] * (q[k,n] * s[k/group, n]).
 *   x   (M,K) bf16 row-major; q int4/int8/e4m3 K-contiguous rows (n*ldb_bytes); s (K/group, N)
 *   M <= 64 is the intended range (decode); group multiple of 128 or == K.
 */
QWIX_API int qwix_hip_gemv_wq(const void* x, int64_t ldx, const void* q, int64_t ldb_bytes, int b_qtype,
                     int64_t M, int64_t N, int64_t K, int64_t group, const void* s,
                     int s_dtype, void* out, int out_dtype, int64_t ldo, void* stream);

/* The same with asymmetric weights (calibration by min/max: dequantize is (q - zero_point) * scale,
 * qarray.py:692-708): out[m,n] = sum_k x[m,k] * ((q[k,n] - zp[k/group, n]) * s[k/group, n]).  zp: int8,
 * (K/group, N) row-major like s.  The zero point leaves through the row sums of x per group:
 * sum_k x (q - zp) = sum_k x q - zp sum_k x, in f32. */
QWIX_API int qwix_hip_gemv_wq_zp(const void* x, int64_t ldx, const void* q, int64_t ldb_bytes, int b_qtype,
                        int64_t M, int64_t N, int64_t K, int64_t group, const void* s, int s_dtype,
                        const int8_t* zp, void* out, int out_dtype, int64_t ldo, void* stream);

/* ---------------------------------------------------------------------------------------
 * Walsh-Hadamard rotation along the last axis (qwix/contrib/hadamard_rot.py:35-117):
 *     y[r, :] = ((x[r, :] * pre_sign) H_n) * post_sign * out_scale
 * H_n Sylvester/natural order, n = 2^p <= 16384, unnormalised; pre/post sign vectors are
 * +-1 arrays of `dtype` (NULL = none); out_scale is 1 for activations and 1/n for the
 * transposed weight.  Result rounded once to `dtype` (f32 butterflies inside).
 */
QWIX_API int qwix_hip_fwht(const void* x, int dtype, int64_t rows, int64_t n, const void* pre_sign,
                  const void* post_sign, float out_scale, void* y, void* stream);

/* The same rotation fused with per-row (tile == n) or per-group (tile | n) absmax
 * quantization of the rotated values; nothing but qvalue/scale is written.
 * Equals qwix_hip_fwht followed by qwix_hip_quantize(outer=rows, reduce=n, inner=1). */
QWIX_API int qwix_hip_fwht_quantize(const void* x, int dtype, int64_t rows, int64_t n,
                           const void* pre_sign, const void* post_sign, float out_scale,
                           int64_t tile, int qtype, void* qvalue, void* scale, void* stream);

/* ---------------------------------------------------------------------------------------
 * Measurement aid; no counterpart in the reference.  Runs int8 (QWIX_INT8) or OCP e4m3 (QWIX_E4M3) MFMAs back to
 * back on operands held in registers (no LDS, no memory traffic after the first loads): 256 workgroups of 8
 * wavefronts, every lane's A / B fragments taken from the caller's arrays `a` / `b` (any bytes; 16-byte aligned),
 * `iters` rounds of 32 int8 or 16 fp8 MFMAs per wavefront.  The rate it reaches is what the matrix cores of the
 * board sustain with THOSE operand bytes under its power limit: the ceiling beside the nominal peak for the
 * quantized GEMMs.  qwix_hip_mfma_ceiling_ops(iters) = operations of one launch.  `sink`: 4 writable bytes. */
QWIX_API double qwix_hip_mfma_ceiling_ops(int64_t iters);
QWIX_API int qwix_hip_mfma_ceiling(const void* a, size_t a_bytes, const void* b, size_t b_bytes, int qtype,
                          int64_t iters, int32_t* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* QWIX_HIP_H_ */
