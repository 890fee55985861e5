// Temporary: entry points whose kernels are not written yet.
#include "common.h"
using namespace qwix;
extern "C" {
int qwix_hip_qgemm_grouped(const void*, int64_t, const void*, int64_t, int, int64_t, int64_t, int64_t, int64_t,
                           const void*, int, int64_t, const void*, int, void*, int, int64_t, int, int32_t*, void*) {
  return fail(QWIX_ERR_UNSUPPORTED, "qgemm_grouped: not built yet");
}
int qwix_hip_gemv_wq(const void*, int64_t, const void*, int64_t, int, int64_t, int64_t, int64_t, int64_t, const void*,
                     int, void*, int, int64_t, void*) {
  return fail(QWIX_ERR_UNSUPPORTED, "gemv_wq: not built yet");
}
int qwix_hip_fwht(const void*, int, int64_t, int64_t, const void*, const void*, float, void*, void*) {
  return fail(QWIX_ERR_UNSUPPORTED, "fwht: not built yet");
}
int qwix_hip_fwht_quantize(const void*, int, int64_t, int64_t, const void*, const void*, float, int64_t, int, void*,
                           void*, void*) {
  return fail(QWIX_ERR_UNSUPPORTED, "fwht_quantize: not built yet");
}
}
