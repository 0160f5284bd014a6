// Error reporting, size queries and version of libksq_hip.
#include <cstring>

#include "ksq_common.h"

namespace ksq {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(KSQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return KSQ_OK;
}

}  // namespace ksq

KSQ_EXPORT int ksq_version(void) { return KSQ_VERSION; }

KSQ_EXPORT const char* ksq_last_error_string(void) { return ksq::g_err; }

KSQ_EXPORT size_t ksq_w4a16_packed_weight_bytes(size_t E, size_t K, size_t N) { return E * K * N / 2; }

KSQ_EXPORT size_t ksq_w4a16_packed_scales_bytes(size_t E, size_t K, size_t N, size_t group, int dtype) {
  if (group == 0) return 0;
  return E * (K / group) * N * (dtype == KSQ_F32 ? 4 : 2);
}

KSQ_EXPORT size_t ksq_w4a16_packed_zeros_bytes(size_t E, size_t K, size_t N, size_t group) {
  if (group == 0) return 0;
  return E * (K / group) * N;
}
