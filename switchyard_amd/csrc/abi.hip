// Error plumbing and version of the C ABI (include/switchyard_moe.h).
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace {
thread_local char g_error[512] = "";
}

int sy_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int sy_check_launch(const char* what) {
  const hipError_t err = hipGetLastError();
  if (err == hipSuccess) return SY_OK;
  return sy_fail(SY_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(err));
}

// Compute units of the current device (cached per device id; read-only after the first call).
int sy_compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

extern "C" SY_API int sy_version(void) { return 200; }  // 0.2.0: the decode-step entry points

extern "C" SY_API const char* sy_last_error(void) { return g_error; }
