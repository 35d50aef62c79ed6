// Error reporting, device queries and version of libm2_amd.so.
#include <stdarg.h>
#include <stdio.h>

#include "m2_internal.h"

namespace m2 {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(M2_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return M2_OK;
}

int num_cus() {
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

}  // namespace m2

extern "C" int m2_version(void) { return M2_AMD_VERSION; }
extern "C" const char* m2_last_error(void) { return m2::g_err; }
