// Error reporting, device queries and ABI version for libttpa.
#include "common.h"

#include <cstdarg>
#include <cstdio>

namespace ttpa {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TTPA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return TTPA_OK;
}

int device_cus() {
  static thread_local int cached_dev = -1, cached_cus = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev != cached_dev) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached_dev = dev;
    cached_cus = n;
  }
  return cached_cus;
}

}  // namespace ttpa

extern "C" int ttpa_abi_version(void) { return TTPA_ABI_VERSION; }
extern "C" const char *ttpa_last_error(void) { return ttpa::g_err; }
extern "C" int ttpa_device_compute_units(void) { return ttpa::device_cus(); }
