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

void arm_profile_events(void *before, void *after);

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

bool ensure_dynamic_lds(const void *kernel, size_t bytes, std::atomic<uint64_t> &done_devices) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const uint64_t bit = (dev >= 0 && dev < 64) ? (uint64_t{1} << dev) : 0;
  if (bit && (done_devices.load(std::memory_order_acquire) & bit)) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  if (bit) done_devices.fetch_or(bit, std::memory_order_release);
  return true;
}

static thread_local hipEvent_t g_ev_before = nullptr, g_ev_after = nullptr;

void take_profile_events(hipEvent_t &before, hipEvent_t &after) {
  before = g_ev_before;
  after = g_ev_after;
  g_ev_before = g_ev_after = nullptr;
}

void arm_profile_events(void *before, void *after) {
  g_ev_before = static_cast<hipEvent_t>(before);
  g_ev_after = static_cast<hipEvent_t>(after);
}

}  // namespace ttpa

extern "C" int ttpa_profile_next_attention(void *before, void *after) {
  if ((before == nullptr) != (after == nullptr))
    return ttpa::fail(TTPA_ERR_INVALID_ARGUMENT, "pass both events or neither");
  ttpa::arm_profile_events(before, after);
  return TTPA_OK;
}

extern "C" int ttpa_abi_version(void) { return TTPA_ABI_VERSION; }
extern "C" const char *ttpa_last_error(void) { return ttpa::g_err; }
extern "C" int ttpa_device_compute_units(void) { return ttpa::device_cus(); }
