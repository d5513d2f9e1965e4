// Host-side plumbing shared by every entry point: version and the thread-local error string.
#include <cstdarg>
#include <cstdio>

#include <hip/hip_runtime.h>

#include <atomic>

#include "../../include/hx_kernels.h"

static thread_local char g_err[512] = "";

void hx_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* hx_last_error(void) { return g_err; }
extern "C" int hx_version(void) { return 1; }

// Compute units of the current device.  The attribute query costs microseconds, so each device is asked once.
int hx_cu_count() {
  static std::atomic<int> cached[64];  // 0 = not asked yet (racing first calls store the same value)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int cus = cached[dev].load(std::memory_order_relaxed);
  if (cus == 0) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    cached[dev].store(cus, std::memory_order_relaxed);
  }
  return cus;
}
