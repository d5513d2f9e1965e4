// Host-side plumbing shared by every entry point: version and the thread-local error string.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>

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

// Kernel paths that have passed the CPU-side checks but not yet a run on the hardware are compiled in and switched off:
// a bit of this mask turns one on.  Initial value: the environment variable HX_FEATURES (a number, read once).
static std::atomic<unsigned> g_features{~0u};  // ~0u: not initialised
static unsigned features_now() {
  unsigned f = g_features.load(std::memory_order_relaxed);
  if (f == ~0u) {
    const char* e = getenv("HX_FEATURES");
    f = e ? (unsigned)strtoul(e, nullptr, 0) & 0x7FFFFFFFu : 0u;
    unsigned expect = ~0u;
    if (!g_features.compare_exchange_strong(expect, f, std::memory_order_relaxed)) f = expect;
  }
  return f;
}
bool hx_feature(unsigned bit) { return (features_now() & bit) != 0; }
extern "C" unsigned hx_get_features(void) { return features_now(); }
extern "C" unsigned hx_set_features(unsigned mask) {
  const unsigned old = features_now();
  g_features.store(mask & 0x7FFFFFFFu, std::memory_order_relaxed);
  return old;
}
