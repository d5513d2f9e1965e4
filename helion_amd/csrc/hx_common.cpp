// Host-side plumbing shared by every entry point: version and the thread-local error string.
#include <cstdarg>
#include <cstdio>

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
