// Status reporting of libfastmem: per-thread last error message, launch check.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

#include "common.hpp"

namespace fm {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return FM_OK;
  set_error("%s: %s", what, hipGetErrorString(e));
  return FM_ERR_LAUNCH;
}

// The process-wide switches of fastmem_debug.h take effect only in a process that asked for them before its
// first call into the library: FASTMEM_DEBUG_HOOKS=1 in the environment.  Anywhere else the setters do
// nothing, so one caller cannot reroute another caller's kernels.
bool debug_hooks_enabled() {
  static const bool on = [] {
    const char* e = getenv("FASTMEM_DEBUG_HOOKS");
    return e && e[0] == '1' && e[1] == 0;
  }();
  return on;
}
}  // namespace fm

extern "C" int fm_debug_hooks_enabled(void) { return fm::debug_hooks_enabled() ? 1 : 0; }
extern "C" int fm_version(void) { return 100; }
extern "C" const char* fm_last_error(void) { return fm::g_err; }
