// Status reporting of libfastmem: per-thread last error message, launch check.
#include <stdarg.h>
#include <stdio.h>

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
}  // namespace fm

extern "C" int fm_version(void) { return 100; }
extern "C" const char* fm_last_error(void) { return fm::g_err; }
