// Error reporting shared by all entry points, and a version tag the loader checks.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

extern "C" const char* me_last_error() { return g_error; }

int me_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

int me_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return me_fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

extern "C" int me_abi_version() { return 8; }
