// The error channel of the C interface: every entry point returns 0 or sets a
// message (per host thread) that nhv_last_error() hands out. Part of every library.
#include "nhv_common.h"
#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

int nhv_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

extern "C" const char* nhv_last_error() { return g_error; }
