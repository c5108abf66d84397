// The error record of the library: one message per host thread.
#include "hal_common.h"
#include "hal_api.h"

static thread_local char g_error[1024] = "";

int hal_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

extern "C" const char* hal_last_error() { return g_error; }

extern "C" int hal_version() { return 1; }
