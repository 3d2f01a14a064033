#include <stdarg.h>
#include "common.h"

static thread_local char g_error[512] = "";

void ts_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* ts_last_error() { return g_error; }

// Version of the C interface; the Python loader refuses a library with another one.
extern "C" int ts_abi_version() { return 1; }
