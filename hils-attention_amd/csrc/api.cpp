// Error reporting shared by every entry point of libhils_amd.so.
#include <stdarg.h>
#include <stdio.h>
#include "../../include/hils_amd.h"

static thread_local char g_err[512] = "";

void hils_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* hils_last_error(void) { return g_err; }
extern "C" int hils_version(void) { return 1; }
