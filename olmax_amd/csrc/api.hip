// Library-wide entry points of libolmax_hip: error reporting and version.
#include "common.h"
#include <string.h>

static thread_local char g_err[512] = "";

int olmax_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" const char* olmax_last_error_string(void) { return g_err; }

extern "C" int32_t olmax_abi_version(void) { return 1; }
