// Error reporting for the C ABI: a thread-local message per failing call.
#include <stdarg.h>
#include <stdio.h>

#include "../../include/emi.h"

static thread_local char g_last_error[512] = "";

extern "C" int emi_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" const char* emi_last_error(void) { return g_last_error; }

extern "C" int emi_abi_version(void) { return EMI_ABI_VERSION; }
