// Thread-local error text and ABI version of libmoespresso_amd.so.
#include <stdarg.h>
#include <stdio.h>

#include "../../include/moespresso_amd.h"

static thread_local char g_last_error[512] = "";

void mspr_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* mspr_last_error(void) { return g_last_error; }

extern "C" int mspr_abi_version(void) { return 5; }
