// Error reporting and version query of the C ABI.
#include <stdarg.h>

#include "common.h"

namespace {
thread_local char g_last_error[512] = "";
}

void msa_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

extern "C" const char* msa_last_error(void) { return g_last_error; }

extern "C" int msa_version(void) { return 1; }
