// Error state + version of the C ABI.
#include "dsa_common.h"
#include <string.h>

static thread_local char g_err[512] = "";

void dsa_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" int dsa_version(void) { return 1; }
extern "C" const char* dsa_last_error(void) { return g_err; }
