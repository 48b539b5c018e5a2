// Error reporting and version query of the C ABI.  No global mutable state besides the
// thread-local error string, so entry points are re-entrant across host threads.
#include "common.h"
#include <string.h>

static thread_local char g_err[512] = {0};

void zp_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* zp_last_error(void) { return g_err; }

extern "C" int zp_abi_version(void) { return 4; }
