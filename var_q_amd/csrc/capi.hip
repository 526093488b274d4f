// Error reporting and version query of the C ABI (varq.h).
#include "varq_common.h"

static thread_local char g_err[512] = "";

int varq_set_error(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" const char *varq_last_error(void) { return g_err; }
extern "C" int varq_abi_version(void) { return VARQ_ABI_VERSION; }
