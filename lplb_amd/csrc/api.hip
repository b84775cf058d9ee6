// Error reporting and version query of the C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace lplb {

static thread_local char g_last_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

} // namespace lplb

extern "C" const char *lplb_last_error(void) { return lplb::g_last_error; }

extern "C" int lplb_abi_version(void) { return LPLB_ABI_VERSION; }
