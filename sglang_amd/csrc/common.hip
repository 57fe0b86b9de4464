// Error reporting and version for the libsglq C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "sglq_common.h"

namespace sglq {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
}  // namespace sglq

extern "C" const char* sglq_last_error(void) { return sglq::g_err; }
extern "C" int sglq_abi_version(void) { return 1; }
