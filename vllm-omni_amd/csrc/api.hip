// Version and error-string entry points of libomni_dit_hip.so.
#include <stdarg.h>

#include "odit_common.h"

namespace odit {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
}  // namespace odit

extern "C" int odit_version(void) { return ODIT_VERSION; }
extern "C" const char* odit_last_error(void) { return odit::g_err; }
