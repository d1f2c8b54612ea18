// Version and error-string entry points of libomni_dit_hip.so.
#include <stdarg.h>

#include <atomic>

#include "odit_common.h"

namespace odit {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

uint64_t next_ticket_epoch() {
  static std::atomic<uint64_t> epoch{0};
  return (epoch.fetch_add(1, std::memory_order_relaxed) + 1) & ((1ull << 47) - 1);
}
}  // namespace odit

extern "C" int odit_version(void) { return ODIT_VERSION; }
extern "C" const char* odit_last_error(void) { return odit::g_err; }
