// Error reporting and build information of the itexhip C ABI (host only).
#include <stdarg.h>

#include "common.hpp"

namespace itexhip {
namespace {
thread_local char g_error[512] = "";
}

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace itexhip

extern "C" const char* itexhip_last_error(void) { return itexhip::g_error; }

extern "C" const char* itexhip_build_info(void) { return "itexhip 0.1 gfx950"; }
