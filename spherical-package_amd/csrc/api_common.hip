// Error reporting and version query of the C ABI.
#include <cstdarg>
#include <cstdio>

#include "sdk_host.hpp"

namespace sdk {
static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace sdk

extern "C" {
const char* sdk_last_error(void) { return sdk::g_error; }
int sdk_version(void) { return 100; }
}
