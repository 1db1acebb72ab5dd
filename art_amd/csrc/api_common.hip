// Library-wide pieces of the artk C-ABI: error string and version.
#include "common.hpp"

namespace artk {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
}  // namespace artk

extern "C" {
int32_t artk_abi_version(void) { return 1; }
const char* artk_last_error(void) { return artk::g_err; }
}
