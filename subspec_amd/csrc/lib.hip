// Library-level entry points: ABI version and the thread-local error message.
#include "common.h"

namespace subspec {
static thread_local char g_error[512] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace subspec

extern "C" int subspec_abi_version(void) { return SUBSPEC_ABI_VERSION; }
extern "C" const char* subspec_last_error(void) { return subspec::g_error; }
