// Error reporting and version of the C ABI declared in include/mega_hip.h.
#include "common.h"

namespace mega {
namespace {
thread_local char g_err[512] = "";
}
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
}  // namespace mega

extern "C" const char* mega_last_error(void) { return mega::g_err; }
extern "C" int mega_abi_version(void) { return 2; }
