// Thread-local error text for the C ABI.
#include <stdarg.h>

#include "ll_common.h"

namespace ll {
static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace ll

extern "C" const char* ll_last_error(void) { return ll::g_error; }
extern "C" int ll_version(void) { return 1; }
