// Library-wide pieces of the C ABI: version and the thread-local error string.
#include <stdarg.h>
#include <string.h>

#include "common.hpp"

namespace based {

static thread_local char g_last_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

}  // namespace based

extern "C" BASED_API int based_hip_version(void) { return 1; }

extern "C" BASED_API const char* based_hip_last_error(void) { return based::g_last_error; }
