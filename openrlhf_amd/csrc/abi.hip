// Library-wide pieces of the C ABI: version and the thread-local error message.
#include <stdarg.h>
#include <string.h>

#include "common.h"

namespace orlhf {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace orlhf

extern "C" int orlhf_version(void) { return ORLHF_ABI_VERSION; }
extern "C" const char* orlhf_last_error(void) { return orlhf::g_error; }
