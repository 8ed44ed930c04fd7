// Error buffer and version of the C ABI.
#include "rd_common.h"

namespace rd {

char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace rd

extern "C" int rd_version(void) { return 100; }
extern "C" const char* rd_last_error(void) { return rd::error_buffer(); }
