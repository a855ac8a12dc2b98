// Error reporting and library identity.
#include "common.hpp"

namespace mv {

char *last_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int status, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return status;
}

}  // namespace mv

extern "C" {
const char *mv_last_error(void) { return mv::last_error_buffer(); }
int mv_version(void) { return 1; }
}
