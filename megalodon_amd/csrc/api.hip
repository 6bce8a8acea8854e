// Library-level entry points: version and error reporting.
#include "common.hpp"

#include <cstring>

namespace mega {

char* last_error_buf() {
  static thread_local char buf[512] = {0};
  return buf;
}

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buf(), 512, fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace mega

extern "C" int mega_version(void) { return 100; }

extern "C" const char* mega_last_error(void) { return mega::last_error_buf(); }
