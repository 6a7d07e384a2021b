// Library-wide pieces of the C ABI: version and thread-local error text.
#include "fg_common.h"

namespace fg {
char* error_buffer() {
  static thread_local char buf[kErrorBufferBytes] = {0};
  return buf;
}
}  // namespace fg

extern "C" int fg_version(void) { return 100; }
extern "C" const char* fg_last_error_string(void) { return fg::error_buffer(); }
