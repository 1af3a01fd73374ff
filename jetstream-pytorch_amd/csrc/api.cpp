// Library-wide state: version and the thread-local error message.
#include "common.h"

namespace jpt {
char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}
}  // namespace jpt

extern "C" {
int32_t jpt_version(void) { return 1; }
const char* jpt_last_error(void) { return jpt::error_buffer(); }
}
