// Library-wide entry points of the C ABI: version and thread-local error text.
#include "common.h"

namespace ttamd {
char* error_buffer() {
  static thread_local char buf[kErrorBufferBytes] = {0};
  return buf;
}
}  // namespace ttamd

extern "C" int ttamd_version(void) { return TTAMD_ABI_VERSION; }
extern "C" const char* ttamd_last_error(void) { return ttamd::error_buffer(); }
