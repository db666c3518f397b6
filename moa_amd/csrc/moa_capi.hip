// Error reporting and version of the C ABI.
#include "moa_common.h"

namespace moa {

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

}  // namespace moa

extern "C" int moa_abi_version(void) { return 1; }

extern "C" const char* moa_last_error(void) { return moa::error_buffer(); }
