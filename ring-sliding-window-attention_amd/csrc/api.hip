// Error buffer and version queries of the C ABI.
#include "rswa_common.h"

namespace rswa {

char* last_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace rswa

extern "C" {

const char* rswa_last_error(void) { return rswa::last_error_buffer(); }

int rswa_version(void) { return RSWA_VERSION; }

uint64_t rswa_sizeof_attn_params(void) { return sizeof(rswa_attn_params); }

}  // extern "C"
