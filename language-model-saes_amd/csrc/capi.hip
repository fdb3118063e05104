// Error text and library identification for libsae_hip.so.
#include "common.h"

namespace sae {

char *error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace sae

extern "C" int sae_abi_version(void) { return 1; }
extern "C" const char *sae_last_error(void) { return sae::error_buffer(); }
