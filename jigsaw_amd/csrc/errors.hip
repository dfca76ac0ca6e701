// Per-thread error message and ABI version of libjigsaw_hip.
#include <stdarg.h>

#include "jg_common.h"

namespace jg {

char* last_error_buf() {
  static thread_local char buf[512] = {0};
  return buf;
}

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buf(), 512, fmt, ap);
  va_end(ap);
}

}  // namespace jg

extern "C" const char* jg_last_error(void) { return jg::last_error_buf(); }
extern "C" int jg_abi_version(void) { return 1; }
