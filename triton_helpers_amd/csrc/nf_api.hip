// Library-wide entry points: ABI version and the thread-local error message.
#include "nf_common.h"

namespace nf {

char* last_error_buf() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buf(), 512, fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace nf

extern "C" int nf_abi_version(void) { return NF_ABI_VERSION; }
extern "C" const char* nf_last_error(void) { return nf::last_error_buf(); }
