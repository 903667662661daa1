// Thread-local error message plumbing and version query.
#include "fr_common.h"

#include <stdarg.h>

namespace fr {

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

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(FR_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return FR_OK;
}

}  // namespace fr

extern "C" int fr_version(void) { return 100; }
extern "C" const char* fr_last_error_string(void) { return fr::error_buffer(); }
