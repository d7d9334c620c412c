// Library identification and error reporting for liblinmt_hip.so.
#include "lh_common.h"

namespace lh {

char *last_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail_arg(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return LH_ERR_ARG;
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return LH_OK;
  snprintf(last_error_buffer(), 512, "%s: %s", what, hipGetErrorString(e));
  return static_cast<int>(e);
}

}  // namespace lh

extern "C" int lh_abi_version(void) { return LH_ABI_VERSION; }

extern "C" const char *lh_last_error(void) { return lh::last_error_buffer(); }
