// Error text and ABI version of the C surface.
#include "common.h"

namespace mi355 {

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
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return MI355_OK;
  return fail(MI355_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
}

}  // namespace mi355

extern "C" int mi355_moe_abi_version(void) { return MI355_MOE_ABI_VERSION; }
extern "C" const char* mi355_moe_last_error(void) { return mi355::error_buffer(); }
