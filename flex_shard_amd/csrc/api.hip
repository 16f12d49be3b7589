// Version and error reporting of the C ABI.
#include "common.hpp"

#include <cstring>

namespace fsh {

char* error_buffer() {
  static thread_local char buffer[512] = {0};
  return buffer;
}

int fail(int code, const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(error_buffer(), 512, fmt, args);
  va_end(args);
  return code;
}

int check_launch(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return fail(FSH_EHIP, "%s: %s", what, hipGetErrorString(err));
  return FSH_OK;
}

}  // namespace fsh

FSH_API int32_t fsh_version(void) { return (0 << 16) | 1; }

FSH_API const char* fsh_last_error(void) { return fsh::error_buffer(); }
