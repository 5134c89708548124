// Host-side plumbing shared by every entry point: version, thread-local error
// text, launch-status check.
#include <map>
#include <mutex>
#include <utility>

#include "common.hip.h"

namespace frnnt {

char *error_buffer() {
  static thread_local char text[512] = {0};
  return text;
}

int fail(int code, const char *fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(error_buffer(), 512, fmt, args);
  va_end(args);
  return code;
}

int check_launch(const char *what) {
  const hipError_t err = hipGetLastError();
  if (err == hipSuccess) return FRNNT_OK;
  return fail(FRNNT_ELAUNCH, "%s: %s", what, hipGetErrorString(err));
}

bool allow_lds(const void *kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return true;
  static std::mutex guard;
  static std::map<std::pair<int, const void *>, size_t> granted;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return false;
  std::lock_guard<std::mutex> lock(guard);
  size_t &have = granted[std::make_pair(device, kernel)];
  if (have >= bytes) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) !=
      hipSuccess)
    return false;
  have = bytes;
  return true;
}

}  // namespace frnnt

extern "C" {

int frnnt_version(void) { return 100; }

const char *frnnt_last_error(void) { return frnnt::error_buffer(); }

}  // extern "C"
