// Error plumbing of libffmoe: thread-local last-error text, launch status.
#include "api.h"
#include <cstdarg>
#include <cstdio>

namespace ffmoe {
static thread_local char g_error[512] = "";

int ff_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
  return code;
}

int ff_launch_status() {
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    snprintf(g_error, sizeof g_error, "kernel launch failed: %s", hipGetErrorString(err));
    return int(err);
  }
  return 0;
}
}  // namespace ffmoe

extern "C" __attribute__((visibility("default"))) const char* ffmoe_last_error(void) { return ffmoe::g_error; }
extern "C" __attribute__((visibility("default"))) int ffmoe_version(void) { return FFMOE_VERSION; }
