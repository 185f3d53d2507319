// common.cpp -- error reporting and library identification.
#include "common.h"

#include <cstring>

namespace bh {
namespace {
thread_local char g_last_error[512] = "";
}

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  fprintf(stderr, "[buddy_hip] %s\n", g_last_error);
  return code;
}
} // namespace bh

extern "C" {

const char *buddy_hip_version(void) { return "libbuddy_hip 0.1 (gfx950)"; }

const char *buddy_hip_last_error(void) { return bh::g_last_error; }

int buddy_hip_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess)
    return 0;
  return n;
}
}
