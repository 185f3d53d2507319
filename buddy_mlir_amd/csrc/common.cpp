// common.cpp -- error reporting and library identification.
#include "common.h"

#include <cstring>
#include <exception>
#include <new>

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

int caught(const char *where) noexcept {
  try {
    throw; // the exception being handled by the caller's catch (...)
  } catch (const std::bad_alloc &) {
    return fail(BUDDY_HIP_ERR_HOST, "%s: out of host memory", where);
  } catch (const std::exception &e) {
    return fail(BUDDY_HIP_ERR_HOST, "%s: %s", where, e.what());
  } catch (...) {
    return fail(BUDDY_HIP_ERR_HOST, "%s: unknown C++ exception", where);
  }
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
