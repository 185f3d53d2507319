// common.cpp -- error reporting and library identification.
#include "common.h"

#include <algorithm>
#include <atomic>
#include <cstring>
#include <deque>
#include <exception>
#include <mutex>
#include <new>
#include <string>

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

namespace {
struct VariantEntry {
  std::string name;
  std::atomic<long long> launches{0};
};
// built on first use: registrations run during the dynamic initialisation of
// several translation units, in no particular order
struct VariantTable {
  std::mutex mu;
  std::deque<VariantEntry> entries; // a deque never moves its elements
};
VariantTable &variants() {
  static VariantTable t;
  return t;
}
} // namespace

int register_variant(const char *family, std::initializer_list<int> params) {
  std::string name = family;
  name += '<';
  bool first = true;
  for (int p : params) {
    if (!first)
      name += ", ";
    name += std::to_string(p);
    first = false;
  }
  name += '>';
  VariantTable &t = variants();
  std::lock_guard<std::mutex> lock(t.mu);
  t.entries.emplace_back();
  t.entries.back().name = std::move(name);
  return (int)t.entries.size() - 1;
}

void note_variant_launch(int id) {
  VariantTable &t = variants();
  VariantEntry *e;
  {
    std::lock_guard<std::mutex> lock(t.mu);
    e = &t.entries[(size_t)id];
  }
  e->launches.fetch_add(1, std::memory_order_relaxed);
}
} // namespace bh

extern "C" {

int64_t buddy_hip_variant_report(char *text, int64_t capacity) try {
  bh::VariantTable &t = bh::variants();
  std::string out;
  {
    std::lock_guard<std::mutex> lock(t.mu);
    for (const bh::VariantEntry &e : t.entries)
      out += e.name + '\t' + std::to_string(e.launches.load(std::memory_order_relaxed)) + '\n';
  }
  if (text && capacity > 0) {
    const size_t n = std::min(out.size(), (size_t)capacity - 1);
    std::memcpy(text, out.data(), n);
    text[n] = 0;
  }
  return (int64_t)out.size() + 1;
} catch (...) {
  return 0;
}

void buddy_hip_variant_reset(void) try {
  bh::VariantTable &t = bh::variants();
  std::lock_guard<std::mutex> lock(t.mu);
  for (bh::VariantEntry &e : t.entries)
    e.launches.store(0, std::memory_order_relaxed);
} catch (...) {
}

const char *buddy_hip_version(void) { return "libbuddy_hip 0.1 (gfx950)"; }

const char *buddy_hip_last_error(void) { return bh::g_last_error; }

int buddy_hip_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess)
    return 0;
  return n;
}
}
