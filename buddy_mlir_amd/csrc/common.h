// common.h -- shared host/device helpers for libbuddy_hip.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "buddy_hip/buddy_hip.h"

namespace bh {

// Records the message for buddy_hip_last_error() and prints it to stderr, the
// way the reference's external kernels report (examples/BuddyOneDNN/
// onednn_ops.cpp:229-241: message on stderr, then return).
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define BH_CHECK_HIP(expr)                                                     \
  do {                                                                         \
    hipError_t _e = (expr);                                                    \
    if (_e != hipSuccess)                                                      \
      return ::bh::fail(BUDDY_HIP_ERR_HIP, "%s failed: %s (%s:%d)", #expr,     \
                        hipGetErrorString(_e), __FILE__, __LINE__);            \
  } while (0)

#define BH_REQUIRE(cond, ...)                                                  \
  do {                                                                         \
    if (!(cond))                                                               \
      return ::bh::fail(BUDDY_HIP_ERR_ARG, __VA_ARGS__);                       \
  } while (0)

inline hipStream_t as_stream(buddy_hip_stream s) {
  return reinterpret_cast<hipStream_t>(s);
}

constexpr int kWave = 64;          // gfx950 wavefront
constexpr int kTileN = 16;         // output channels per packed tile
constexpr int kTileK = 64;         // k values per packed tile
constexpr int kTileBytes = 1024;   // one wavefront-wide 128-bit load

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

#if defined(__HIPCC__)
// Sum across the 64 lanes of a wavefront; every lane gets the total.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1)
    v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1)
    v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
#endif

} // namespace bh
