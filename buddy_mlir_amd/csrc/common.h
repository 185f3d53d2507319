// common.h -- shared host/device helpers for libbuddy_hip.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <initializer_list>
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

// What an exported function does when a C++ exception reaches its outermost
// scope (a std::vector that cannot grow, a standard-library error): message on
// stderr and in buddy_hip_last_error(), then an ordinary error return, like the
// reference's external kernels (examples/BuddyOneDNN/onednn_ops.cpp:229-241).
// Every extern "C" definition is a function-try-block ending in one of the
// BH_CATCH_* handlers, so nothing unwinds through the C ABI.
int caught(const char *where) noexcept;

#define BH_CATCH_INT(name)                                                     \
  catch (...) { return ::bh::caught(name); }
#define BH_CATCH_VOID(name)                                                    \
  catch (...) { (void)::bh::caught(name); }
#define BH_CATCH_NULL(name)                                                    \
  catch (...) {                                                                \
    (void)::bh::caught(name);                                                  \
    return nullptr;                                                            \
  }

// A kernel that asks for more dynamic LDS than the default limit needs
// hipFuncAttributeMaxDynamicSharedMemorySize raised once per device.  One
// DynLdsOnce per launch site (a function-local static) keeps a bit per device;
// host threads that launch at the same time on separate streams may both make
// the (idempotent) call, none skips it before it has succeeded.
struct DynLdsOnce {
  std::atomic<uint64_t> done{0};
};
inline hipError_t ensure_dyn_lds(DynLdsOnce &once, const void *kernel, int bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (once.done.load(std::memory_order_acquire) & bit)
    return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess)
    once.done.fetch_or(bit, std::memory_order_release);
  return e;
}

inline hipStream_t as_stream(buddy_hip_stream s) {
  return reinterpret_cast<hipStream_t>(s);
}

constexpr int kWave = 64;          // gfx950 wavefront
constexpr int kTileN = 16;         // output channels per packed tile
constexpr int kTileK = 64;         // k values per packed tile
constexpr int kTileBytes = 1024;   // one wavefront-wide 128-bit load

// ---- which template instantiations of the hand-scheduled kernels were launched
// Every instantiation a launch site can reach registers itself when the library
// is loaded (a static member of Variant<Family, params...>, instantiated where
// the launch site names it) and counts its launches, so that a test can ask
// whether every compiled variant of such a kernel has met the oracle
// (buddy_hip_variant_report).
int register_variant(const char *family, std::initializer_list<int> params);
void note_variant_launch(int id);
template <typename Family, int... P> struct Variant {
  static inline const int id = register_variant(Family::name, {P...});
};
#define BH_VARIANT_FAMILY(tag, text)                                           \
  struct tag {                                                                 \
    static constexpr const char *name = text;                                  \
  }
#define BH_NOTE_VARIANT(...) ::bh::note_variant_launch(::bh::Variant<__VA_ARGS__>::id)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// The k-slices per channel group are a power of two (the planners only double or
// halve them), so a wavefront finds its slice with a shift and a mask instead of
// the forty-odd scalar instructions of a division ahead of its first load.
inline bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

#if defined(__HIPCC__)
__device__ __forceinline__ int shift_of(int pow2) { return __builtin_ctz((unsigned)pow2); }

// One-instruction transcendental forms (v_exp_f32, v_rcp_f32, v_rsq_f32: 1 ulp)
// for the epilogues of the decode kernels, where a single wavefront finishes a
// tile alone and the library routines' twenty-odd dependent instructions each
// would sit on the critical path of the launch.
__device__ __forceinline__ float fast_exp(float x) {
  return __builtin_amdgcn_exp2f(x * 1.44269504088896341f);
}
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float fast_rsqrt(float x) { return __builtin_amdgcn_rsqf(x); }

// Cross-lane reductions on DPP (data-parallel primitives: a VALU operand read
// from another lane of the same row of 16, a few cycles) instead of
// ds_bpermute round trips through the LDS crossbar.
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// every lane gets the sum of its row of 16 lanes
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f<0xB1>(v);  // quad_perm [1,0,3,2]
  v += dpp_f<0x4E>(v);  // quad_perm [2,3,0,1]
  v += dpp_f<0x141>(v); // row_half_mirror
  v += dpp_f<0x140>(v); // row_mirror
  return v;
}
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));
  v = fmaxf(v, dpp_f<0x4E>(v));
  v = fmaxf(v, dpp_f<0x141>(v));
  v = fmaxf(v, dpp_f<0x140>(v));
  return v;
}
__device__ __forceinline__ float lane_f(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
// Sum across the 64 lanes of a wavefront; every lane gets the total.
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  return (lane_f(v, 0) + lane_f(v, 16)) + (lane_f(v, 32) + lane_f(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
  v = row16_max(v);
  return fmaxf(fmaxf(lane_f(v, 0), lane_f(v, 16)), fmaxf(lane_f(v, 32), lane_f(v, 48)));
}
// Maximum of an unsigned value over the 64 lanes.  With the bit pattern of |x|
// (sign cleared) as the value this is a magnitude maximum in which a NaN or an
// infinity wins over every finite number, where fmaxf would drop a NaN.
__device__ __forceinline__ unsigned wave_max_u32(unsigned v) {
  v = max(v, (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, true));
  v = max(v, (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, true));
  v = max(v, (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, true));
  v = max(v, (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xf, 0xf, true));
  const unsigned a = __builtin_amdgcn_readlane((int)v, 0), b = __builtin_amdgcn_readlane((int)v, 16);
  const unsigned c = __builtin_amdgcn_readlane((int)v, 32), d = __builtin_amdgcn_readlane((int)v, 48);
  return max(max(a, b), max(c, d));
}
// v of this lane and v of lane ^ 32 (W = 32) or lane ^ 16 (W = 16), in an order
// that depends on the lane: for commutative merges.  One VALU instruction
// (v_permlane32_swap / v_permlane16_swap) instead of a trip through the LDS
// crossbar (ds_bpermute).
template <int W> __device__ __forceinline__ void lane_pair(float v, float &a, float &b) {
  static_assert(W == 16 || W == 32, "rows (16) or halves (32) of a wavefront");
  const unsigned u = __float_as_uint(v);
  if constexpr (W == 32) {
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    a = __uint_as_float(r[0]);
    b = __uint_as_float(r[1]);
  } else {
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __uint_as_float(r[0]);
    b = __uint_as_float(r[1]);
  }
}
template <int W> __device__ __forceinline__ float sum_xor(float v) {
  float a, b;
  lane_pair<W>(v, a, b);
  return a + b;
}
// every lane gets the sum over the lanes l, l ^ 16, l ^ 32, l ^ 48
__device__ __forceinline__ float sum_rows(float v) { return sum_xor<32>(sum_xor<16>(v)); }
// sum over the 4 lanes of a quad / the 8 lanes of two adjacent quads
__device__ __forceinline__ float quad_sum(float v) {
  v += dpp_f<0xB1>(v);
  v += dpp_f<0x4E>(v);
  return v;
}
#endif

} // namespace bh
