// launch_floor_kernels.hip -- the probe kernels of launch_floor_probe, built
// twice: as namespace `plain`, and as namespace `preload` with
// -mllvm -amdgpu-kernarg-preload-count=14, where the command processor hands
// the first 14 argument words to every wave in SGPRs instead of the wave
// loading them from memory when it starts.
#include <hip/hip_runtime.h>

#include "launch_floor_kernels.h"

namespace PROBE_NS {
namespace {

__global__ void probe_empty() {}

// reads all 30 argument words (scalar loads at wave start; a struct is never
// preloaded), stores nothing
__global__ void probe_args(Args30 a, int *sink) {
  int s = 0;
#pragma unroll
  for (int i = 0; i < 30; ++i)
    s += a.v[i];
  if (s == 0x7fffabcd)
    *sink = s;
}

// 14 argument words as separate parameters
__global__ void probe_args_split(int a0, int a1, int a2, int a3, int a4, int a5, int a6,
                                 int a7, int a8, int a9, int a10, int a11, int a12,
                                 int a13, int *sink) {
  const int s = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7 + a8 + a9 + a10 + a11 + a12 + a13;
  if (s == 0x7fffabcd)
    *sink = s;
}

// one cold 1 KiB load per wavefront (the first tile of a GEMV), nothing stored
__global__ void probe_touch(const int4 *w, unsigned tiles, int *sink) {
  const unsigned wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int4 v = w[(size_t)(wave % tiles) * 64 + (threadIdx.x & 63)];
  if ((v.x ^ v.y ^ v.z ^ v.w) == 0x7fffabcd)
    *sink = v.x;
}

// the same, and every wavefront stores 64 bytes of what it loaded (the kernel
// ends with dirty lines to write back)
__global__ void probe_touch_store(const int4 *w, unsigned tiles, int *out) {
  const unsigned wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int4 v = w[(size_t)(wave % tiles) * 64 + (threadIdx.x & 63)];
  if ((threadIdx.x & 63) < 16)
    out[wave * 16 + (threadIdx.x & 15)] = v.x ^ v.y ^ v.z ^ v.w;
}

// the same, with the wavefronts of a workgroup meeting in LDS behind a barrier
// before one of them stores (the shape of a GEMV's tail)
__global__ void probe_touch_meet_store(const int4 *w, unsigned tiles, int *out) {
  __shared__ int meet[16][17];
  const unsigned wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const unsigned wave = blockIdx.x * (blockDim.x >> 6) + wid;
  const int4 v = w[(size_t)(wave % tiles) * 64 + lane];
  if (lane < 16)
    meet[wid][lane] = v.x ^ v.y ^ v.z ^ v.w;
  __syncthreads();
  if (wid == 0 && lane < 16) {
    int s = 0;
    for (unsigned i = 0; i < (blockDim.x >> 6); ++i)
      s += meet[i][lane];
    out[blockIdx.x * 16 + lane] = s;
  }
}

// every wavefront records the 100 MHz clock when it starts (dispatch spread),
// with `lds` bytes of dynamic LDS per workgroup
__global__ void probe_start_time(unsigned long long *t, int a0, int a1, int a2, int a3,
                                 int a4, int a5, int a6, int a7, int a8, int a9, int a10,
                                 int a11) {
  extern __shared__ int dyn_lds[];
  if ((threadIdx.x & 63) == 0) {
    const unsigned wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const unsigned long long now = wall_clock64();
    t[wave] = now;
    if (now == (unsigned long long)(a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7 + a8 + a9 + a10 + a11))
      dyn_lds[0] = 1;
  }
}

// 4096 one-cycle instructions: as 16 KiB of straight-line code, and as a loop
// over 256 bytes of code
__global__ void probe_code_straight() {
#pragma unroll
  for (int i = 0; i < 64; ++i)
    asm volatile(".rept 64\n s_nop 0\n .endr" ::: "memory");
}
__global__ void probe_code_loop() {
#pragma unroll 1
  for (int i = 0; i < 64; ++i)
    asm volatile(".rept 64\n s_nop 0\n .endr" ::: "memory");
}

} // namespace

void launch(int which, int blocks, int threads, hipStream_t st, const Args30 &a,
            const void *w, unsigned tiles, int *sink) {
  const dim3 gb(blocks), tb(threads);
  switch (which) {
  case kEmpty: hipLaunchKernelGGL(probe_empty, gb, tb, 0, st); break;
  case kArgs30: hipLaunchKernelGGL(probe_args, gb, tb, 0, st, a, sink); break;
  case kArgs14:
    hipLaunchKernelGGL(probe_args_split, gb, tb, 0, st, a.v[0], a.v[1], a.v[2], a.v[3],
                       a.v[4], a.v[5], a.v[6], a.v[7], a.v[8], a.v[9], a.v[10], a.v[11],
                       a.v[12], a.v[13], sink);
    break;
  case kTouch:
    hipLaunchKernelGGL(probe_touch, gb, tb, 0, st, static_cast<const int4 *>(w), tiles, sink);
    break;
  case kTouchStore:
    hipLaunchKernelGGL(probe_touch_store, gb, tb, 0, st, static_cast<const int4 *>(w), tiles,
                       sink);
    break;
  case kTouchMeetStore:
    hipLaunchKernelGGL(probe_touch_meet_store, gb, tb, 0, st, static_cast<const int4 *>(w),
                       tiles, sink);
    break;
  case kStartTime:
    hipLaunchKernelGGL(probe_start_time, gb, tb, tiles /* dynamic LDS bytes */, st,
                       reinterpret_cast<unsigned long long *>(sink), a.v[0], a.v[1], a.v[2],
                       a.v[3], a.v[4], a.v[5], a.v[6], a.v[7], a.v[8], a.v[9], a.v[10], a.v[11]);
    break;
  case kCodeStraight: hipLaunchKernelGGL(probe_code_straight, gb, tb, 0, st); break;
  case kCodeLoop: hipLaunchKernelGGL(probe_code_loop, gb, tb, 0, st); break;
  }
}

} // namespace PROBE_NS
