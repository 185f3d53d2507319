// gemv_w4a16.hip -- the reference's int4 weight-only decode GEMV (W4A16).
//
// Replaces the kernel that
// midend/lib/Conversion/MatMulOptimization/Int4DequantMatMulVectorizationDecode.cpp
// :385-468 generates: C[n] = C[n] + (sum_k a[k] * w[k][n]) * scale[n] with f16
// activations, scales, accumulator and output, int4 weights packed two per
// byte along n ([K, N/2] bytes: low nibble = even channel, high = odd;
// tools/buddy-codegen/import_model.py:810-815), and the nibble packing itself.
//
// The reference accumulates in f16, k in order: every step rounds to 11
// significand bits, so a kernel that sums in another order (or in f32) does not
// reproduce its results to 1e-3.  This kernel therefore keeps the reference's
// order: a thread owns the two channels of one byte column and walks k, rounding
// the f32 fused multiply-add to f16 after every step, which is exactly what f16
// arithmetic is on the reference's x86 target.  The result equals the
// reference's bit for bit; the price is that only N/2 threads stream the matrix
// (its own layout is already coalesced for that: a row of bytes per k).
#include "common.h"

namespace bh {
namespace {

typedef unsigned short u16;

__device__ __forceinline__ float f16_bits_to_f32(u16 h) {
  union {
    u16 u;
    _Float16 f;
  } x;
  x.u = h;
  return (float)x.f;
}
__device__ __forceinline__ float round_to_f16(float v) { return (float)(_Float16)v; }
__device__ __forceinline__ u16 f32_to_f16_bits(float v) {
  union {
    u16 u;
    _Float16 f;
  } x;
  x.f = (_Float16)v;
  return x.u;
}

constexpr int kThreads = 64;
constexpr int kStage = 2048; // activations staged per round

__global__ void __launch_bounds__(kThreads)
w4a16_gemv_kernel(const u16 *__restrict__ a, const int8_t *__restrict__ packed,
                  const u16 *__restrict__ scale, u16 *__restrict__ c, int K, int N,
                  int first_col) {
#pragma clang fp contract(off)
  __shared__ float a_s[kStage];
  const int cols = N / 2;
  const int j = first_col + blockIdx.x * kThreads + threadIdx.x;
  const bool live = j < cols;
  const int8_t *col = packed + (live ? j : 0);
  float acc0 = 0.f, acc1 = 0.f; // always exactly representable in f16
  for (int k0 = 0; k0 < K; k0 += kStage) {
    const int kn = min(kStage, K - k0);
    __syncthreads();
    for (int i = threadIdx.x; i < kn; i += kThreads)
      a_s[i] = f16_bits_to_f32(a[k0 + i]);
    __syncthreads();
    constexpr int U = 8;
    for (int kk = 0; kk < kn; kk += U) {
      int b[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        b[u] = col[(size_t)(k0 + min(kk + u, kn - 1)) * cols];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (kk + u < kn) {
          // low = ((b & 0x0F) << 4) >> 4, high = b >> 4 (arithmetic, 8 bits)
          const float lo = (float)((int)((unsigned)b[u] << 28) >> 28);
          const float hi = (float)((int)((unsigned)b[u] << 24) >> 28);
          const float x = a_s[kk + u];
          acc0 = round_to_f16(fmaf(x, lo, acc0));
          acc1 = round_to_f16(fmaf(x, hi, acc1));
        }
      }
    }
  }
  if (!live)
    return;
  const int n = 2 * j;
  const float s0 = round_to_f16(acc0 * f16_bits_to_f32(scale[n]));
  const float s1 = round_to_f16(acc1 * f16_bits_to_f32(scale[n + 1]));
  c[n] = f32_to_f16_bits(f16_bits_to_f32(c[n]) + s0);
  c[n + 1] = f32_to_f16_bits(f16_bits_to_f32(c[n + 1]) + s1);
}

// The same arithmetic for a full block of 64 byte columns whose rows can be read
// as aligned 16-byte pieces.  One wavefront per block; the matrix strip
// [K, 64 bytes] goes through LDS in blocks of kRows rows: the block after the one
// being consumed is in flight in registers (kRows * 64 B = 32 KiB per
// wavefront), which is what hides the memory latency when only N/128
// wavefronts can work at all.
constexpr int kRows = 512;                 // rows per block
constexpr int kLoads = kRows * 64 / (64 * 16); // 16-byte loads per lane and block

__global__ void __launch_bounds__(kThreads)
w4a16_gemv_block_kernel(const u16 *__restrict__ a, const int8_t *__restrict__ packed,
                        const u16 *__restrict__ scale, u16 *__restrict__ c, int K, int N) {
#pragma clang fp contract(off)
  __shared__ __attribute__((aligned(16))) unsigned char w_s[kRows * 64];
  __shared__ float a_s[kRows];
  const int cols = N / 2;
  const int lane = threadIdx.x;
  const int j = blockIdx.x * 64 + lane;
  // lane L fetches 16 bytes of row (i * 16 + L / 4), columns (L % 4) * 16 ..
  const int8_t *src = packed + (size_t)blockIdx.x * 64 + (lane & 3) * 16;
  const int lrow = lane >> 2;
  uint4 regs[kLoads];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int k = min(k0 + i * 16 + lrow, K - 1);
      regs[i] = *reinterpret_cast<const uint4 *>(src + (size_t)k * cols);
    }
  };
  float acc0 = 0.f, acc1 = 0.f; // always exactly representable in f16
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += kRows) {
    const int kn = min(kRows, K - k0);
    __syncthreads(); // the block before this one has been consumed
#pragma unroll
    for (int i = 0; i < kLoads; ++i)
      *reinterpret_cast<uint4 *>(w_s + (i * 16 + lrow) * 64 + (lane & 3) * 16) = regs[i];
    for (int i = lane; i < kn; i += kThreads)
      a_s[i] = f16_bits_to_f32(a[k0 + i]);
    __syncthreads();
    if (k0 + kRows < K)
      fetch(k0 + kRows);
    constexpr int U = 8;
    for (int kk = 0; kk < kn; kk += U) {
      int b[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        b[u] = (signed char)w_s[min(kk + u, kn - 1) * 64 + lane];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (kk + u < kn) {
          const float lo = (float)((int)((unsigned)b[u] << 28) >> 28);
          const float hi = (float)((int)((unsigned)b[u] << 24) >> 28);
          const float x = a_s[kk + u];
          acc0 = round_to_f16(fmaf(x, lo, acc0));
          acc1 = round_to_f16(fmaf(x, hi, acc1));
        }
      }
    }
  }
  const int n = 2 * j;
  const float s0 = round_to_f16(acc0 * f16_bits_to_f32(scale[n]));
  const float s1 = round_to_f16(acc1 * f16_bits_to_f32(scale[n + 1]));
  c[n] = f32_to_f16_bits(f16_bits_to_f32(c[n]) + s0);
  c[n + 1] = f32_to_f16_bits(f16_bits_to_f32(c[n + 1]) + s1);
}

// two int4 (stored as int8 in [-8, 7]) per byte, element 2i low, 2i+1 high
__global__ void __launch_bounds__(256)
pack_int4_kernel(const int8_t *__restrict__ q, int64_t pairs, int8_t *__restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= pairs)
    return;
  const unsigned lo = (unsigned)q[2 * i] & 0x0Fu, hi = ((unsigned)q[2 * i + 1] & 0x0Fu) << 4;
  out[i] = (int8_t)(lo | hi);
}

} // namespace
} // namespace bh

extern "C" {

int buddy_hip_pack_int4(const int8_t *q, int64_t count, int8_t *packed,
                        buddy_hip_stream stream) {
  BH_REQUIRE(q && packed && count > 0, "pack_int4: bad argument");
  BH_REQUIRE(count % 2 == 0, "pack_int4: odd element count %lld", (long long)count);
  hipLaunchKernelGGL(bh::pack_int4_kernel, dim3((unsigned)bh::ceil_div(count / 2, 256)),
                     dim3(256), 0, bh::as_stream(stream), q, count / 2, packed);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int buddy_hip_gemv_w4a16(const uint16_t *A, const int8_t *packed, const uint16_t *scale,
                         uint16_t *C, int64_t K, int64_t N, buddy_hip_stream stream) {
  BH_REQUIRE(A && packed && scale && C, "gemv_w4a16: null pointer");
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30),
             "gemv_w4a16: bad shape K=%lld N=%lld", (long long)K, (long long)N);
  BH_REQUIRE(N % 2 == 0, "gemv_w4a16: N=%lld is odd (two channels per byte)",
             (long long)N);
  // full blocks of 64 byte columns with 16-byte readable rows take the blocked
  // kernel, the ragged rest (or everything, if rows are not aligned) the plain one
  const int64_t cols = N / 2;
  int64_t blocked = 0;
  if (cols % 16 == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0)
    blocked = cols / 64 * 64;
  if (blocked) {
    hipLaunchKernelGGL(bh::w4a16_gemv_block_kernel, dim3((unsigned)(blocked / 64)),
                       dim3(bh::kThreads), 0, bh::as_stream(stream), A, packed, scale, C,
                       (int)K, (int)N);
  }
  if (blocked < cols) {
    hipLaunchKernelGGL(bh::w4a16_gemv_kernel,
                       dim3((unsigned)bh::ceil_div(cols - blocked, bh::kThreads)),
                       dim3(bh::kThreads), 0, bh::as_stream(stream), A, packed, scale, C,
                       (int)K, (int)N, (int)blocked);
  }
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}
}
