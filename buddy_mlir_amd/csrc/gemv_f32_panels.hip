// gemv_f32_panels.hip -- the reference's panel-packed f32 decode weights on the
// device: the packing itself and the GEMV that reads it.
//
// pack_decode_matmul_weights (frontend/Python/graph/transform/
// pack_decode_weights.py:94-108) stores B[K,N] as N/V panels of [K][V]:
//   flat[nt*K*V + k*V + v] = B[k, nt*V + v]        (V = 32)
// and MatMulVectorizationDecodePackedPattern (midend/lib/Conversion/
// MatMulOptimization/MatMulVectorizationDecodePacked.cpp:207-248) walks one
// panel per task with linear offset n0*K + k*V.  A weight file written in that
// order can be consumed as is: one workgroup per panel, 32 lanes across v
// (128 contiguous bytes per row), 8 rows in flight per load, rows met in LDS.
#include "common.h"

namespace bh {
namespace {

__global__ void __launch_bounds__(256)
pack_panels_kernel(const float *__restrict__ B, float *__restrict__ P, int64_t K,
                   int64_t N, int V, int inverse) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= K * N)
    return;
  const int64_t k = i / N, n = i % N;
  const int64_t packed = (n / V) * K * V + k * V + n % V;
  if (inverse)
    P[i] = B[packed]; // B holds the panels, P the plain matrix
  else
    P[packed] = B[i];
}

__global__ void __launch_bounds__(256)
gemv_panels_kernel(const float *__restrict__ x, const float *__restrict__ flatB,
                   float *__restrict__ y, int K, int N, int zero_init) {
  constexpr int V = 32;
  __shared__ float red[8][V];
  const int v = threadIdx.x & 31, kg = threadIdx.x >> 5;
  const int64_t n0 = (int64_t)blockIdx.x * V;
  const float *panel = flatB + n0 * K;
  float acc = 0.f;
  for (int k = kg; k < K; k += 8)
    acc = fmaf(x[k], panel[(int64_t)k * V + v], acc);
  red[kg][v] = acc;
  __syncthreads();
  if (kg == 0) {
    float s = zero_init ? 0.f : y[n0 + v];
#pragma unroll
    for (int g = 0; g < 8; ++g)
      s += red[g][v];
    y[n0 + v] = s;
  }
}

} // namespace
} // namespace bh

extern "C" {

int buddy_hip_pack_panels_f32(const float *B, int64_t K, int64_t N, int V,
                              float *packed, buddy_hip_stream stream) {
  BH_REQUIRE(B && packed && K > 0 && N > 0 && V > 0, "pack_panels: bad argument");
  // pack_decode_weights.py:95-99 refuses a ragged last panel
  BH_REQUIRE(N % V == 0, "pack_panels: N=%lld not divisible by V=%d", (long long)N, V);
  hipLaunchKernelGGL(bh::pack_panels_kernel, dim3((unsigned)bh::ceil_div(K * N, 256)),
                     dim3(256), 0, bh::as_stream(stream), B, packed, K, N, V, 0);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int buddy_hip_unpack_panels_f32(const float *packed, int64_t K, int64_t N, int V,
                                float *B, buddy_hip_stream stream) {
  BH_REQUIRE(B && packed && K > 0 && N > 0 && V > 0, "unpack_panels: bad argument");
  BH_REQUIRE(N % V == 0, "unpack_panels: N=%lld not divisible by V=%d", (long long)N, V);
  hipLaunchKernelGGL(bh::pack_panels_kernel, dim3((unsigned)bh::ceil_div(K * N, 256)),
                     dim3(256), 0, bh::as_stream(stream), packed, B, K, N, V, 1);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int buddy_hip_gemv_f32_panels(const float *x, const float *packed, float *y,
                              int64_t K, int64_t N, unsigned flags,
                              buddy_hip_stream stream) {
  BH_REQUIRE(x && packed && y, "gemv_f32_panels: null pointer");
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30) && N % 32 == 0,
             "gemv_f32_panels: K=%lld N=%lld (N must be a multiple of 32)",
             (long long)K, (long long)N);
  hipLaunchKernelGGL(bh::gemv_panels_kernel, dim3((unsigned)(N / 32)), dim3(256), 0,
                     bh::as_stream(stream), x, packed, y, (int)K, (int)N,
                     (flags & BUDDY_HIP_GEMV_ACCUMULATE) ? 0 : 1);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}
}
