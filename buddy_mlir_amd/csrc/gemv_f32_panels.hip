// gemv_f32_panels.hip -- the reference's panel-packed f32 decode weights on the
// device: the packing itself and the GEMV that reads it.
//
// pack_decode_matmul_weights (frontend/Python/graph/transform/
// pack_decode_weights.py:94-108) stores B[K,N] as N/V panels of [K][V]:
//   flat[nt*K*V + k*V + v] = B[k, nt*V + v]        (V = 32)
// and MatMulVectorizationDecodePackedPattern (midend/lib/Conversion/
// MatMulOptimization/MatMulVectorizationDecodePacked.cpp:207-248) walks one
// panel per task with linear offset n0*K + k*V.  A weight file written in that
// order can be consumed as is: a panel is a row-major [K, 32] matrix of its own,
// so one workgroup per panel runs the row-major f32 GEMV kernel on it (8 float4
// lanes across v, a wavefront load = 8 rows = 1 KiB of contiguous panel).
#include "common.h"

namespace bh {
int launch_gemv_f32_panels32(const float *x, const float *packed, float *y, int64_t K,
                             int64_t N, bool accumulate, hipStream_t stream);
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

} // namespace
} // namespace bh

extern "C" {

int buddy_hip_pack_panels_f32(const float *B, int64_t K, int64_t N, int V,
                              float *packed, buddy_hip_stream stream) try {
  BH_REQUIRE(B && packed && K > 0 && N > 0 && V > 0, "pack_panels: bad argument");
  // pack_decode_weights.py:95-99 refuses a ragged last panel
  BH_REQUIRE(N % V == 0, "pack_panels: N=%lld not divisible by V=%d", (long long)N, V);
  hipLaunchKernelGGL(bh::pack_panels_kernel, dim3((unsigned)bh::ceil_div(K * N, 256)),
                     dim3(256), 0, bh::as_stream(stream), B, packed, K, N, V, 0);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_pack_panels_f32")

int buddy_hip_unpack_panels_f32(const float *packed, int64_t K, int64_t N, int V,
                                float *B, buddy_hip_stream stream) try {
  BH_REQUIRE(B && packed && K > 0 && N > 0 && V > 0, "unpack_panels: bad argument");
  BH_REQUIRE(N % V == 0, "unpack_panels: N=%lld not divisible by V=%d", (long long)N, V);
  hipLaunchKernelGGL(bh::pack_panels_kernel, dim3((unsigned)bh::ceil_div(K * N, 256)),
                     dim3(256), 0, bh::as_stream(stream), packed, B, K, N, V, 1);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_unpack_panels_f32")

int buddy_hip_gemv_f32_panels(const float *x, const float *packed, float *y,
                              int64_t K, int64_t N, unsigned flags,
                              buddy_hip_stream stream) try {
  return bh::launch_gemv_f32_panels32(x, packed, y, K, N,
                                      (flags & BUDDY_HIP_GEMV_ACCUMULATE) != 0,
                                      bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_gemv_f32_panels")
}
