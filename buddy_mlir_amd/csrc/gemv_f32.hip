// gemv_f32.hip -- plain f32 decode GEMV: y[N] = bias[N] + x[K] . B[K,N].
//
// The f32 sibling of the int8 kernel: the loop nest of
// midend/lib/Conversion/MatMulOptimization/MatMulVectorizationDecode.cpp:142-175
// (and of MatMulVectorizationDecodePacked.cpp:207-248 for the panel-packed
// layout, which exists to fix a CPU page-stride problem that a GPU reading
// whole rows across lanes does not have).  In the reference's shipped w8a32
// build the q/k/v projections are this kernel followed by a bias add
// (examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:73-85).
//
// B is row-major with N contiguous, so lanes run along n: a wavefront reads
// four rows x 64 columns per 128-bit load; the 16 wavefronts of a workgroup
// take interleaved rows of the same 64 columns and meet in LDS.
#include "common.h"

namespace bh {
namespace {

constexpr int kWaves = 16;

__global__ void __launch_bounds__(kWaves * 64)
gemv_f32_kernel(const float *__restrict__ x, const float *__restrict__ B,
                const float *__restrict__ bias, float *__restrict__ y, int K,
                int N, int64_t ldb, int accumulate) {
  __shared__ float4 red[kWaves][64];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int col = blockIdx.x * 64 + (lane & 15) * 4; // 4 columns per lane
  const int rsub = lane >> 4;                        // 4 rows per wavefront load
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  const bool full = col + 3 < N && ((ldb & 3) == 0) &&
                    ((reinterpret_cast<uintptr_t>(B) & 15) == 0);
  for (int k = wave * 4 + rsub; k < K; k += kWaves * 4) {
    const float xv = x[k];
    const float *row = B + (int64_t)k * ldb + col;
    float4 b;
    if (full)
      b = *reinterpret_cast<const float4 *>(row);
    else
      b = make_float4(col < N ? row[0] : 0.f, col + 1 < N ? row[1] : 0.f,
                      col + 2 < N ? row[2] : 0.f, col + 3 < N ? row[3] : 0.f);
    acc.x = fmaf(xv, b.x, acc.x);
    acc.y = fmaf(xv, b.y, acc.y);
    acc.z = fmaf(xv, b.z, acc.z);
    acc.w = fmaf(xv, b.w, acc.w);
  }
  red[wave][lane] = acc;
  __syncthreads();
  if (tid < 16) { // 16 lanes x 4 columns = the workgroup's 64 columns
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int w = 0; w < kWaves; ++w)
      for (int r = 0; r < 4; ++r) {
        const float4 v = red[w][r * 16 + tid];
        s.x += v.x;
        s.y += v.y;
        s.z += v.z;
        s.w += v.w;
      }
    const int c0 = blockIdx.x * 64 + tid * 4;
    const float out[4] = {s.x, s.y, s.z, s.w};
    for (int j = 0; j < 4; ++j) {
      const int n = c0 + j;
      if (n < N) {
        float v = out[j];
        if (bias)
          v = bias[n] + v; // tosa.add(bias, matmul)
        y[n] = accumulate ? y[n] + v : v;
      }
    }
  }
}

__global__ void __launch_bounds__(256)
bias_rows_kernel(float *__restrict__ C, const float *__restrict__ bias, int64_t M,
                 int64_t N) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < M * N)
    C[i] = bias[i % N];
}

} // namespace

int launch_gemv_f32(const float *x, const float *B, const float *bias, float *y,
                    int64_t K, int64_t N, int64_t ldb, bool accumulate,
                    hipStream_t stream) {
  BH_REQUIRE(x && B && y, "gemv_f32: null pointer");
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30) && ldb >= N,
             "gemv_f32: bad shape K=%lld N=%lld ldb=%lld", (long long)K,
             (long long)N, (long long)ldb);
  hipLaunchKernelGGL(gemv_f32_kernel, dim3((unsigned)ceil_div(N, 64)),
                     dim3(kWaves * 64), 0, stream, x, B, bias, y, (int)K, (int)N,
                     ldb, accumulate ? 1 : 0);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_bias_rows(float *C, const float *bias, int64_t M, int64_t N,
                     hipStream_t stream) {
  BH_REQUIRE(C && bias && M > 0 && N > 0, "bias_rows: bad argument");
  hipLaunchKernelGGL(bias_rows_kernel, dim3((unsigned)ceil_div(M * N, 256)),
                     dim3(256), 0, stream, C, bias, M, N);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace bh

extern "C" {

int buddy_hip_gemv_f32(const float *x, const float *B, const float *bias,
                       float *y, int64_t K, int64_t N, unsigned flags,
                       buddy_hip_stream stream) {
  return bh::launch_gemv_f32(x, B, bias, y, K, N, N,
                             (flags & BUDDY_HIP_GEMV_ACCUMULATE) != 0,
                             bh::as_stream(stream));
}
}
