// gemv_w8a8.hip -- w8a8 matmul: dynamic per-tensor int8 activations times int8
// weights with exact int32 partial sums.
//
// Replaces quantized_matmul_op / _quantize_activation_i8
// (frontend/Python/ops/linalg.py:12728-12847):
//   s_a  = max(absmax(x) * (1/127), 1e-10)            (:12737-12760)
//   x_q  = clamp(f32(i32(x * (1/s_a))), -128, 127)     (:12761-12792; the TOSA
//          f32 -> i32 cast rounds to nearest even)
//   acc  = x_q (i8) . W (i8) -> i32                    (:12814-12831)
//   y    = f32(acc) * (s_a * s_w[n])                   (:12833-12845)
// The int8 weights are the same wave-tile packed copy the w8a32 kernels read;
// the dot products run on v_dot4_i32_i8 (four multiply-adds per lane per
// instruction), so the partial sums are exact integers whatever the order.
//
// Above 16 rows the product runs on the int8 matrix cores (the i8 x i8 -> i32
// branch of the reference's BLIS kernel,
// midend/lib/Conversion/MatMulOptimization/MatMulBlisVectorization.cpp:668-724):
// the quantised activations are written as one plane in the layout the prefill
// matmul reads, by two launches (partial maxima over the tensor, then one
// workgroup per row), and the prefill kernel multiplies it with whole K per
// workgroup, so that the int32 sums stay whole.
#include "common.h"
#include <algorithm>
#include "gemm.h"

namespace bh {
namespace {

// absmax over the whole activation tensor, one workgroup
__global__ void __launch_bounds__(1024)
w8a8_quantize_kernel(const float *__restrict__ x, int64_t n, int M, int K, int Kp,
                     int8_t *__restrict__ xq, float *__restrict__ scale_out) {
  __shared__ float red[16];
  __shared__ float s_inv;
  float m = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += 1024)
    m = fmaxf(m, fabsf(x[i]));
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0)
    red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = red[0];
    for (int w = 1; w < 16; ++w)
      t = fmaxf(t, red[w]);
    const float r127 = 1.0f / 127.0f;
    float s = t * r127;
    s = fmaxf(s, 1e-10f);
    *scale_out = s;
    s_inv = 1.0f / s;
  }
  __syncthreads();
  const float inv = s_inv;
  // rows are padded to Kp (a multiple of 64) with zeros
  for (int64_t i = threadIdx.x; i < (int64_t)M * Kp; i += 1024) {
    const int m_ = (int)(i / Kp), k = (int)(i % Kp);
    float r = 0.f;
    if (k < K) {
      r = rintf(x[(int64_t)m_ * K + k] * inv);
      r = fminf(fmaxf(r, -128.0f), 127.0f);
    }
    xq[i] = (int8_t)r;
  }
}

constexpr int kMaxParts = 1024; // workgroups of the partial-maximum launch

// stage 1 of the quantisation of many rows: workgroup g leaves the largest
// magnitude of its share of the tensor in part[g]
__global__ void __launch_bounds__(256)
w8a8_absmax_parts_kernel(const float *__restrict__ x, int64_t n, float *__restrict__ part) {
  __shared__ float red[4];
  float m = 0.f;
  const int64_t stride = (int64_t)gridDim.x * 256, first = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) { // 16 bytes per load, the tail one by one
    const int64_t n4 = n / 4;
    for (int64_t i = first; i < n4; i += stride) {
      const float4 v = reinterpret_cast<const float4 *>(x)[i];
      m = fmaxf(fmaxf(m, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w)));
    }
    for (int64_t i = 4 * n4 + first; i < n; i += stride)
      m = fmaxf(m, fabsf(x[i]));
  } else {
    for (int64_t i = first; i < n; i += stride)
      m = fmaxf(m, fabsf(x[i]));
  }
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0)
    red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0)
    part[blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// stage 2: workgroup `row` writes row `row` of the plane ([Mp][Kp], zeros past M
// and K) and its step, the activation scale (1 for padding rows)
__global__ void __launch_bounds__(256)
w8a8_rows_to_plane_kernel(const float *__restrict__ x, int M, int K, int Kp,
                          const float *__restrict__ part, int parts,
                          int8_t *__restrict__ plane, float *__restrict__ steps,
                          float *__restrict__ scale_out) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  float m = 0.f;
  for (int i = threadIdx.x; i < parts; i += 256)
    m = fmaxf(m, part[i]);
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0)
    red[threadIdx.x >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float r127 = 1.0f / 127.0f;
  const float s = fmaxf(m * r127, 1e-10f);
  const float inv = 1.0f / s;
  if (threadIdx.x == 0) {
    steps[row] = row < M ? s : 1.0f;
    if (row == 0)
      *scale_out = s;
  }
  const float *xr = x + (int64_t)row * K;
  for (int k0 = threadIdx.x * 4; k0 < Kp; k0 += 256 * 4) {
    unsigned word = 0;
    if (row < M) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float r = 0.f;
        if (k0 + e < K) {
          r = rintf(xr[k0 + e] * inv);
          r = fminf(fmaxf(r, -128.0f), 127.0f);
        }
        word |= ((unsigned)(int)r & 0xffu) << (8 * e);
      }
    }
    *reinterpret_cast<unsigned *>(plane + (size_t)row * Kp + k0) = word;
  }
}

template <int M>
__global__ void __launch_bounds__(256)
w8a8_gemv_kernel(const int4 *__restrict__ W, const int8_t *__restrict__ xq,
                 const float *__restrict__ a_scale, const float *__restrict__ wscale,
                 float *__restrict__ C, int32_t *__restrict__ acc_out, int rows,
                 int N, int groups, int chunks, int Kp) {
  // 4 wavefronts split the k range of one channel group
  __shared__ int red[4][M][16];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int g = blockIdx.x;
  const int per = (chunks + 3) / 4;
  const int t0 = min(wave * per, chunks), t1 = min(t0 + per, chunks);
  // the two scales of the result: asked for with the first loads, not at the
  // very end of the launch behind the meeting of the wavefronts
  const float comb = *a_scale * wscale[min(g * 16 + (lane & 15), N - 1)];
  int acc[M];
#pragma unroll
  for (int m = 0; m < M; ++m)
    acc[m] = 0;
  const int4 *w = W + ((size_t)g * chunks) * 64 + lane;
  const int kg = lane >> 4;
  for (int t = t0; t < t1; ++t) {
    const int4 wv = w[(size_t)t * 64];
#pragma unroll
    for (int m = 0; m < M; ++m) {
      if (m < rows) {
        const int4 xv = *reinterpret_cast<const int4 *>(xq + (size_t)m * Kp + t * 64 + kg * 16);
        int a = acc[m];
        a = __builtin_amdgcn_sdot4(wv.x, xv.x, a, false);
        a = __builtin_amdgcn_sdot4(wv.y, xv.y, a, false);
        a = __builtin_amdgcn_sdot4(wv.z, xv.z, a, false);
        a = __builtin_amdgcn_sdot4(wv.w, xv.w, a, false);
        acc[m] = a;
      }
    }
  }
#pragma unroll
  for (int m = 0; m < M; ++m) {
    acc[m] += __shfl_xor(acc[m], 16, 64);
    acc[m] += __shfl_xor(acc[m], 32, 64);
  }
  if (lane < 16) {
#pragma unroll
    for (int m = 0; m < M; ++m)
      red[wave][m][lane] = acc[m];
  }
  __syncthreads();
  if (wave == 0 && lane < 16) {
    const int n = g * 16 + lane;
    if (n < N) {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        if (m < rows) {
          const int tot = red[0][m][lane] + red[1][m][lane] + red[2][m][lane] + red[3][m][lane];
          if (acc_out)
            acc_out[(size_t)m * N + n] = tot;
          C[(size_t)m * N + n] = (float)tot * comb;
        }
      }
    }
  }
}

} // namespace
} // namespace bh

extern "C" {

size_t buddy_hip_w8a8_workspace_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0)
    return 0;
  if (M <= 16)
    return (size_t)(M * bh::round_up(K, 64)) + 64;
  // the plane with its row steps, the partial maxima, the scale
  const bh::GemmStagingLayout l = bh::gemm_staging_layout(M, K);
  return l.bytes_digits(1) + sizeof(float) * (bh::kMaxParts + 16);
}

int buddy_hip_w8a8_matmul(const float *A, const int8_t *packed, const float *wscale,
                          float *C, int32_t *acc_out, int64_t M, int64_t K,
                          int64_t N, void *workspace, size_t workspace_bytes,
                          buddy_hip_stream stream) try {
  BH_REQUIRE(A && packed && wscale && C && workspace, "w8a8_matmul: null pointer");
  BH_REQUIRE(M >= 1 && M < (1 << 24), "w8a8_matmul: M=%lld outside 1..2^24", (long long)M);
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30), "w8a8_matmul: bad shape");
  BH_REQUIRE(workspace_bytes >= buddy_hip_w8a8_workspace_bytes(M, K),
             "w8a8_matmul: workspace of %zu bytes needed, %zu given",
             buddy_hip_w8a8_workspace_bytes(M, K), workspace_bytes);
  BH_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(packed) & 15) == 0,
             "w8a8_matmul: workspace and weights must be 16-byte aligned");
  hipStream_t st = bh::as_stream(stream);
  if (M > 16) {
    BH_REQUIRE(K <= (1 << 17), "w8a8_matmul: K=%lld above 131072 with more than 16 rows",
               (long long)K);
    const bh::GemmStagingLayout l = bh::gemm_staging_layout(M, K);
    int8_t *plane = static_cast<int8_t *>(workspace);
    float *steps = reinterpret_cast<float *>(plane + (size_t)l.rows_padded * l.cols_padded);
    float *part = steps + l.rows_padded, *scale = part + bh::kMaxParts;
    const int parts = (int)std::min<int64_t>(bh::kMaxParts, bh::ceil_div(M * K, 4096)); // 16 values per thread at least
    hipLaunchKernelGGL(bh::w8a8_absmax_parts_kernel, dim3(parts), dim3(256), 0, st, A, M * K,
                       part);
    hipLaunchKernelGGL(bh::w8a8_rows_to_plane_kernel, dim3(l.rows_padded), dim3(256), 0, st, A,
                       (int)M, (int)K, l.cols_padded, part, parts, plane, steps, scale);
    BH_CHECK_HIP(hipGetLastError());
    return bh::launch_gemm_w8a8_plane(plane, packed, wscale, C, acc_out, M, K, N, st);
  }
  const int Kp = (int)bh::round_up(K, 64);
  int8_t *xq = static_cast<int8_t *>(workspace);
  float *scale = reinterpret_cast<float *>(xq + (size_t)M * Kp);
  // the scale slot must be 4-byte aligned: M*Kp is a multiple of 64
  hipLaunchKernelGGL(bh::w8a8_quantize_kernel, dim3(1), dim3(1024), 0, st, A, M * K,
                     (int)M, (int)K, Kp, xq, scale);
  const int groups = (int)bh::ceil_div(N, 16), chunks = Kp / 64;
  const int4 *W = reinterpret_cast<const int4 *>(packed);
#define BH_W8A8(MT)                                                            \
  hipLaunchKernelGGL(bh::w8a8_gemv_kernel<MT>, dim3(groups), dim3(256), 0, st, W, \
                     xq, scale, wscale, C, acc_out, (int)M, (int)N, groups,    \
                     chunks, Kp)
  if (M == 1)
    BH_W8A8(1);
  else if (M <= 4)
    BH_W8A8(4);
  else
    BH_W8A8(16);
#undef BH_W8A8
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_w8a8_matmul")
}
