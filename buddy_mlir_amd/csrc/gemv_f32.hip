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
// B is row-major with N contiguous.  A sum over k must stay inside a workgroup
// (no cross-workgroup reduction: it would cost an L2 write-back), so a workgroup
// owns a strip of columns and all of K.  The q|k|v shape is narrow for this chip
// (2048 columns): there a strip is 16 columns -- one 64-byte piece of every row,
// 128 workgroups -- and a wavefront load reads 16 rows x 64 bytes (4 lanes of
// float4 per row).  From 4096 columns on the strip is 32 columns, from 8192 on 64
// (256-byte pieces, 4 rows per load): longer pieces of a row per request are worth
// more than more workgroups once there are 128 of them (29.9 -> 15.5 us at
// 1536 x 8960).  The 8 wavefronts take interleaved row blocks, all their loads in
// flight at once, and meet in LDS in a fixed order.
// RMSNorm can be fused in like in the int8 kernel: the norm weight multiplies x
// as it is used, the sum of squares is gathered on the way (by the lanes of
// column group 0 only, so every k counts once) and the rsqrt factor multiplies
// the finished sums.
#include "common.h"

namespace bh {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 load_stream4(const float *p) {
  const v4f v = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}

// Sum over the lanes S, 2 S, ... 32 apart (S a power of two: lanes that are equal
// modulo S stay apart): DPP inside a row of 16 lanes, lane swaps across rows, no
// trip through LDS.
template <int S> __device__ __forceinline__ float sum_lanes_apart(float v) {
  static_assert(S == 2 || S == 4 || S == 8 || S == 16, "2, 4, 8 or 16 lanes apart");
  if (S <= 2)
    v += dpp_f<0x4E>(v);  // quad_perm [2,3,0,1]: lane ^ 2
  if (S <= 4)
    v += dpp_f<0x124>(v); // row_ror:4: lanes 4, 8, 12 further on ...
  if (S <= 8)
    v += dpp_f<0x128>(v); // ... with row_ror:8
  return sum_rows(v);
}

constexpr int kWaves = 8;
constexpr int kUnroll = 12;        // loads in flight per lane         // loads in flight per lane

// kCols = columns per workgroup: 16 (64-byte pieces of a row, the most workgroups)
// for narrow matrices, 32 or 64 (longer pieces, fewer and larger requests per row)
// once that still gives every compute unit a workgroup.
template <int kCols>
__global__ void __launch_bounds__(kWaves * 64)
gemv_f32_kernel(const float *__restrict__ x, const float *__restrict__ B,
                const float *__restrict__ bias, const float *__restrict__ norm_w,
                float norm_eps, float norm_inv_k, float *__restrict__ y, int K, int N,
                int64_t ldb, int64_t block_stride, int accumulate) {
  // block_stride != 0: the columns of workgroup b are a matrix of their own, kCols
  // wide, at B + b * block_stride (the reference's panel-packed layout)
  __shared__ float red[kWaves][kCols + 1];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int kLanesPerRow = kCols / 4;        // float4 lanes across a row piece
  constexpr int kRowsPerLoad = 64 / kLanesPerRow; // rows per wavefront load
  const int c4 = lane % kLanesPerRow, rsub = lane / kLanesPerRow;
  const int col = blockIdx.x * kCols + c4 * 4;
  const int bcol = block_stride ? c4 * 4 : col;
  B += (int64_t)blockIdx.x * block_stride;
  const bool full = blockIdx.x * kCols + kCols <= N && ((ldb & 3) == 0) &&
                    ((reinterpret_cast<uintptr_t>(B) & 15) == 0);
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  float ss = 0.f;
  // row blocks wave, wave + kWaves, ... of kRowsPerLoad rows each, kUnroll at a time
  for (int kb = wave * kRowsPerLoad; kb < K; kb += kWaves * kRowsPerLoad * kUnroll) {
    float4 b[kUnroll];
    float xv[kUnroll], nw[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int k = kb + u * kWaves * kRowsPerLoad + rsub;
      const int kc = min(k, K - 1); // rows past the end repeat the last, times zero
      const float *row = B + (int64_t)kc * ldb + bcol;
      if (full)
        b[u] = load_stream4(row); // read once per launch: past the caches
      else
        b[u] = make_float4(col < N ? row[0] : 0.f, col + 1 < N ? row[1] : 0.f,
                           col + 2 < N ? row[2] : 0.f, col + 3 < N ? row[3] : 0.f);
      xv[u] = k < K ? x[kc] : 0.f;
      nw[u] = norm_w ? norm_w[kc] : 1.f;
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (norm_w && c4 == 0)
        ss = fmaf(xv[u], xv[u], ss);
      const float xs = xv[u] * nw[u];
      acc.x = fmaf(xs, b[u].x, acc.x);
      acc.y = fmaf(xs, b[u].y, acc.y);
      acc.z = fmaf(xs, b[u].z, acc.z);
      acc.w = fmaf(xs, b[u].w, acc.w);
    }
  }
  // the row lanes of a column group hold different k: lanes kLanesPerRow apart ... 32 apart
  acc.x = sum_lanes_apart<kLanesPerRow>(acc.x);
  acc.y = sum_lanes_apart<kLanesPerRow>(acc.y);
  acc.z = sum_lanes_apart<kLanesPerRow>(acc.z);
  acc.w = sum_lanes_apart<kLanesPerRow>(acc.w);
  ss = sum_lanes_apart<kLanesPerRow>(ss);
  if (lane < kLanesPerRow) {
    red[wave][lane * 4 + 0] = acc.x;
    red[wave][lane * 4 + 1] = acc.y;
    red[wave][lane * 4 + 2] = acc.z;
    red[wave][lane * 4 + 3] = acc.w;
    if (lane == 0)
      red[wave][kCols] = ss;
  }
  __syncthreads();
  if (tid < kCols) {
    float s = 0.f, sq = 0.f;
    for (int w = 0; w < kWaves; ++w) {
      s += red[w][tid];
      sq += red[w][kCols];
    }
    const int n = blockIdx.x * kCols + tid;
    if (n < N) {
      float v = s;
      if (norm_w) // x' = w (.) (x * r): r is common to the row
        v *= 1.0f / sqrtf(sq * norm_inv_k + norm_eps);
      if (bias)
        v = bias[n] + v; // tosa.add(bias, matmul)
      y[n] = accumulate ? y[n] + v : v;
    }
  }
}

// ---- the same product over 1 KiB tiles --------------------------------------
// A device-side re-layout for matrices the library owns (the model path's f32
// q|k|v weights): tile = 32 rows x 8 columns, row-major inside, tiles of one
// 8-column strip contiguous along k, zero padded:
//   T[((n/8) * ceil(K/32) + k/32) * 256 + (k%32) * 8 + n%8] = B[k, n].
// A wavefront load is one whole tile (lane = float4: row lane/2, half lane%2), a
// workgroup streams one contiguous strip, and a 2048-column matrix gives 256
// workgroups instead of 128 with 64-byte pieces of 8 KB-apart rows.
constexpr int kTileCols = 8, kTileRows = 32, kTileUnroll = 6;

__global__ void __launch_bounds__(256)
tile_f32_kernel(const float *__restrict__ B, int K, int N, int64_t ldb,
                float *__restrict__ T, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total)
    return;
  const int blocks = (K + kTileRows - 1) / kTileRows;
  const int c = (int)(i & 7), r = (int)((i >> 3) & 31);
  const int64_t tile = i >> 8;
  const int64_t k = (tile % blocks) * kTileRows + r, n = (tile / blocks) * kTileCols + c;
  T[i] = (k < K && n < N) ? B[k * ldb + n] : 0.f;
}

__global__ void __launch_bounds__(kWaves * 64)
gemv_f32_tiles_kernel(const float *__restrict__ x, const float *__restrict__ T,
                      const float *__restrict__ bias, const float *__restrict__ norm_w,
                      float norm_eps, float norm_inv_k, float *__restrict__ y, int K,
                      int N, int accumulate) {
  __shared__ float red[kWaves][kTileCols + 1];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane & 1, row = lane >> 1;
  const int blocks = (K + kTileRows - 1) / kTileRows;
  const float4 *strip = reinterpret_cast<const float4 *>(T) +
                        (int64_t)blockIdx.x * blocks * 64 + lane;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  float ss = 0.f;
  for (int b0 = wave; b0 < blocks; b0 += kWaves * kTileUnroll) {
    float4 b[kTileUnroll];
    float xv[kTileUnroll], nw[kTileUnroll];
#pragma unroll
    for (int u = 0; u < kTileUnroll; ++u) {
      const int blk = b0 + u * kWaves;
      const int bc = min(blk, blocks - 1); // past the end: the last tile again, x = 0
      b[u] = load_stream4(reinterpret_cast<const float *>(strip + (int64_t)bc * 64));
      const int k = blk * kTileRows + row;
      const int kc = min(k, K - 1);
      xv[u] = (blk < blocks && k < K) ? x[kc] : 0.f;
      nw[u] = norm_w ? norm_w[kc] : 1.f;
    }
#pragma unroll
    for (int u = 0; u < kTileUnroll; ++u) {
      if (norm_w && half == 0)
        ss = fmaf(xv[u], xv[u], ss);
      const float xs = xv[u] * nw[u];
      acc.x = fmaf(xs, b[u].x, acc.x);
      acc.y = fmaf(xs, b[u].y, acc.y);
      acc.z = fmaf(xs, b[u].z, acc.z);
      acc.w = fmaf(xs, b[u].w, acc.w);
    }
  }
  acc.x = sum_lanes_apart<2>(acc.x);
  acc.y = sum_lanes_apart<2>(acc.y);
  acc.z = sum_lanes_apart<2>(acc.z);
  acc.w = sum_lanes_apart<2>(acc.w);
  ss = sum_lanes_apart<2>(ss);
  if (lane < 2) {
    red[wave][lane * 4 + 0] = acc.x;
    red[wave][lane * 4 + 1] = acc.y;
    red[wave][lane * 4 + 2] = acc.z;
    red[wave][lane * 4 + 3] = acc.w;
    if (lane == 0)
      red[wave][kTileCols] = ss;
  }
  __syncthreads();
  if (tid < kTileCols) {
    float s = 0.f, sq = 0.f;
    for (int w = 0; w < kWaves; ++w) {
      s += red[w][tid];
      sq += red[w][kTileCols];
    }
    const int n = blockIdx.x * kTileCols + tid;
    if (n < N) {
      float v = s;
      if (norm_w)
        v *= 1.0f / sqrtf(sq * norm_inv_k + norm_eps);
      if (bias)
        v = bias[n] + v;
      y[n] = accumulate ? y[n] + v : v;
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

int launch_gemv_f32_norm(const float *x, const float *B, const float *bias,
                         const float *norm_w, float norm_eps, float *y, int64_t K,
                         int64_t N, int64_t ldb, bool accumulate, hipStream_t stream) {
  BH_REQUIRE(x && B && y, "gemv_f32: null pointer");
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30) && ldb >= N,
             "gemv_f32: bad shape K=%lld N=%lld ldb=%lld", (long long)K,
             (long long)N, (long long)ldb);
  const int cols = N >= 64 * 128 ? 64 : N >= 32 * 128 ? 32 : 16;
#define BH_LAUNCH_F32(C)                                                                  \
  hipLaunchKernelGGL(gemv_f32_kernel<C>, dim3((unsigned)ceil_div(N, C)), dim3(kWaves * 64), \
                     0, stream, x, B, bias, norm_w, norm_eps, 1.0f / (float)K, y, (int)K,  \
                     (int)N, ldb, (int64_t)0, accumulate ? 1 : 0)
  if (cols == 64)
    BH_LAUNCH_F32(64);
  else if (cols == 32)
    BH_LAUNCH_F32(32);
  else
    BH_LAUNCH_F32(16);
#undef BH_LAUNCH_F32
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_gemv_f32_panels32(const float *x, const float *packed, float *y, int64_t K,
                             int64_t N, bool accumulate, hipStream_t stream) {
  BH_REQUIRE(x && packed && y, "gemv_f32_panels: null pointer");
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30) && N % 32 == 0,
             "gemv_f32_panels: K=%lld N=%lld (N must be a multiple of 32)", (long long)K,
             (long long)N);
  hipLaunchKernelGGL(gemv_f32_kernel<32>, dim3((unsigned)(N / 32)), dim3(kWaves * 64), 0,
                     stream, x, packed, (const float *)nullptr, (const float *)nullptr, 0.f,
                     1.0f / (float)K, y, (int)K, (int)N, (int64_t)32, K * 32,
                     accumulate ? 1 : 0);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_gemv_f32(const float *x, const float *B, const float *bias, float *y,
                    int64_t K, int64_t N, int64_t ldb, bool accumulate,
                    hipStream_t stream) {
  return launch_gemv_f32_norm(x, B, bias, nullptr, 0.f, y, K, N, ldb, accumulate, stream);
}

int64_t f32_tiles_elems(int64_t K, int64_t N) {
  return round_up(K, kTileRows) * round_up(N, kTileCols);
}

int launch_tile_f32(const float *B, int64_t K, int64_t N, int64_t ldb, float *T,
                    hipStream_t stream) {
  BH_REQUIRE(B && T, "tile_f32: null pointer");
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30) && ldb >= N,
             "tile_f32: bad shape K=%lld N=%lld ldb=%lld", (long long)K, (long long)N,
             (long long)ldb);
  const int64_t total = f32_tiles_elems(K, N);
  hipLaunchKernelGGL(tile_f32_kernel, dim3((unsigned)ceil_div(total, 256)), dim3(256), 0,
                     stream, B, (int)K, (int)N, ldb, T, total);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_gemv_f32_tiles(const float *x, const float *T, const float *bias,
                          const float *norm_w, float norm_eps, float *y, int64_t K,
                          int64_t N, bool accumulate, hipStream_t stream) {
  BH_REQUIRE(x && T && y, "gemv_f32_tiles: null pointer");
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30),
             "gemv_f32_tiles: bad shape K=%lld N=%lld", (long long)K, (long long)N);
  BH_REQUIRE((reinterpret_cast<uintptr_t>(T) & 15) == 0,
             "gemv_f32_tiles: tiles must be 16-byte aligned");
  hipLaunchKernelGGL(gemv_f32_tiles_kernel, dim3((unsigned)ceil_div(N, kTileCols)),
                     dim3(kWaves * 64), 0, stream, x, T, bias, norm_w, norm_eps,
                     1.0f / (float)K, y, (int)K, (int)N, accumulate ? 1 : 0);
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
                       buddy_hip_stream stream) try {
  return bh::launch_gemv_f32(x, B, bias, y, K, N, N,
                             (flags & BUDDY_HIP_GEMV_ACCUMULATE) != 0,
                             bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_gemv_f32")
}

extern "C" {
size_t buddy_hip_f32_tiles_bytes(int64_t K, int64_t N) {
  if (K <= 0 || N <= 0)
    return 0;
  return (size_t)bh::f32_tiles_elems(K, N) * sizeof(float);
}

int buddy_hip_tile_f32(const float *B, int64_t K, int64_t N, float *tiles,
                       buddy_hip_stream stream) try {
  return bh::launch_tile_f32(B, K, N, N, tiles, bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_tile_f32")

int buddy_hip_gemv_f32_tiles(const float *x, const float *tiles, const float *bias,
                             const float *norm_w, float norm_eps, float *y, int64_t K,
                             int64_t N, unsigned flags, buddy_hip_stream stream) try {
  return bh::launch_gemv_f32_tiles(x, tiles, bias, norm_w, norm_eps, y, K, N,
                                   (flags & BUDDY_HIP_GEMV_ACCUMULATE) != 0,
                                   bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_gemv_f32_tiles")
}
