// quant_pack.hip -- device-side per-channel int8 quantizer and the wave-tile
// weight layout (pack / unpack).
//
// Quantizer: tools/buddy-codegen/import_model.py:837-848,874-880.
// Layout: replaces frontend/Python/graph/transform/pack_decode_weights.py:102-108.
#include "common.h"

namespace bh {
namespace {

// |W| column maximum.  Non-negative IEEE floats order like their bit patterns,
// so the maximum is taken with an integer atomicMax: order-independent, hence
// deterministic.
__global__ void __launch_bounds__(256)
colwise_absmax_kernel(const float *__restrict__ W, int64_t K, int64_t N,
                      int64_t rows_per_block, unsigned *__restrict__ amax_bits) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N)
    return;
  const int64_t k0 = (int64_t)blockIdx.y * rows_per_block;
  const int64_t k1 = k0 + rows_per_block < K ? k0 + rows_per_block : K;
  float m = 0.0f;
  for (int64_t k = k0; k < k1; ++k)
    m = fmaxf(m, fabsf(W[k * N + n]));
  atomicMax(&amax_bits[n], __float_as_uint(m));
}

// The same for four adjacent columns per thread (N a multiple of 4, W 16-byte
// aligned): 16-byte loads, four times the bytes in flight.
__global__ void __launch_bounds__(256)
colwise_absmax4_kernel(const float *__restrict__ W, int64_t K, int64_t N,
                       int64_t rows_per_block, unsigned *__restrict__ amax_bits) {
  const int64_t n = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (n >= N)
    return;
  const int64_t k0 = (int64_t)blockIdx.y * rows_per_block;
  const int64_t k1 = k0 + rows_per_block < K ? k0 + rows_per_block : K;
  float m0 = 0.f, m1 = 0.f, m2 = 0.f, m3 = 0.f;
  const float *p = W + k0 * N + n;
  int64_t k = k0;
  for (; k + 4 <= k1; k += 4, p += 4 * N) { // four rows requested together
    const float4 a = *reinterpret_cast<const float4 *>(p);
    const float4 b = *reinterpret_cast<const float4 *>(p + N);
    const float4 c = *reinterpret_cast<const float4 *>(p + 2 * N);
    const float4 d = *reinterpret_cast<const float4 *>(p + 3 * N);
    m0 = fmaxf(fmaxf(m0, fabsf(a.x)), fmaxf(fabsf(b.x), fmaxf(fabsf(c.x), fabsf(d.x))));
    m1 = fmaxf(fmaxf(m1, fabsf(a.y)), fmaxf(fabsf(b.y), fmaxf(fabsf(c.y), fabsf(d.y))));
    m2 = fmaxf(fmaxf(m2, fabsf(a.z)), fmaxf(fabsf(b.z), fmaxf(fabsf(c.z), fabsf(d.z))));
    m3 = fmaxf(fmaxf(m3, fabsf(a.w)), fmaxf(fabsf(b.w), fmaxf(fabsf(c.w), fabsf(d.w))));
  }
  for (; k < k1; ++k, p += N) {
    const float4 a = *reinterpret_cast<const float4 *>(p);
    m0 = fmaxf(m0, fabsf(a.x));
    m1 = fmaxf(m1, fabsf(a.y));
    m2 = fmaxf(m2, fabsf(a.z));
    m3 = fmaxf(m3, fabsf(a.w));
  }
  atomicMax(&amax_bits[n], __float_as_uint(m0));
  atomicMax(&amax_bits[n + 1], __float_as_uint(m1));
  atomicMax(&amax_bits[n + 2], __float_as_uint(m2));
  atomicMax(&amax_bits[n + 3], __float_as_uint(m3));
}

// scale = (amax / 127).clamp(min=1e-10)      (import_model.py:838,875)
__global__ void __launch_bounds__(256)
finalize_scale_kernel(float *__restrict__ scale, int64_t N, float qmax) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N)
    return;
  float s = scale[n] / qmax;
  scale[n] = s < 1e-10f ? 1e-10f : s;
}

// q = clamp(round(W / scale), -128, 127).to(int8)   (import_model.py:845-847)
// torch.round is round-half-to-even = rintf; the f32 division is IEEE
// (hipcc rounds divisions correctly by default).
__global__ void __launch_bounds__(256)
quantize_kernel(const float *__restrict__ W, const float *__restrict__ scale,
                int64_t K, int64_t N, int8_t *__restrict__ q, float lo,
                float hi) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= K * N)
    return;
  const int64_t n = i % N;
  float r = rintf(W[i] / scale[n]);
  r = fminf(fmaxf(r, lo), hi);
  q[i] = (int8_t)r;
}

// The same for four adjacent elements of a row per thread (N a multiple of 4, W
// 16-byte and q 4-byte aligned); blockIdx.y is the row.
__global__ void __launch_bounds__(256)
quantize4_kernel(const float *__restrict__ W, const float *__restrict__ scale, int64_t N,
                 int8_t *__restrict__ q, float lo, float hi) {
  const int64_t n = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (n >= N)
    return;
  const int64_t row = blockIdx.y;
  const float4 w = *reinterpret_cast<const float4 *>(W + row * N + n);
  const float4 s = *reinterpret_cast<const float4 *>(scale + n);
  const float r0 = fminf(fmaxf(rintf(w.x / s.x), lo), hi);
  const float r1 = fminf(fmaxf(rintf(w.y / s.y), lo), hi);
  const float r2 = fminf(fmaxf(rintf(w.z / s.z), lo), hi);
  const float r3 = fminf(fmaxf(rintf(w.w / s.w), lo), hi);
  char4 out;
  out.x = (signed char)r0;
  out.y = (signed char)r1;
  out.z = (signed char)r2;
  out.w = (signed char)r3;
  *reinterpret_cast<char4 *>(q + row * N + n) = out;
}

// One thread writes one lane's 16 bytes of one tile.
__global__ void __launch_bounds__(256)
pack_w8_kernel(const int8_t *__restrict__ W, int64_t K, int64_t N,
               int64_t chunks, int64_t total_lanes, int tn,
               int8_t *__restrict__ P) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total_lanes)
    return;
  const int lane = (int)(t & 63);
  const int64_t tile = t >> 6;
  const int64_t c = tile % chunks, g = tile / chunks;
  const int64_t n = g * tn + (lane % tn);
  const int64_t kb = c * (1024 / tn) + (lane / tn) * 16;
  union {
    int8_t b[16];
    int4 v;
  } u;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int64_t k = kb + j;
    u.b[j] = (n < N && k < K) ? W[k * N + n] : (int8_t)0;
  }
  reinterpret_cast<int4 *>(P)[t] = u.v;
}

__global__ void __launch_bounds__(256)
unpack_w8_kernel(const int8_t *__restrict__ P, int64_t K, int64_t N,
                 int64_t chunks, int tn, int8_t *__restrict__ W) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= K * N)
    return;
  const int64_t k = i / N, n = i % N;
  const int tk = 1024 / tn;
  const int64_t g = n / tn, c = k / tk;
  const int lane = (int)(((k % tk) / 16) * tn + (n % tn));
  W[i] = P[((g * chunks + c) * 64 + lane) * 16 + (k % 16)];
}

} // namespace
} // namespace bh

extern "C" {

static bool valid_tile_n(int tn) { return tn == 16 || tn == 8 || tn == 4; }

size_t buddy_hip_w8_packed_bytes_tiles(int64_t K, int64_t N, int tile_n) {
  if (K <= 0 || N <= 0 || !valid_tile_n(tile_n))
    return 0;
  return (size_t)(bh::round_up(K, 1024 / tile_n) * bh::round_up(N, tile_n));
}

size_t buddy_hip_w8_packed_bytes(int64_t K, int64_t N) {
  return buddy_hip_w8_packed_bytes_tiles(K, N, bh::kTileN);
}

int buddy_hip_pack_w8_tiles(const int8_t *W, int64_t K, int64_t N, int tile_n,
                            int8_t *packed, buddy_hip_stream stream) try {
  BH_REQUIRE(W && packed, "pack_w8: null pointer");
  BH_REQUIRE(K > 0 && N > 0, "pack_w8: bad shape K=%lld N=%lld", (long long)K,
             (long long)N);
  BH_REQUIRE(valid_tile_n(tile_n), "pack_w8: tile_n=%d (16, 8 or 4)", tile_n);
  const int64_t chunks = bh::ceil_div(K, 1024 / tile_n);
  const int64_t groups = bh::ceil_div(N, tile_n);
  const int64_t lanes = groups * chunks * 64;
  hipLaunchKernelGGL(bh::pack_w8_kernel, dim3((unsigned)bh::ceil_div(lanes, 256)),
                     dim3(256), 0, bh::as_stream(stream), W, K, N, chunks,
                     lanes, tile_n, packed);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_pack_w8_tiles")

int buddy_hip_pack_w8(const int8_t *W, int64_t K, int64_t N, int8_t *packed,
                      buddy_hip_stream stream) try {
  return buddy_hip_pack_w8_tiles(W, K, N, bh::kTileN, packed, stream);
} BH_CATCH_INT("buddy_hip_pack_w8")

int buddy_hip_unpack_w8_tiles(const int8_t *packed, int64_t K, int64_t N,
                              int tile_n, int8_t *W, buddy_hip_stream stream) try {
  BH_REQUIRE(W && packed, "unpack_w8: null pointer");
  BH_REQUIRE(K > 0 && N > 0, "unpack_w8: bad shape K=%lld N=%lld", (long long)K,
             (long long)N);
  BH_REQUIRE(valid_tile_n(tile_n), "unpack_w8: tile_n=%d (16, 8 or 4)", tile_n);
  const int64_t chunks = bh::ceil_div(K, 1024 / tile_n);
  hipLaunchKernelGGL(bh::unpack_w8_kernel,
                     dim3((unsigned)bh::ceil_div(K * N, 256)), dim3(256), 0,
                     bh::as_stream(stream), packed, K, N, chunks, tile_n, W);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_unpack_w8_tiles")

int buddy_hip_unpack_w8(const int8_t *packed, int64_t K, int64_t N, int8_t *W,
                        buddy_hip_stream stream) try {
  return buddy_hip_unpack_w8_tiles(packed, K, N, bh::kTileN, W, stream);
} BH_CATCH_INT("buddy_hip_unpack_w8")

static int quantize_per_channel(const float *W, int64_t K, int64_t N, int8_t *q,
                                float *scale, float qmax, float lo, float hi,
                                buddy_hip_stream stream) {
  BH_REQUIRE(W && q && scale, "quantize: null pointer");
  BH_REQUIRE(K > 0 && N > 0, "quantize: bad shape K=%lld N=%lld",
             (long long)K, (long long)N);
  hipStream_t st = bh::as_stream(stream);
  BH_CHECK_HIP(hipMemsetAsync(scale, 0, sizeof(float) * (size_t)N, st));
  const int64_t rows = 64;
  // four columns per thread where rows can be read as aligned 16-byte pieces
  const bool vec = N % 4 == 0 && K <= 65535 &&
                   ((reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(scale)) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(q) & 3) == 0;
  if (vec) {
    hipLaunchKernelGGL(bh::colwise_absmax4_kernel,
                       dim3((unsigned)bh::ceil_div(N / 4, 256), (unsigned)bh::ceil_div(K, rows)),
                       dim3(256), 0, st, W, K, N, rows, reinterpret_cast<unsigned *>(scale));
  } else {
    hipLaunchKernelGGL(bh::colwise_absmax_kernel,
                       dim3((unsigned)bh::ceil_div(N, 256), (unsigned)bh::ceil_div(K, rows)),
                       dim3(256), 0, st, W, K, N, rows, reinterpret_cast<unsigned *>(scale));
  }
  hipLaunchKernelGGL(bh::finalize_scale_kernel,
                     dim3((unsigned)bh::ceil_div(N, 256)), dim3(256), 0, st,
                     scale, N, qmax);
  if (vec) {
    hipLaunchKernelGGL(bh::quantize4_kernel,
                       dim3((unsigned)bh::ceil_div(N / 4, 256), (unsigned)K), dim3(256), 0, st, W,
                       scale, N, q, lo, hi);
  } else {
    hipLaunchKernelGGL(bh::quantize_kernel,
                       dim3((unsigned)bh::ceil_div(K * N, 256)), dim3(256), 0, st,
                       W, scale, K, N, q, lo, hi);
  }
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int buddy_hip_quantize_w8(const float *W, int64_t K, int64_t N, int8_t *q,
                          float *scale, buddy_hip_stream stream) try {
  return quantize_per_channel(W, K, N, q, scale, 127.0f, -128.0f, 127.0f, stream);
} BH_CATCH_INT("buddy_hip_quantize_w8")

int buddy_hip_quantize_w4(const float *W, int64_t K, int64_t N, int8_t *q,
                          float *scale, buddy_hip_stream stream) try {
  return quantize_per_channel(W, K, N, q, scale, 7.0f, -8.0f, 7.0f, stream);
} BH_CATCH_INT("buddy_hip_quantize_w4")
}
