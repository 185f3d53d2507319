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
                            int8_t *packed, buddy_hip_stream stream) {
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
}

int buddy_hip_pack_w8(const int8_t *W, int64_t K, int64_t N, int8_t *packed,
                      buddy_hip_stream stream) {
  return buddy_hip_pack_w8_tiles(W, K, N, bh::kTileN, packed, stream);
}

int buddy_hip_unpack_w8_tiles(const int8_t *packed, int64_t K, int64_t N,
                              int tile_n, int8_t *W, buddy_hip_stream stream) {
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
}

int buddy_hip_unpack_w8(const int8_t *packed, int64_t K, int64_t N, int8_t *W,
                        buddy_hip_stream stream) {
  return buddy_hip_unpack_w8_tiles(packed, K, N, bh::kTileN, W, stream);
}

static int quantize_per_channel(const float *W, int64_t K, int64_t N, int8_t *q,
                                float *scale, float qmax, float lo, float hi,
                                buddy_hip_stream stream) {
  BH_REQUIRE(W && q && scale, "quantize: null pointer");
  BH_REQUIRE(K > 0 && N > 0, "quantize: bad shape K=%lld N=%lld",
             (long long)K, (long long)N);
  hipStream_t st = bh::as_stream(stream);
  BH_CHECK_HIP(hipMemsetAsync(scale, 0, sizeof(float) * (size_t)N, st));
  const int64_t rows = 64;
  hipLaunchKernelGGL(bh::colwise_absmax_kernel,
                     dim3((unsigned)bh::ceil_div(N, 256),
                          (unsigned)bh::ceil_div(K, rows)),
                     dim3(256), 0, st, W, K, N, rows,
                     reinterpret_cast<unsigned *>(scale));
  hipLaunchKernelGGL(bh::finalize_scale_kernel,
                     dim3((unsigned)bh::ceil_div(N, 256)), dim3(256), 0, st,
                     scale, N, qmax);
  hipLaunchKernelGGL(bh::quantize_kernel,
                     dim3((unsigned)bh::ceil_div(K * N, 256)), dim3(256), 0, st,
                     W, scale, K, N, q, lo, hi);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int buddy_hip_quantize_w8(const float *W, int64_t K, int64_t N, int8_t *q,
                          float *scale, buddy_hip_stream stream) {
  return quantize_per_channel(W, K, N, q, scale, 127.0f, -128.0f, 127.0f, stream);
}

int buddy_hip_quantize_w4(const float *W, int64_t K, int64_t N, int8_t *q,
                          float *scale, buddy_hip_stream stream) {
  return quantize_per_channel(W, K, N, q, scale, 7.0f, -8.0f, 7.0f, stream);
}
}
