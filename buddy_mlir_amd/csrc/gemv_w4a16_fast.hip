// gemv_w4a16_fast.hip -- the int4 weight-only decode GEMV (W4A16) as a streaming
// kernel: C[n] = f16(f32(C[n]) + (sum_k a[k] * w[k][n]) * scale[n]).
//
// Same operands as the kernel of gemv_w4a16.hip (the one that
// midend/lib/Conversion/MatMulOptimization/Int4DequantMatMulVectorizationDecode.cpp
// :385-468 generates: f16 activations, scales and C, int4 weights), another
// summation: the reference adds in f16, k in order, and loses about sqrt(K) * 2^-11
// of the sum's magnitude on the way; that chain of K dependent roundings is what
// the bit-exact kernel spends its time on.  Here the products are exact and the
// sum is exact up to one rounding of each activation to 2^-31 of the largest of
// its run, so the result is at least as close to the real-number sum as the
// reference's own, and the launch is bound by the bytes it reads (half a byte
// per weight).  It cannot equal the reference bit for bit and is opt-in.
//
// Weights come in "int4 wave tiles" (pack_w4_tiles below): 16 channels x 128 k
// in 1 KiB, lane L of a wavefront owning 16 bytes whose low nibbles are
// k = 128 c + 16 (L / 16) + 0..15 of channel 16 g + L % 16 and whose high
// nibbles are the same k + 64.  (x << 4) & 0xf0f0f0f0 and x & 0xf0f0f0f0 turn a
// lane's four dwords into two A operands of v_mfma_i32_16x16x64_i8 holding
// 16 w (a nibble in the top half of a byte is the signed value times 16): three
// VALU instructions per 32 weights, and the factor 1/16 goes into the step.
// The activations are cut into four int8 digit planes per wavefront run exactly
// as in gemv_w8a32.hip's one-row kernel and are the B operand.
#include "common.h"

#include <algorithm>

namespace bh {
namespace {

typedef unsigned short u16;
typedef int v4i32 __attribute__((ext_vector_type(4)));

constexpr int kW4TileK = 128;     // k per int4 tile (two matrix instructions)
constexpr int kFastMaxWaves = 16; // wavefronts per workgroup
constexpr int kPlaneBytes = 4 * kTileK; // four digit planes of 64 k

__device__ __forceinline__ float h2f(u16 h) {
  union {
    u16 u;
    _Float16 f;
  } x;
  x.u = h;
  return (float)x.f;
}
__device__ __forceinline__ u16 f2h(float v) {
  union {
    u16 u;
    _Float16 f;
  } x;
  x.f = (_Float16)v;
  return x.u;
}

struct FastArgs {
  const u16 *A;      // [K] f16 bits
  const int4 *W;     // int4 wave tiles
  const u16 *scale;  // [N]
  u16 *C;            // [N]
  int K, N, groups, chunks; // channel groups of 16, tiles of 128 k per group
  int G, KS;         // channel groups x k-slices = wavefronts of a workgroup
};

// U: int4 tiles a wavefront multiplies per round (a run longer than U tiles
// takes several rounds, each with its own step).
// The arguments are four pointers and six integers, 14 words that the command
// processor preloads into SGPRs (this file is built with
// -amdgpu-kernarg-preload-count=14), so that a wavefront's first loads do not
// wait for a read of the argument block.
template <int U>
__global__ void __launch_bounds__(kFastMaxWaves *kWave)
    w4a16_fast_kernel(const u16 *pA, const int4 *pW, const u16 *pscale, u16 *pC, int pK, int pN,
                      int pgroups, int pchunks, int pG, int pKS) {
  FastArgs a;
  a.A = pA, a.W = pW, a.scale = pscale, a.C = pC;
  a.K = pK, a.N = pN, a.groups = pgroups, a.chunks = pchunks, a.G = pG, a.KS = pKS;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int nwaves = a.G * a.KS;
  const int ksh = shift_of(a.KS);
  const int gl = wave >> ksh, ks = wave & (a.KS - 1);
  const int g = blockIdx.x * a.G + gl;
  const bool live = g < a.groups;
  const int per = (a.chunks + a.KS - 1) >> ksh;
  const int t0 = min(ks * per, a.chunks), t1 = min(t0 + per, a.chunks);
  const int4 *w = a.W + ((size_t)(live ? g : 0) * a.chunks) * 64 + lane;
  const int n = g * kTileN + lane;
  const bool writer = ks == 0 && lane < kTileN && live && n < a.N;
  // requested before the stream and first looked at after it (a conversion
  // here would make the wavefront wait out two cold loads before it asks for
  // its weights)
  unsigned scale_bits = 0, c_bits = 0;
  if (writer) {
    scale_bits = a.scale[n];
    c_bits = a.C[n];
  }
  // planes of four 64-k tiles (two int4 tiles) at a time, private to the wavefront
  // (first in LDS: they are read 16 bytes at a time and must stay 16-byte aligned
  // whatever the number of wavefronts; the meeting place of the k-slices follows)
  unsigned char *planes = reinterpret_cast<unsigned char *>(lds) + (size_t)wave * (4 * kPlaneBytes);
  float *meet = lds + (size_t)nwaves * (4 * kPlaneBytes / sizeof(float));
  const int col = lane & 15, kq = lane >> 4;
  const unsigned char *my_b = planes + min(col, 3) * kTileK + 16 * kq;
  constexpr int XV = (U + 1) / 2; // groups of 256 k
  auto lds_turn = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  float sum[4] = {0.f, 0.f, 0.f, 0.f};
  for (int r0 = t0; r0 < t1; r0 += U) {
    const int r1 = min(r0 + U, t1);
    // activations of the round: a lane takes four consecutive k per group
    // (8 aligned bytes that start inside the row)
    float x[XV][4];
    const int klast = max(min((a.K + 3) & ~3, r1 * kW4TileK) - 4, 0);
#pragma unroll
    for (int q = 0; q < XV; ++q) {
      const int kc = min(r0 * kW4TileK + q * 256 + 4 * lane, klast);
      const uint2 v = *reinterpret_cast<const uint2 *>(a.A + kc);
      x[q][0] = h2f((u16)(v.x & 0xffffu));
      x[q][1] = h2f((u16)(v.x >> 16));
      x[q][2] = h2f((u16)(v.y & 0xffffu));
      x[q][3] = h2f((u16)(v.y >> 16));
    }
    int4 wt[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const v4i32 v = __builtin_nontemporal_load(
          reinterpret_cast<const v4i32 *>(w + (size_t)min(r0 + u, r1 - 1) * 64));
      wt[u] = make_int4(v.x, v.y, v.z, v.w);
    }
    unsigned mb = 0;
#pragma unroll
    for (int q = 0; q < XV; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int k = r0 * kW4TileK + q * 256 + 4 * lane + e;
        const bool in = k < r1 * kW4TileK && k < a.K;
        x[q][e] = in ? x[q][e] : 0.f;
        mb = max(mb, __float_as_uint(x[q][e]) & 0x7fffffffu);
      }
    mb = wave_max_u32(mb);
    const int ex = (int)(mb >> 23) - 127;
    const int e2 = max(ex + 1 - 30, -126);
    const bool finite = mb < 0x7f800000u;
    const float step = finite ? __uint_as_float((unsigned)(e2 + 127) << 23)
                              : __uint_as_float(0x7fc00000u);
    const float inv = __uint_as_float((unsigned)(127 - e2) << 23);
    auto cut_group = [&](int q) {
      unsigned y[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = (int)__builtin_rintf(x[q][e] * inv); // exact: |.| < 2^30
        y[e] = (unsigned)r + 0x00808080u;
      }
      const unsigned ta = __builtin_amdgcn_perm(y[1], y[0], 0x05010400u);
      const unsigned tb = __builtin_amdgcn_perm(y[3], y[2], 0x05010400u);
      const unsigned tc = __builtin_amdgcn_perm(y[1], y[0], 0x07030602u);
      const unsigned td = __builtin_amdgcn_perm(y[3], y[2], 0x07030602u);
      const unsigned d0 = __builtin_amdgcn_perm(tb, ta, 0x05040100u) ^ 0x80808080u;
      const unsigned d1 = __builtin_amdgcn_perm(tb, ta, 0x07060302u) ^ 0x80808080u;
      const unsigned d2 = __builtin_amdgcn_perm(td, tc, 0x05040100u) ^ 0x80808080u;
      const unsigned d3 = __builtin_amdgcn_perm(td, tc, 0x07060302u);
      unsigned *p = reinterpret_cast<unsigned *>(planes + (lane >> 4) * kPlaneBytes) + (lane & 15);
      p[0] = d0;
      p[kTileK / 4] = d1;
      p[2 * kTileK / 4] = d2;
      p[3 * kTileK / 4] = d3;
    };
    v4i32 acc = {0, 0, 0, 0}, acc_hi = {0, 0, 0, 0}; // two chains of dependent instructions
    lds_turn(); // the reads of the round before are over
    cut_group(0);
#pragma unroll
    for (int q = 0; q < XV; ++q) {
      lds_turn();
      v4i32 b[4];
#pragma unroll
      for (int t = 0; t < 4; ++t)
        b[t] = *reinterpret_cast<const v4i32 *>(my_b + t * kPlaneBytes);
      if (q + 1 < XV) {
        lds_turn();
        cut_group(q + 1);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int u = 2 * q + j;
        if (u < U) {
          if (r0 + u < r1) {
            const int4 t = wt[u < U ? u : 0];
            const v4i32 lo = {(int)(((unsigned)t.x << 4) & 0xf0f0f0f0u),
                              (int)(((unsigned)t.y << 4) & 0xf0f0f0f0u),
                              (int)(((unsigned)t.z << 4) & 0xf0f0f0f0u),
                              (int)(((unsigned)t.w << 4) & 0xf0f0f0f0u)};
            const v4i32 hi = {(int)((unsigned)t.x & 0xf0f0f0f0u), (int)((unsigned)t.y & 0xf0f0f0f0u),
                              (int)((unsigned)t.z & 0xf0f0f0f0u), (int)((unsigned)t.w & 0xf0f0f0f0u)};
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(lo, b[2 * j], acc, 0, 0, 0);
            acc_hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(hi, b[2 * j + 1], acc_hi, 0, 0, 0);
          }
        }
      }
    }
    // lane (kq, col): channels 4 kq + i for digit col; 16 w was multiplied
    float colscale = step * 0.0625f;
    colscale = col == 1 ? colscale * 256.0f : colscale;
    colscale = col == 2 ? colscale * 65536.0f : colscale;
    colscale = col == 3 ? colscale * 16777216.0f : colscale;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float v = (float)(acc[i] + acc_hi[i]) * colscale; // below 2^26 each
      sum[i] += (v + dpp_f<0x101>(v)) + (dpp_f<0x102>(v) + dpp_f<0x103>(v));
    }
  }
  // the k-slices meet in LDS in slice order: [wave][channel]
  float *mine = meet + (size_t)wave * 17;
  if (col == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      mine[4 * kq + i] = sum[i];
  }
  if (a.KS > 1) {
    __syncthreads();
    if (ks != 0)
      return;
  } else {
    lds_turn();
  }
  // (the empty asm keeps the compiler from converting, and so waiting for, the
  // two values where they were loaded)
  asm volatile("" : "+v"(scale_bits), "+v"(c_bits));
  if (writer) {
    float r = 0.f;
    for (int s = 0; s < a.KS; ++s)
      r += meet[(size_t)(wave + s) * 17 + lane];
    a.C[n] = f2h(fmaf(r, h2f((u16)scale_bits), h2f((u16)c_bits)));
  }
}

// reference layout [K, N/2] (low nibble = even channel) -> int4 wave tiles; one
// thread per output byte
__global__ void __launch_bounds__(256)
pack_w4_tiles_kernel(const int8_t *__restrict__ packed, int K, int N, int chunks,
                     int64_t total, int8_t *__restrict__ tiles) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total)
    return;
  const int b = (int)(i & 15), L = (int)((i >> 4) & 63);
  const int64_t tile = i >> 10;
  const int c = (int)(tile % chunks), g = (int)(tile / chunks);
  const int n = g * kTileN + (L & 15);
  const int k_lo = c * kW4TileK + (L >> 4) * 16 + b, k_hi = k_lo + 64;
  auto nibble = [&](int k) -> unsigned {
    if (k >= K || n >= N)
      return 0u;
    const unsigned byte = (unsigned char)packed[(int64_t)k * (N / 2) + n / 2];
    return (n & 1) ? byte >> 4 : byte & 0x0Fu;
  };
  tiles[i] = (int8_t)(nibble(k_lo) | (nibble(k_hi) << 4));
}

template <int U> int launch_fast(const FastArgs &a, unsigned blocks, size_t lds, hipStream_t s) {
  BH_REQUIRE(is_pow2(a.KS), "w4a16: %d k-slices (the kernel shifts by their count)", a.KS);
  hipLaunchKernelGGL(w4a16_fast_kernel<U>, dim3(blocks), dim3(a.G * a.KS * kWave), lds, s, a.A,
                     a.W, a.scale, a.C, a.K, a.N, a.groups, a.chunks, a.G, a.KS);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace
} // namespace bh

extern "C" {

size_t buddy_hip_w4_tiles_bytes(int64_t K, int64_t N) {
  if (K <= 0 || N <= 0)
    return 0;
  return (size_t)bh::ceil_div(N, bh::kTileN) * (size_t)bh::ceil_div(K, bh::kW4TileK) * 1024;
}

int buddy_hip_pack_w4_tiles(const int8_t *packed, int64_t K, int64_t N, int8_t *tiles,
                            buddy_hip_stream stream) try {
  BH_REQUIRE(packed && tiles, "pack_w4_tiles: null pointer");
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30) && N % 2 == 0,
             "pack_w4_tiles: bad shape K=%lld N=%lld (N even)", (long long)K, (long long)N);
  const int64_t total = (int64_t)buddy_hip_w4_tiles_bytes(K, N);
  hipLaunchKernelGGL(bh::pack_w4_tiles_kernel, dim3((unsigned)bh::ceil_div(total, 256)),
                     dim3(256), 0, bh::as_stream(stream), packed, (int)K, (int)N,
                     (int)bh::ceil_div(K, bh::kW4TileK), total, tiles);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_pack_w4_tiles")

int buddy_hip_gemv_w4a16_fast(const uint16_t *A, const int8_t *tiles, const uint16_t *scale,
                              uint16_t *C, int64_t K, int64_t N, buddy_hip_stream stream) try {
  BH_REQUIRE(A && tiles && scale && C, "gemv_w4a16_fast: null pointer");
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30),
             "gemv_w4a16_fast: bad shape K=%lld N=%lld", (long long)K, (long long)N);
  BH_REQUIRE((reinterpret_cast<uintptr_t>(A) & 7) == 0 &&
                 (reinterpret_cast<uintptr_t>(tiles) & 15) == 0,
             "gemv_w4a16_fast: A must be 8-byte and the tiles 16-byte aligned");
  bh::FastArgs a;
  a.A = A;
  a.W = reinterpret_cast<const int4 *>(tiles);
  a.scale = scale;
  a.C = C;
  a.K = (int)K;
  a.N = (int)N;
  a.groups = (int)bh::ceil_div(N, bh::kTileN);
  a.chunks = (int)bh::ceil_div(K, bh::kW4TileK);
  // k-slices per channel group: the most (a power of two up to 16) that still
  // leave a wavefront three tiles (3 KiB in flight per wavefront, what the int8
  // kernel's launches settled on), fewer tiles only where the launch would
  // otherwise have under ~2000 wavefronts; a workgroup has at least four
  // wavefronts.  Measured at 1536 -> 8960, 4096 -> 4096 and 8960 -> 1536: every
  // cut between 2 and 6 tiles per wavefront is within 0.1 us of the best.
  a.KS = 1;
  for (int ks = bh::kFastMaxWaves; ks > 1; ks /= 2) {
    if (ks > a.chunks)
      continue;
    const bool three_tiles = bh::ceil_div(a.chunks, ks) >= 3;
    if (three_tiles || (int64_t)a.groups * ks < 2048) {
      a.KS = ks;
      break;
    }
  }
  const int U = (int)std::min<int64_t>(bh::ceil_div(a.chunks, a.KS), 8); // longer runs take rounds
  a.G = a.KS < 4 ? 4 / a.KS : 1;
  const unsigned blocks = (unsigned)bh::ceil_div(a.groups, a.G);
  const int waves = a.G * a.KS;
  const size_t lds = sizeof(float) * waves * 17 + (size_t)waves * 4 * bh::kPlaneBytes;
  hipStream_t s = bh::as_stream(stream);
  switch (U) {
  case 1: return bh::launch_fast<1>(a, blocks, lds, s);
  case 2: return bh::launch_fast<2>(a, blocks, lds, s);
  case 3: return bh::launch_fast<3>(a, blocks, lds, s);
  case 4: return bh::launch_fast<4>(a, blocks, lds, s);
  case 5: return bh::launch_fast<5>(a, blocks, lds, s);
  case 6: return bh::launch_fast<6>(a, blocks, lds, s);
  case 7: return bh::launch_fast<7>(a, blocks, lds, s);
  default: return bh::launch_fast<8>(a, blocks, lds, s);
  }
} BH_CATCH_INT("buddy_hip_gemv_w4a16_fast")
}
