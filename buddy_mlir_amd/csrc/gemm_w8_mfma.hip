// gemm_w8_mfma.hip -- prefill matmul: C[M,N] (+)= A[M,K] . (int8 W[K,N] * scale)
// on the bf16 matrix cores.
//
// Replaces the BLIS-style kernel with dequantisation fused into B packing that
// midend/lib/Conversion/MatMulOptimization/MatMulBlisVectorization.cpp:351-360,
// 398-986 generates for M > 1.
//
// Shape of the kernel:
//  * the weights are read from the same wave-tile packed copy the decode GEMV
//    streams (one resident copy serves prefill and decode).  A lane's 16 bytes
//    of a 16 x 64 tile are, as they lie, two 8-wide operand fragments of
//    v_mfma_f32_16x16x32_bf16 (rows = the tile's 16 channels): they go from
//    global memory to registers, are converted to bf16 (|q| <= 128 is exact)
//    and fed to the matrix core.  No LDS on the way;
//  * the activations are converted once per call to bf16 terms (one term =
//    "activations cast to bf16"; three terms carry all 24 significand bits of
//    the f32 input) in a [term][row][k] buffer.  A lane's fragment of the other
//    operand (columns = 16 activation rows) is 32 contiguous bytes of that
//    buffer, so it is loaded straight from L2 as well;
//  * a wavefront owns 64 rows x 64 channels of C (4 x 4 accumulators); the four
//    wavefronts of a workgroup split K and meet in LDS, in slice order;
//  * workgroup ids are laid out so that the row blocks of one column tile run
//    on the same XCD (ids equal modulo 8) and share the weight tiles in its L2;
//  * the per-channel scale is applied once to the f32 accumulators, where the
//    reference multiplies every element before the FMA.
#include "gemm.h"

#include <algorithm>
#include <map>
#include <mutex>

namespace bh {
namespace {

constexpr int kRowsPerWave = 64;   // 4 row blocks of 16
constexpr int kGroupsPerWave = 4;  // 4 channel groups of 16
constexpr int kSlices = 4;         // k-slices = wavefronts per workgroup

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16;

__device__ __forceinline__ u16 bf16_rne(float x) {
  unsigned u = __float_as_uint(x);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (u16)(u >> 16);
}
__device__ __forceinline__ float bf16_to_f32(u16 b) {
  return __uint_as_float((unsigned)b << 16);
}
__device__ __forceinline__ unsigned pack2(u16 lo, u16 hi) {
  return (unsigned)lo | ((unsigned)hi << 16);
}
// two int8 (bytes j, j+1 of v) -> two exact bf16
__device__ __forceinline__ unsigned q2_to_bf16x2(int v, int j) {
  const float a = (float)(signed char)(v >> (8 * j));
  const float b = (float)(signed char)(v >> (8 * j + 8));
  return (__float_as_uint(a) >> 16) | (__float_as_uint(b) & 0xffff0000u);
}
__device__ __forceinline__ bf16x8 frag_from(int lo, int hi) {
  union {
    uint4 u;
    bf16x8 v;
  } x;
  x.u = make_uint4(q2_to_bf16x2(lo, 0), q2_to_bf16x2(lo, 2), q2_to_bf16x2(hi, 0),
                   q2_to_bf16x2(hi, 2));
  return x.v;
}
__device__ __forceinline__ bf16x8 as_frag(const uint4 &u) {
  union {
    uint4 u;
    bf16x8 v;
  } x;
  x.u = u;
  return x.v;
}

// A[M, K] f32 -> terms x [Mp, Kp] bf16, zero padded; term t holds the bf16
// rounding of what the terms before it left over.
__global__ void __launch_bounds__(256)
activations_to_bf16(const float *__restrict__ A, int64_t lda, int M, int K, int Mp,
                    int Kp, int terms, u16 *__restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; // 8 k per thread
  const int kq = Kp / 8;
  if (i >= (int64_t)Mp * kq)
    return;
  const int m = (int)(i / kq), k0 = (int)(i % kq) * 8;
  float r[8];
#pragma unroll
  for (int e = 0; e < 8; ++e)
    r[e] = (m < M && k0 + e < K) ? A[(int64_t)m * lda + k0 + e] : 0.f;
  for (int t = 0; t < terms; ++t) {
    u16 h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      h[e] = bf16_rne(r[e]);
      r[e] -= bf16_to_f32(h[e]);
    }
    *reinterpret_cast<uint4 *>(out + ((size_t)t * Mp + m) * Kp + k0) =
        make_uint4(pack2(h[0], h[1]), pack2(h[2], h[3]), pack2(h[4], h[5]),
                   pack2(h[6], h[7]));
  }
}

// 8 consecutive values of a row -> `terms` bf16 terms in the staging layout
__device__ __forceinline__ void store_terms(float (&r)[8], int terms, u16 *out,
                                            size_t term_stride) {
  for (int t = 0; t < terms; ++t) {
    u16 h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      h[e] = bf16_rne(r[e]);
      r[e] -= bf16_to_f32(h[e]);
    }
    *reinterpret_cast<uint4 *>(out + t * term_stride) =
        make_uint4(pack2(h[0], h[1]), pack2(h[2], h[3]), pack2(h[4], h[5]),
                   pack2(h[6], h[7]));
  }
}

// One workgroup per row: y = w * (x * rsqrt(sum(x^2) / n + eps)) -> staging
__global__ void __launch_bounds__(256)
rmsnorm_to_staging_kernel(const float *__restrict__ x, const float *__restrict__ w, int n,
                          float inv_n, float eps, int terms, int Mp, int Kp,
                          u16 *__restrict__ out) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  const float *xr = x + (size_t)row * n;
  float s = 0.f;
  for (int i = threadIdx.x; i < n; i += 256)
    s = fmaf(xr[i], xr[i], s);
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0)
    red[threadIdx.x >> 6] = s;
  __syncthreads();
  const float tot = (red[0] + red[1]) + (red[2] + red[3]);
  const float rs = 1.0f / sqrtf(tot * inv_n + eps);
  for (int k0 = threadIdx.x * 8; k0 < Kp; k0 += 256 * 8) {
    float r[8];
#pragma unroll
    for (int e = 0; e < 8; ++e)
      r[e] = k0 + e < n ? w[k0 + e] * (xr[k0 + e] * rs) : 0.f;
    store_terms(r, terms, out + (size_t)row * Kp + k0, (size_t)Mp * Kp);
  }
}

__global__ void __launch_bounds__(256)
silu_mul_to_staging_kernel(const float *__restrict__ g, const float *__restrict__ u,
                           int64_t ld, int rows, int n, int terms, int Mp, int Kp,
                           u16 *__restrict__ out) {
  const int kq = Kp / 8;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)rows * kq)
    return;
  const int row = (int)(i / kq), k0 = (int)(i % kq) * 8;
  float r[8], gv[8], uv[8];
  const float *gr = g + (size_t)row * ld + k0, *ur = u + (size_t)row * ld + k0;
  if (k0 + 7 < n && ((reinterpret_cast<uintptr_t>(gr) | reinterpret_cast<uintptr_t>(ur)) & 15) == 0) {
    const float4 g0 = *reinterpret_cast<const float4 *>(gr), g1 = *reinterpret_cast<const float4 *>(gr + 4);
    const float4 u0 = *reinterpret_cast<const float4 *>(ur), u1 = *reinterpret_cast<const float4 *>(ur + 4);
    gv[0] = g0.x; gv[1] = g0.y; gv[2] = g0.z; gv[3] = g0.w;
    gv[4] = g1.x; gv[5] = g1.y; gv[6] = g1.z; gv[7] = g1.w;
    uv[0] = u0.x; uv[1] = u0.y; uv[2] = u0.z; uv[3] = u0.w;
    uv[4] = u1.x; uv[5] = u1.y; uv[6] = u1.z; uv[7] = u1.w;
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      gv[e] = k0 + e < n ? gr[e] : 0.f;
      uv[e] = k0 + e < n ? ur[e] : 0.f;
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float sig = 1.0f / (1.0f + expf(-gv[e]));
    r[e] = k0 + e < n ? (gv[e] * sig) * uv[e] : 0.f;
  }
  store_terms(r, terms, out + (size_t)row * Kp + k0, (size_t)Mp * Kp);
}

struct GemmArgs {
  const u16 *Abf; // [terms][Mp][Kp]
  const int4 *W;
  const float *scale;
  const float *bias;
  float *C;
  int64_t ldc;
  int M, N, Mp, Kp, groups, chunks;
  int ncols, cols_padded; // column tiles of 64 channels; padded to the XCD count
  int accumulate;
};

template <int TERMS> struct ChunkOperands {
  int4 w[kGroupsPerWave];
  uint4 a[TERMS][4][2]; // [term][row block][k half]
};

template <int TERMS>
__device__ __forceinline__ void load_chunk(const int4 *const (&wp)[kGroupsPerWave],
                                           const u16 *ap, size_t term_stride,
                                           size_t rb_stride, int c,
                                           ChunkOperands<TERMS> &o) {
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g)
    o.w[g] = wp[g][(size_t)c * 64];
#pragma unroll
  for (int t = 0; t < TERMS; ++t)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
      const uint4 *src = reinterpret_cast<const uint4 *>(
          ap + t * term_stride + rb * rb_stride + (size_t)c * kTileK);
      o.a[t][rb][0] = src[0];
      o.a[t][rb][1] = src[1];
    }
}

template <int TERMS>
__global__ void __launch_bounds__(kSlices *kWave) gemm_w8_bf16_kernel(GemmArgs a) {
  extern __shared__ __attribute__((aligned(16))) float red[]; // [slice][64][lane]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = blockIdx.x % a.cols_padded, rbk = blockIdx.x / a.cols_padded;
  if (col >= a.ncols)
    return; // padding id
  const int m0 = rbk * kRowsPerWave, g0 = col * kGroupsPerWave;
  const int per = (a.chunks + kSlices - 1) / kSlices;
  const int c0 = min(wave * per, a.chunks), c1 = min(c0 + per, a.chunks);

  f32x4 acc[kGroupsPerWave][4];
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
      acc[g][rb] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int4 *wp[kGroupsPerWave];
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g) // groups past the end repeat the last one
    wp[g] = a.W + ((size_t)min(g0 + g, a.groups - 1) * a.chunks) * 64 + lane;
  const size_t term_stride = (size_t)a.Mp * a.Kp, rb_stride = (size_t)16 * a.Kp;
  const u16 *ap = a.Abf + (size_t)(m0 + (lane & 15)) * a.Kp + (lane >> 4) * 16;

  ChunkOperands<TERMS> cur, nxt;
  if (c0 < c1)
    load_chunk<TERMS>(wp, ap, term_stride, rb_stride, c0, cur);
  for (int c = c0; c < c1; ++c) {
    if (c + 1 < c1)
      load_chunk<TERMS>(wp, ap, term_stride, rb_stride, c + 1, nxt);
#pragma unroll
    for (int g = 0; g < kGroupsPerWave; ++g) {
      const bf16x8 w0 = frag_from(cur.w[g].x, cur.w[g].y);
      const bf16x8 w1 = frag_from(cur.w[g].z, cur.w[g].w);
#pragma unroll
      for (int t = 0; t < TERMS; ++t)
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
          acc[g][rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              w0, as_frag(cur.a[t][rb][0]), acc[g][rb], 0, 0, 0);
          acc[g][rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              w1, as_frag(cur.a[t][rb][1]), acc[g][rb], 0, 0, 0);
        }
    }
    if (c + 1 < c1)
      cur = nxt;
  }

  // ---- the k-slices meet in LDS; wavefront w finishes channel group w ------
  float *mine = red + (size_t)wave * 64 * kWave;
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        mine[((g * 4 + rb) * 4 + r) * kWave + lane] = acc[g][rb][r];
  __syncthreads();
  const int g = wave;
  if (g0 + g >= a.groups)
    return;
  // lane holds channels n..n+3 of row m for each row block
  const int n = (g0 + g) * kTileN + (lane >> 4) * 4;
  float s[4], b[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    s[r] = n + r < a.N ? a.scale[n + r] : 0.f;
    b[r] = (a.bias && n + r < a.N) ? a.bias[n + r] : 0.f;
  }
  const bool vec = n + 3 < a.N && (a.ldc & 3) == 0 &&
                   (reinterpret_cast<uintptr_t>(a.C) & 15) == 0;
#pragma unroll
  for (int rb = 0; rb < 4; ++rb) {
    const int m = m0 + rb * 16 + (lane & 15);
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float sum = 0.f;
#pragma unroll
      for (int sl = 0; sl < kSlices; ++sl)
        sum += red[((size_t)sl * 64 + (g * 4 + rb) * 4 + r) * kWave + lane];
      v[r] = sum * s[r];
    }
    if (m >= a.M)
      continue;
    float *c = a.C + (int64_t)m * a.ldc + n;
    if (vec) {
      float4 o = make_float4(v[0], v[1], v[2], v[3]);
      if (a.accumulate) {
        const float4 p = *reinterpret_cast<const float4 *>(c);
        o = make_float4(p.x + o.x, p.y + o.y, p.z + o.z, p.w + o.w);
      } else {
        o = make_float4(b[0] + o.x, b[1] + o.y, b[2] + o.z, b[3] + o.w);
      }
      *reinterpret_cast<float4 *>(c) = o;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n + r < a.N)
          c[r] = a.accumulate ? c[r] + v[r] : b[r] + v[r];
    }
  }
}

// Wide matrices (enough column tiles to fill the chip without splitting K):
// a workgroup owns 64 rows x 256 channels, one 64-channel span per wavefront,
// every wavefront runs the whole K.  The activation fragments of a chunk are the
// same for the four wavefronts: wavefront w fetches row block w for everyone
// and leaves it in LDS in fragment order (lane l of fragment f at f*1 KiB +
// 16 l: conflict-free by construction), so the fragments cross L2 -> CU once per
// workgroup.  Weights stay on the register path.
//
// Global loads run kRing - 2 chunks ahead of the matrix cores.  The compiler
// sinks ordinary loads down to their first use (and then waits for them there),
// so the loads of this loop are issued by hand and waited for by hand: a fetch
// is kFetchLoads loads in a fixed order, vmcnt counts them in order, and each
// wait names the registers it releases so that nothing reads them earlier.
constexpr int kRing = 5;

typedef int v4i32 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void issue_load(v4i32 &dst, const void *p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
template <int TERMS> struct FetchRegs {
  v4i32 w[kGroupsPerWave];
  v4i32 a[TERMS][2];
};
// Waits until at most N loads are in flight; the registers of `f` are only
// valid after it.
template <int N, int TERMS> __device__ __forceinline__ void wait_loads(FetchRegs<TERMS> &f) {
  static_assert(kGroupsPerWave == 4, "operand list below");
  asm volatile("s_waitcnt vmcnt(%4)"
               : "+v"(f.w[0]), "+v"(f.w[1]), "+v"(f.w[2]), "+v"(f.w[3])
               : "n"(N)
               : "memory");
#pragma unroll
  for (int t = 0; t < TERMS; ++t)
    asm volatile("" : "+v"(f.a[t][0]), "+v"(f.a[t][1])::"memory");
}
__device__ __forceinline__ bf16x8 frag_from_v(int lo, int hi) { return frag_from(lo, hi); }

// RB = row blocks of 16 per workgroup (4 or 3: whichever leaves the shorter last
// round of workgroups on the chip).
template <int TERMS, int RB>
__global__ void __launch_bounds__(kSlices *kWave) gemm_w8_bf16_wide_kernel(GemmArgs a) {
  constexpr int L = kGroupsPerWave + 2 * TERMS; // loads per fetch
  extern __shared__ __attribute__((aligned(16))) v4i32 frag_s[]; // [2][TERMS][2 RB][64]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = blockIdx.x % a.cols_padded, rbk = blockIdx.x / a.cols_padded;
  if (col >= a.ncols)
    return; // padding id
  const int m0 = rbk * RB * 16;
  const int g0 = (col * kSlices + wave) * kGroupsPerWave;

  f32x4 acc[kGroupsPerWave][RB];
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
      acc[g][rb] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int4 *wp[kGroupsPerWave];
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g) // groups past the end repeat the last one
    wp[g] = a.W + ((size_t)min(g0 + g, a.groups - 1) * a.chunks) * 64 + lane;
  const size_t term_stride = (size_t)a.Mp * a.Kp;
  // this wavefront fetches row block `wave` of the activation tile (with three
  // row blocks the fourth wavefront repeats the third's loads and stages nothing)
  const int my_rb = min(wave, RB - 1);
  const u16 *ap = a.Abf + (size_t)(m0 + my_rb * 16 + (lane & 15)) * a.Kp + (lane >> 4) * 16;

  FetchRegs<TERMS> ring[kRing];
  // chunks past the end are fetched again from the last chunk (never used):
  // every fetch is exactly L loads, which is what keeps the counts below exact
  auto fetch = [&](int c, FetchRegs<TERMS> &f) {
    const int cc = min(c, a.chunks - 1);
#pragma unroll
    for (int g = 0; g < kGroupsPerWave; ++g)
      issue_load(f.w[g], wp[g] + (size_t)cc * 64);
#pragma unroll
    for (int t = 0; t < TERMS; ++t) {
      const u16 *src = ap + t * term_stride + (size_t)cc * kTileK;
      issue_load(f.a[t][0], src);
      issue_load(f.a[t][1], src + 8);
    }
  };
  auto stage = [&](const FetchRegs<TERMS> &f, int buf) { // own row block -> LDS
    if (wave >= RB)
      return;
#pragma unroll
    for (int t = 0; t < TERMS; ++t) {
      v4i32 *dst = frag_s + (((size_t)buf * TERMS + t) * 2 * RB + wave * 2) * kWave + lane;
      dst[0] = f.a[t][0];
      dst[kWave] = f.a[t][1];
    }
  };
#pragma unroll
  for (int u = 0; u < kRing; ++u)
    fetch(u, ring[u]);
  wait_loads<(kRing - 1) * L, TERMS>(ring[0]); // chunk 0 has arrived
  stage(ring[0], 0);
  __syncthreads();
  for (int c0 = 0; c0 < a.chunks; c0 += kRing) {
#pragma unroll
    for (int u = 0; u < kRing; ++u) {
      const int c = c0 + u;
      if (c < a.chunks) {
        const int buf = c & 1;
        FetchRegs<TERMS> &cur = ring[u];
        FetchRegs<TERMS> &nxt = ring[(u + 1) % kRing];
        // in flight: chunks c+1 .. c+kRing-1 (chunk c was waited for when it was
        // staged).  Release chunk c+1 and put its row block into the other
        // buffer, whose readers passed the barrier that closed chunk c-1.
        wait_loads<(kRing - 2) * L, TERMS>(nxt);
        stage(nxt, buf ^ 1);
        bf16x8 wf[kGroupsPerWave][2];
#pragma unroll
        for (int g = 0; g < kGroupsPerWave; ++g) {
          wf[g][0] = frag_from(cur.w[g].x, cur.w[g].y);
          wf[g][1] = frag_from(cur.w[g].z, cur.w[g].w);
        }
#pragma unroll
        for (int t = 0; t < TERMS; ++t)
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            const v4i32 *src = frag_s + (((size_t)buf * TERMS + t) * 2 * RB + rb * 2) * kWave + lane;
            union {
              v4i32 i;
              bf16x8 v;
            } a0, a1;
            a0.i = src[0];
            a1.i = src[kWave];
#pragma unroll
            for (int g = 0; g < kGroupsPerWave; ++g) {
              acc[g][rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[g][0], a0.v, acc[g][rb], 0, 0, 0);
              acc[g][rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[g][1], a1.v, acc[g][rb], 0, 0, 0);
            }
          }
        // the registers of chunk c are free: fetch the chunk kRing further on
        // (its weights were converted above; wf holds them now)
        fetch(c + kRing, cur);
        __syncthreads();
      }
    }
  }
  // loads of the repeated last chunk may still be in flight: the ring registers
  // stay allocated until they have landed (without these ties the compiler may
  // put a temporary of the epilogue into one of them before the wait, and the
  // late load would overwrite it)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int u = 0; u < kRing; ++u)
    wait_loads<0, TERMS>(ring[u]);

  // ---- epilogue: lane holds channels n..n+3 of row m for each row block ------
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g) {
    if (g0 + g >= a.groups)
      continue;
    const int n = (g0 + g) * kTileN + (lane >> 4) * 4;
    float s[4], b[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s[r] = n + r < a.N ? a.scale[n + r] : 0.f;
      b[r] = (a.bias && n + r < a.N) ? a.bias[n + r] : 0.f;
    }
    const bool vec = n + 3 < a.N && (a.ldc & 3) == 0 &&
                     (reinterpret_cast<uintptr_t>(a.C) & 15) == 0;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int m = m0 + rb * 16 + (lane & 15);
      if (m >= a.M)
        continue;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r)
        v[r] = acc[g][rb][r] * s[r];
      float *c = a.C + (int64_t)m * a.ldc + n;
      if (vec) {
        float4 o = make_float4(v[0], v[1], v[2], v[3]);
        if (a.accumulate) {
          const float4 p = *reinterpret_cast<const float4 *>(c);
          o = make_float4(p.x + o.x, p.y + o.y, p.z + o.z, p.w + o.w);
        } else {
          o = make_float4(b[0] + o.x, b[1] + o.y, b[2] + o.z, b[3] + o.w);
        }
        *reinterpret_cast<float4 *>(c) = o;
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < a.N)
            c[r] = a.accumulate ? c[r] + v[r] : b[r] + v[r];
      }
    }
  }
}

// bf16 staging of the activations: one grow-only device buffer per stream, so
// that calls on different streams do not share it.  Calls on one stream are
// ordered, and the buffer is only read by the matmul that follows the
// conversion on that stream.
struct Staging {
  u16 *ptr = nullptr;
  size_t bytes = 0;
  // what the buffer holds
  const float *src = nullptr;
  int64_t lda = 0;
  int M = 0, K = 0, terms = 0;
};
std::mutex g_staging_mutex;
std::map<hipStream_t, Staging> g_staging;

// what the staged copy holds: bf16 terms (1..3) or digit planes (16 + digits)
int precision_key(const GemmW8Args &in) { return in.digits ? 16 + in.digits : in.terms; }

int staging_for(hipStream_t stream, size_t bytes, const GemmW8Args &in, u16 **out,
                bool *holds_input) {
  std::lock_guard<std::mutex> lock(g_staging_mutex);
  Staging &s = g_staging[stream];
  *holds_input = in.reuse_staged_a && s.ptr && s.src == in.A && s.lda == in.lda &&
                 s.M == (int)in.M && s.K == (int)in.K && s.terms == precision_key(in);
  s.src = in.A;
  s.lda = in.lda;
  s.M = (int)in.M;
  s.K = (int)in.K;
  s.terms = precision_key(in);
  if (s.bytes < bytes) {
    if (s.ptr) {
      BH_CHECK_HIP(hipStreamSynchronize(stream)); // an earlier matmul may still read it
      BH_CHECK_HIP(hipFree(s.ptr));
      s.ptr = nullptr;
      s.bytes = 0;
    }
    BH_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&s.ptr), bytes));
    s.bytes = bytes;
  }
  *out = s.ptr;
  return BUDDY_HIP_OK;
}

BH_VARIANT_FAMILY(WideFamily, "gemm_w8_bf16_wide_kernel");
BH_VARIANT_FAMILY(SplitFamily, "gemm_w8_bf16_kernel");

template <int TERMS, int RB>
int launch_wide(const GemmArgs &a, unsigned blocks, hipStream_t stream) {
  constexpr size_t lds = sizeof(v4i32) * 2 * TERMS * 2 * RB * kWave;
  BH_NOTE_VARIANT(WideFamily, TERMS, RB);
  hipLaunchKernelGGL((gemm_w8_bf16_wide_kernel<TERMS, RB>), dim3(blocks),
                     dim3(kSlices * kWave), lds, stream, a);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

template <int TERMS>
int launch_terms(const GemmArgs &a, unsigned blocks, hipStream_t stream) {
  constexpr size_t lds = sizeof(float) * kSlices * 64 * kWave;
  auto kernel = gemm_w8_bf16_kernel<TERMS>;
  static DynLdsOnce dyn_lds;
  BH_CHECK_HIP(ensure_dyn_lds(dyn_lds, reinterpret_cast<const void *>(kernel),
                              (int)lds));
  BH_NOTE_VARIANT(SplitFamily, TERMS);
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kSlices * kWave), lds, stream, a);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace

GemmStagingLayout gemm_staging_layout(int64_t M, int64_t K) {
  GemmStagingLayout l;
  // padded rows cover the last 64-row block and the last 48-row block
  l.rows_padded = (int)std::max(round_up(M, 64), round_up(M, 48));
  l.cols_padded = (int)round_up(K, kTileK);
  return l;
}

int launch_rmsnorm_to_staging(const float *x, const float *w, int rows, int n, float eps,
                              int terms, unsigned short *staged, hipStream_t stream) {
  BH_REQUIRE(x && w && staged && rows > 0 && n > 0 && terms >= 1 && terms <= 3,
             "rmsnorm_to_staging: bad argument");
  const GemmStagingLayout l = gemm_staging_layout(rows, n);
  hipLaunchKernelGGL(rmsnorm_to_staging_kernel, dim3(rows), dim3(256), 0, stream, x, w, n,
                     1.0f / (float)n, eps, terms, l.rows_padded, l.cols_padded, staged);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_silu_mul_to_staging(const float *g, const float *u, int64_t ld, int rows, int n, int terms,
                               unsigned short *staged, hipStream_t stream) {
  BH_REQUIRE(g && u && staged && rows > 0 && n > 0 && terms >= 1 && terms <= 3,
             "silu_mul_to_staging: bad argument");
  const GemmStagingLayout l = gemm_staging_layout(rows, n);
  const int64_t threads = (int64_t)rows * (l.cols_padded / 8);
  hipLaunchKernelGGL(silu_mul_to_staging_kernel, dim3((unsigned)ceil_div(threads, 256)),
                     dim3(256), 0, stream, g, u, ld, rows, n, terms, l.rows_padded,
                     l.cols_padded, staged);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_gemm_w8(const GemmW8Args &in, hipStream_t stream) {
  BH_REQUIRE((in.A || in.staged) && in.W && in.scale && in.C, "gemm_w8: null pointer");
  BH_REQUIRE(in.M > 0 && in.K > 0 && in.N > 0 && in.M < (1 << 24) &&
                 in.K < (1 << 24) && in.N < (1 << 24),
             "gemm_w8: bad shape M=%lld K=%lld N=%lld", (long long)in.M,
             (long long)in.K, (long long)in.N);
  BH_REQUIRE((in.staged || in.lda >= in.K) && in.ldc >= (in.silu_pair ? in.N / 2 : in.N),
             "gemm_w8: row stride below row length");
  BH_REQUIRE(!in.silu_pair || in.digits, "gemm_w8: the SiLU pair runs on digit planes only");
  BH_REQUIRE(!in.then_norm_w || (in.digits && in.then_norm_staged),
             "gemm_w8: a following norm needs digit planes and a buffer for them");
  // one bf16 term (activations cast to bf16) or three (every f32 bit); three
  // digit planes (23 bits below the row's maximum) or two (15 bits: the fixed
  // point counterpart of the bf16 cast, for the same third less matrix work)
  BH_REQUIRE(in.terms == 1 || in.terms == 3, "gemm_w8: terms=%d (1 or 3)", in.terms);
  BH_REQUIRE(in.digits == 0 || in.digits == 2 || in.digits == 3,
             "gemm_w8: digits=%d (0, 2 or 3)", in.digits);
  BH_REQUIRE(in.digits == 0 || in.K <= (1 << 17),
             "gemm_w8: K=%lld beyond 2^17 would overflow the int32 sums of the digit planes",
             (long long)in.K);
  BH_REQUIRE(!(in.bias && in.accumulate), "gemm_w8: bias with accumulate");
  BH_REQUIRE((reinterpret_cast<uintptr_t>(in.W) & 15) == 0,
             "gemm_w8: packed weights must be 16-byte aligned");
  GemmArgs a;
  a.W = reinterpret_cast<const int4 *>(in.W);
  a.scale = in.scale;
  a.bias = in.bias;
  a.C = in.C;
  a.ldc = in.ldc;
  a.M = (int)in.M;
  a.N = (int)in.N;
  a.groups = (int)ceil_div(in.N, kTileN);
  a.chunks = (int)ceil_div(in.K, kTileK);
  const GemmStagingLayout layout = gemm_staging_layout(in.M, in.K);
  a.Mp = layout.rows_padded;
  a.Kp = layout.cols_padded;
  a.ncols = (int)ceil_div(a.groups, kGroupsPerWave);
  a.cols_padded = (int)round_up(a.ncols, 8);
  a.accumulate = in.accumulate ? 1 : 0;
  u16 *abf = static_cast<u16 *>(const_cast<void *>(in.staged));
  bool staged = in.staged != nullptr;
  const size_t staging_bytes =
      in.digits ? layout.bytes_digits(in.digits) : layout.bytes(in.terms);
  int rc = staged ? BUDDY_HIP_OK : staging_for(stream, staging_bytes, in, &abf, &staged);
  if (rc)
    return rc;
  if (in.digits) {
    if (!staged &&
        (rc = launch_activations_to_digits(in.A, in.lda, in.M, in.K, in.digits, abf, stream)))
      return rc;
    return launch_gemm_w8_digits(in, abf, stream);
  }
  a.Abf = abf;
  if (!staged) {
    const int64_t threads = (int64_t)a.Mp * (a.Kp / 8);
    hipLaunchKernelGGL(activations_to_bf16, dim3((unsigned)ceil_div(threads, 256)),
                       dim3(256), 0, stream, in.A, in.lda, a.M, (int)in.K, a.Mp, a.Kp,
                       in.terms, abf);
    BH_CHECK_HIP(hipGetLastError());
  }
  // wide matrices: a workgroup per 64 rows x 256 channels, no split of K
  const int wide_cols = (int)ceil_div(a.groups, kGroupsPerWave * kSlices);
  if ((int64_t)wide_cols * (a.Mp / kRowsPerWave) >= 200) {
    // 64 or 48 rows per workgroup: the chip runs 256 workgroups at a time (one
    // wavefront per SIMD), so the time is rounds x rows; ties go to 64 rows,
    // which convert each weight tile fewer times
    const int64_t wg4 = wide_cols * ceil_div(in.M, 64), wg3 = wide_cols * ceil_div(in.M, 48);
    const bool three = ceil_div(wg3, 256) * 3 < ceil_div(wg4, 256) * 4;
    const int rows = three ? 48 : 64;
    a.ncols = wide_cols;
    a.cols_padded = (int)round_up(wide_cols, 8);
    const unsigned wb = (unsigned)(a.cols_padded * ceil_div(in.M, rows));
    if (three)
      return in.terms == 1 ? launch_wide<1, 3>(a, wb, stream) : launch_wide<3, 3>(a, wb, stream);
    return in.terms == 1 ? launch_wide<1, 4>(a, wb, stream) : launch_wide<3, 4>(a, wb, stream);
  }
  const unsigned blocks = (unsigned)(a.cols_padded * (a.Mp / kRowsPerWave));
  return in.terms == 1 ? launch_terms<1>(a, blocks, stream) : launch_terms<3>(a, blocks, stream);
}

void release_gemm_staging(hipStream_t stream) {
  release_gemm_i8_workspace(stream);
  std::lock_guard<std::mutex> lock(g_staging_mutex);
  auto it = g_staging.find(stream);
  if (it == g_staging.end())
    return;
  if (it->second.ptr) {
    (void)hipStreamSynchronize(stream);
    (void)hipFree(it->second.ptr);
  }
  g_staging.erase(it);
}

} // namespace bh

extern "C" {

int buddy_hip_gemm_w8a32(const float *A, const int8_t *packed, const float *scale,
                         float *C, int64_t M, int64_t K, int64_t N,
                         unsigned flags, buddy_hip_stream stream) try {
  bh::GemmW8Args a;
  a.A = A;
  a.lda = K;
  a.W = packed;
  a.scale = scale;
  a.C = C;
  a.ldc = N;
  a.M = M;
  a.K = K;
  a.N = N;
  a.accumulate = (flags & BUDDY_HIP_GEMV_ACCUMULATE) != 0;
  a.terms = (flags & BUDDY_HIP_GEMM_A_F32_EXACT) ? 3 : 1;
  a.digits = (flags & BUDDY_HIP_GEMM_A_I8_DIGITS) ? ((flags & BUDDY_HIP_GEMM_TWO_DIGITS) ? 2 : 3) : 0;
  BH_REQUIRE(a.digits || !(flags & BUDDY_HIP_GEMM_TWO_DIGITS),
             "gemm_w8a32: BUDDY_HIP_GEMM_TWO_DIGITS needs BUDDY_HIP_GEMM_A_I8_DIGITS");
  if (flags & BUDDY_HIP_GEMM_SILU_PAIR) {
    BH_REQUIRE(a.digits, "gemm_w8a32: BUDDY_HIP_GEMM_SILU_PAIR needs BUDDY_HIP_GEMM_A_I8_DIGITS");
    a.silu_pair = true;
    a.N = 2 * N; // both matrices; the result has N channels
  }
  return bh::launch_gemm_w8(a, bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_gemm_w8a32")
}
