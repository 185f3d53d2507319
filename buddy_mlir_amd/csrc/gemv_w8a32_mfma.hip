// gemv_w8a32_mfma.hip -- the int8 dequant matmul for small batches (2..16 rows)
// on the matrix cores.
//
// The reference has no kernel of its own for 1 < M <= 16: its decode patterns
// fire for m == 1 only (DequantMatMulVectorizationDecode.cpp:212-217) and the
// BLIS kernel (MatMulBlisVectorization.cpp:398-986) is the one vectorised
// kernel for M > 1.  On the GPU the f32 FMA pipe cannot keep up with HBM beyond
// a few rows (2 + M instructions per weight byte), so the rows go through
// v_mfma_f32_16x16x32_bf16: the 16 channels of a wave tile are the MFMA's rows,
// the batch rows its columns.  A lane's 16 weight bytes are two 8-wide A
// fragments (exact in bf16); the activations are staged in LDS as three bf16
// terms (all 24 significand bits), so six MFMAs consume one 1 KiB tile.  The
// weights stream exactly as in the one-row kernel, from the same packed copy.
#include "gemv_w8a32.h"

namespace bh {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned short u16;

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * kWave;
constexpr int kTerms = 3;
constexpr int kCols = 16;       // batch rows = MFMA columns
constexpr int kSpanTiles = 8;   // tiles staged per round, over all k-slices

struct MfmaArgs {
  const float *A;
  const int4 *W0, *W1;
  const float *s0, *s1, *bias;
  float *C;
  int64_t lda, ldc;
  int K, N, groups, chunks, G, KS, TR, rows;
};

__device__ __forceinline__ int4 load_stream(const int4 *p) {
  const v4i v = __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p));
  return make_int4(v.x, v.y, v.z, v.w);
}
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
__device__ __forceinline__ float silu(float g) {
  const float sig = 1.0f / (1.0f + expf(-g));
  return g * sig;
}

template <int EPI>
__global__ void __launch_bounds__(kThreads) gemv_w8a32_mfma_kernel(MfmaArgs a) {
  constexpr bool DUAL = (EPI == kEpiSiluMul);
  constexpr int U = DUAL ? 2 : 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int gl = wave / a.KS, ks = wave % a.KS;
  const int g = blockIdx.x * a.G + gl;
  const bool live = g < a.groups;
  const int per = (a.chunks + a.KS - 1) / a.KS; // tiles per k-slice
  const int t0 = min(ks * per, a.chunks), t1 = min(t0 + per, a.chunks);
  const int TR = a.TR;
  const int span = a.KS * TR * kTileK;   // staged k per row and round
  const int rs = span + 8;               // row stride in bf16 elements
  u16 *xs = reinterpret_cast<u16 *>(smem); // [kTerms][kCols][rs]
  float *red = reinterpret_cast<float *>(smem + sizeof(u16) * kTerms * kCols * rs);

  f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  const size_t wbase = ((size_t)(live ? g : 0) * a.chunks) * 64 + lane;
  const int4 *w0 = a.W0 + wbase;
  const int4 *w1 = DUAL ? a.W1 + wbase : a.W0 + wbase;
  const int m = lane & 15, kg = lane >> 4;
  const int nrounds = (per + TR - 1) / TR;

  for (int rd = 0; rd < nrounds; ++rd) {
    const int r0 = t0 + rd * TR, r1 = min(r0 + TR, t1);
    int4 wa[U], wb[U];
    if (r0 < r1) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int t = min(r0 + u, a.chunks - 1);
        wa[u] = load_stream(w0 + (size_t)t * 64);
        if (DUAL)
          wb[u] = load_stream(w1 + (size_t)t * 64);
      }
    }
    if (rd != 0)
      __syncthreads();
    // stage: slice s of the round covers tiles s*per + rd*TR .. + TR
    for (int i = tid; i < kCols * (span / 4); i += kThreads) {
      const int row = i / (span / 4), q = i % (span / 4);
      const int kk = q * 4; // position inside the staged span
      const int s = kk / (TR * kTileK), within = kk % (TR * kTileK);
      const int sl0 = min(s * per, a.chunks);
      const int kend = min(a.K, min(sl0 + per, a.chunks) * kTileK);
      const int k = (sl0 + rd * TR) * kTileK + within;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (row < a.rows && k < kend) {
        const float *src = a.A + (int64_t)row * a.lda + k;
        if (k + 3 < kend && ((reinterpret_cast<uintptr_t>(src) & 15) == 0))
          v = *reinterpret_cast<const float4 *>(src);
        else
          v = make_float4(src[0], k + 1 < kend ? src[1] : 0.f,
                          k + 2 < kend ? src[2] : 0.f, k + 3 < kend ? src[3] : 0.f);
      }
      // three truncated bf16 terms: each residual is exactly representable
      float r[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int t = 0; t < kTerms; ++t) {
        unsigned h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          h[e] = __float_as_uint(r[e]) & 0xffff0000u;
          r[e] -= __uint_as_float(h[e]);
        }
        *reinterpret_cast<uint2 *>(xs + ((size_t)t * kCols + row) * rs + kk) =
            make_uint2((h[0] >> 16) | h[1], (h[2] >> 16) | h[3]);
      }
    }
    __syncthreads();
    const u16 *xrow = xs + (size_t)m * rs + ks * TR * kTileK + kg * 16;
    for (int t = r0; t < r1; t += U) {
      int4 na[U], nb[U];
      const bool more = t + U < r1;
      if (more) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int tt = min(t + U + u, a.chunks - 1);
          na[u] = load_stream(w0 + (size_t)tt * 64);
          if (DUAL)
            nb[u] = load_stream(w1 + (size_t)tt * 64);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (t + u < r1) {
          const u16 *xt = xrow + (t + u - r0) * kTileK;
          const bf16x8 a_lo = frag_from(wa[u].x, wa[u].y), a_hi = frag_from(wa[u].z, wa[u].w);
          bf16x8 b_lo, b_hi;
          if (DUAL) {
            b_lo = frag_from(wb[u].x, wb[u].y);
            b_hi = frag_from(wb[u].z, wb[u].w);
          }
#pragma unroll
          for (int term = 0; term < kTerms; ++term) {
            const u16 *xp = xt + (size_t)term * kCols * rs;
            const bf16x8 x_lo = *reinterpret_cast<const bf16x8 *>(xp);
            const bf16x8 x_hi = *reinterpret_cast<const bf16x8 *>(xp + 8);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, x_lo, acc0, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, x_hi, acc0, 0, 0, 0);
            if (DUAL) {
              acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_lo, x_lo, acc1, 0, 0, 0);
              acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_hi, x_hi, acc1, 0, 0, 0);
            }
          }
        }
      }
      if (more) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          wa[u] = na[u];
          if (DUAL)
            wb[u] = nb[u];
        }
      }
    }
  }

  // k-slices of one channel group meet in LDS, in slice order
  if (a.KS > 1) {
    __syncthreads(); // staging area no longer read
    float *mine = red + (size_t)wave * 64 * 8;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      mine[lane * 8 + i] = acc0[i];
      if (DUAL)
        mine[lane * 8 + 4 + i] = acc1[i];
    }
    __syncthreads();
    if (ks != 0)
      return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float r0 = 0.f, r1 = 0.f;
      for (int s = 0; s < a.KS; ++s) {
        const float *o = red + (size_t)(wave + s) * 64 * 8 + lane * 8;
        r0 += o[i];
        if (DUAL)
          r1 += o[4 + i];
      }
      acc0[i] = r0;
      acc1[i] = r1;
    }
  }
  // lane holds batch row m and channels kg*4 .. kg*4+3 of the group
  if (live && m < a.rows) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = g * kTileN + kg * 4 + i;
      if (n < a.N) {
        float *c = a.C + (int64_t)m * a.ldc + n;
        const float v = acc0[i] * a.s0[n];
        if (EPI == kEpiSiluMul)
          *c = silu(v) * (acc1[i] * a.s1[n]);
        else if (EPI == kEpiAccum)
          *c = *c + v;
        else
          *c = a.bias ? a.bias[n] + v : v;
      }
    }
  }
}

template <int EPI>
int launch_epi(const MfmaArgs &ka, int blocks, size_t lds, hipStream_t stream) {
  auto kernel = gemv_w8a32_mfma_kernel<EPI>;
  static bool attr_set = false;
  if (!attr_set) {
    BH_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     96 * 1024));
    attr_set = true;
  }
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kThreads), lds, stream, ka);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace

// Small-batch path of launch_gemv (2 <= M <= 16, no fused RMSNorm).
int launch_gemv_mfma(const GemvArgs &a, hipStream_t stream) {
  MfmaArgs ka;
  ka.A = a.A;
  ka.W0 = reinterpret_cast<const int4 *>(a.W0);
  ka.W1 = reinterpret_cast<const int4 *>(a.W1);
  ka.s0 = a.s0;
  ka.s1 = a.s1;
  ka.bias = a.bias;
  ka.C = a.C;
  ka.lda = a.lda;
  ka.ldc = a.ldc;
  ka.K = (int)a.K;
  ka.N = (int)a.N;
  ka.groups = (int)ceil_div(a.N, kTileN);
  ka.chunks = (int)ceil_div(a.K, kTileK);
  ka.rows = a.M;
  // k-slices inside the workgroup when the matrix is narrow
  int ks = 1;
  while (ks < kWaves && ks < kSpanTiles / 2 && (int64_t)ka.groups * ks < 2048 &&
         ka.chunks / (ks * 2) >= 2)
    ks *= 2;
  ka.KS = ks;
  ka.G = kWaves / ks;
  ka.TR = kSpanTiles / ks;
  const int blocks = (int)ceil_div(ka.groups, ka.G);
  const int span = kSpanTiles * kTileK;
  const size_t lds = sizeof(u16) * kTerms * kCols * (span + 8) +
                     sizeof(float) * kWaves * 64 * 8;
  switch (a.epilogue) {
  case kEpiStore: return launch_epi<kEpiStore>(ka, blocks, lds, stream);
  case kEpiAccum: return launch_epi<kEpiAccum>(ka, blocks, lds, stream);
  case kEpiSiluMul: return launch_epi<kEpiSiluMul>(ka, blocks, lds, stream);
  }
  return fail(BUDDY_HIP_ERR_ARG, "gemv: unknown epilogue %d", a.epilogue);
}

} // namespace bh
