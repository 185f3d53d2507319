// gemv_w8a32.hip -- int8 weight-only decode GEMV / small-batch matmul.
//
// Replaces the loop nest that
// midend/lib/Conversion/MatMulOptimization/DequantMatMulVectorizationDecode.cpp
// :250-321 generates (parallel over 32-wide n panels, sequential k, scale
// applied once after the reduction, result added to C).
//
// The kernel is HBM-bound, so its shape follows the memory system:
//  * weights live in 1 KiB wave tiles (16 channels x 64 k); one wavefront
//    streams one channel group's K extent with 128-bit loads, 1 KiB per
//    instruction, contiguous from tile to tile;
//  * a workgroup is 4 wavefronts = 4 adjacent channel groups over the same k
//    range, so the activation slice is staged in LDS once per 64 channels;
//  * the k range is split over blockIdx.y when the matrix alone cannot fill
//    256 CUs; partial sums meet in a workspace and the last workgroup to
//    arrive (a ticket per block column) adds them in split order, so the result
//    does not depend on arrival order;
//  * the scale, bias, residual add and SiLU*up are applied to the finished sums
//    in the same kernel, and RMSNorm can be applied to the activations while
//    they are staged.
// No MFMA: at M <= 16 the arithmetic is far below the bandwidth ridge.
#include "gemv_w8a32.h"

#include <cstdlib>

namespace bh {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kThreads = kWavesPerBlock * kWave;
constexpr int kMaxCounters = 4096;
constexpr size_t kCounterBytes = kMaxCounters * sizeof(unsigned);
constexpr size_t kMaxLdsBytes = 96 * 1024;

struct GemvPlan {
  int64_t chunks, groups, np;
  int bx, splits, cps;
  size_t lds_bytes, partial_bytes;
};

int target_blocks() {
  static int v = [] {
    const char *e = getenv("BUDDY_HIP_GEMV_TARGET_BLOCKS");
    int t = e ? atoi(e) : 0;
    return t > 0 ? t : 1024;
  }();
  return v;
}

GemvPlan make_plan(int64_t M, int64_t K, int64_t N, bool dual) {
  GemvPlan p;
  p.chunks = ceil_div(K, kTileK);
  p.groups = ceil_div(N, kTileN);
  p.np = p.groups * kTileN;
  p.bx = (int)ceil_div(p.groups, kWavesPerBlock);
  // enough workgroups to cover 256 CUs several times over, but at least two
  // tiles per wavefront
  int64_t want = ceil_div(target_blocks(), p.bx);
  int64_t max_by_work = p.chunks / 2 > 0 ? p.chunks / 2 : 1;
  int64_t s = want < max_by_work ? want : max_by_work;
  if (s < 1)
    s = 1;
  // the activation slice of one split must fit in LDS
  const int64_t max_cps = (int64_t)(kMaxLdsBytes / (sizeof(float) * kTileK * M));
  int64_t cps = ceil_div(p.chunks, s);
  if (cps > max_cps)
    cps = max_cps;
  p.cps = (int)cps;
  p.splits = (int)ceil_div(p.chunks, cps);
  if (p.bx > kMaxCounters) { // never split matrices that wide
    p.splits = 1;
    p.cps = (int)p.chunks;
  }
  p.lds_bytes = sizeof(float) * (size_t)M * p.cps * kTileK + 64 * sizeof(float);
  p.partial_bytes = p.splits > 1 ? sizeof(float) * (size_t)p.splits *
                                       (dual ? 2 : 1) * M * p.np
                                 : 0;
  return p;
}

struct KernelArgs {
  const float *A;
  const int4 *W0, *W1;
  const float *s0, *s1, *bias, *norm_w;
  float *C;
  float *partial;
  unsigned *counters;
  int64_t lda, ldc;
  float norm_eps, norm_inv_k;
  int K, N, np, groups, chunks, cps, splits;
  int rows; // valid rows; the kernel is compiled for the next power of two
};

typedef int v4i __attribute__((ext_vector_type(4)));

// Weights are read exactly once per launch: stream them past the caches.
__device__ __forceinline__ int4 load_stream(const int4 *p) {
  const v4i v = __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p));
  return make_int4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ float byte_to_float(int v, int j) {
  return (float)(signed char)(v >> (8 * j));
}

// acc[m] += sum_j x[m][j] * w[j] for the lane's 16 k values.
template <int M>
__device__ __forceinline__ void fma_tile(const int4 &w, const float *xl,
                                         int kspan, float (&acc)[M]) {
  float wf[16];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    wf[j] = byte_to_float(w.x, j);
    wf[4 + j] = byte_to_float(w.y, j);
    wf[8 + j] = byte_to_float(w.z, j);
    wf[12 + j] = byte_to_float(w.w, j);
  }
#pragma unroll
  for (int m = 0; m < M; ++m) {
    const float4 *xv = reinterpret_cast<const float4 *>(xl + m * kspan);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 x = xv[q];
      acc[m] = fmaf(x.x, wf[4 * q + 0], acc[m]);
      acc[m] = fmaf(x.y, wf[4 * q + 1], acc[m]);
      acc[m] = fmaf(x.z, wf[4 * q + 2], acc[m]);
      acc[m] = fmaf(x.w, wf[4 * q + 3], acc[m]);
    }
  }
}

__device__ __forceinline__ float silu(float g) {
  // (g * sigmoid(g)), sigmoid = 1/(1+exp(-g))
  // examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:225-227
  const float sig = 1.0f / (1.0f + expf(-g));
  return g * sig;
}

template <int EPI>
__device__ __forceinline__ void finish(const KernelArgs &a, int m, int n,
                                       float raw0, float raw1) {
  float *c = a.C + (int64_t)m * a.ldc + n;
  float v = raw0 * a.s0[n];
  if (EPI == kEpiSiluMul) {
    const float u = raw1 * a.s1[n];
    *c = silu(v) * u;
  } else if (EPI == kEpiAccum) {
    *c = *c + v;
  } else {
    *c = a.bias ? a.bias[n] + v : v;
  }
}

template <int M, int EPI, bool NORM>
__global__ void __launch_bounds__(kThreads) gemv_w8a32_kernel(KernelArgs a) {
  constexpr bool DUAL = (EPI == kEpiSiluMul);
  extern __shared__ float lds[];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int g = blockIdx.x * kWavesPerBlock + wave;
  const int split = blockIdx.y;
  const int c0 = split * a.cps;
  const int nch = min(a.cps, a.chunks - c0);
  const int k0 = c0 * kTileK;
  const int kspan = a.cps * kTileK;
  float *xs = lds;
  float *red = lds + M * kspan;

  // ---- stage the activation slice (optionally RMS-normalised) ------------
  float rms[M];
#pragma unroll
  for (int m = 0; m < M; ++m)
    rms[m] = 1.0f;
  if (NORM) {
    // sum of squares over the whole row, every workgroup for itself
    float ss[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float s = 0.f;
      for (int k = tid; k < (m < a.rows ? a.K : 0); k += kThreads) {
        const float v = a.A[(int64_t)m * a.lda + k];
        s = fmaf(v, v, s);
      }
      ss[m] = wave_sum(s);
    }
    if (lane == 0) {
#pragma unroll
      for (int m = 0; m < M; ++m)
        red[wave * 16 + m] = ss[m];
    }
    __syncthreads();
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const float tot = (red[m] + red[16 + m]) + (red[32 + m] + red[48 + m]);
      rms[m] = 1.0f / sqrtf(tot * a.norm_inv_k + a.norm_eps);
    }
  }
  {
    const int span = nch * kTileK;
#pragma unroll
    for (int m = 0; m < M; ++m) {
      for (int kk = tid; kk < span; kk += kThreads) {
        const int k = k0 + kk;
        const bool live = k < a.K && m < a.rows;
        float v = live ? a.A[(int64_t)m * a.lda + k] : 0.f;
        if (NORM && live)
          v = a.norm_w[k] * (v * rms[m]);
        xs[m * kspan + kk] = v;
      }
    }
  }
  __syncthreads();

  // ---- stream this wavefront's channel group -----------------------------
  float acc0[M], acc1[M]; // acc1 is dead code unless DUAL
#pragma unroll
  for (int m = 0; m < M; ++m) {
    acc0[m] = 0.f;
    acc1[m] = 0.f;
  }

  if (g < a.groups) {
    const size_t base = ((size_t)g * a.chunks + c0) * 64 + lane;
    const int4 *w0 = a.W0 + base;
    const int4 *w1 = DUAL ? a.W1 + base : nullptr;
    const float *xl = xs + (lane >> 4) * 16;
    constexpr int U = DUAL ? 2 : 4;
    int c = 0;
    for (; c + U <= nch; c += U) {
      int4 wa[U], wb[DUAL ? U : 1];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        wa[u] = load_stream(w0 + (size_t)(c + u) * 64);
        if (DUAL)
          wb[u] = load_stream(w1 + (size_t)(c + u) * 64);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        fma_tile<M>(wa[u], xl + (c + u) * kTileK, kspan, acc0);
        if (DUAL)
          fma_tile<M>(wb[u], xl + (c + u) * kTileK, kspan, acc1);
      }
    }
    for (; c < nch; ++c) {
      const int4 wa = load_stream(w0 + (size_t)c * 64);
      fma_tile<M>(wa, xl + c * kTileK, kspan, acc0);
      if (DUAL) {
        const int4 wb = load_stream(w1 + (size_t)c * 64);
        fma_tile<M>(wb, xl + c * kTileK, kspan, acc1);
      }
    }
  }
  // the four 16-lane rows hold the four k sub-ranges of the same channels
#pragma unroll
  for (int m = 0; m < M; ++m) {
    acc0[m] += __shfl_xor(acc0[m], 16, 64);
    acc0[m] += __shfl_xor(acc0[m], 32, 64);
    if (DUAL) {
      acc1[m] += __shfl_xor(acc1[m], 16, 64);
      acc1[m] += __shfl_xor(acc1[m], 32, 64);
    }
  }
  const int n = g * kTileN + lane;

  if (a.splits == 1) {
    if (lane < kTileN && g < a.groups && n < a.N) {
#pragma unroll
      for (int m = 0; m < M; ++m)
        if (m < a.rows)
          finish<EPI>(a, m, n, acc0[m], DUAL ? acc1[m] : 0.f);
    }
    return;
  }

  // ---- split-K: publish partial sums, last arrival reduces ---------------
  constexpr int NMAT = DUAL ? 2 : 1;
  if (lane < kTileN && g < a.groups) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      a.partial[((size_t)(split * NMAT + 0) * M + m) * a.np + n] = acc0[m];
      if (DUAL)
        a.partial[((size_t)(split * NMAT + 1) * M + m) * a.np + n] = acc1[m];
    }
  }
  __threadfence();
  __syncthreads();
  __shared__ int is_last;
  if (tid == 0) {
    const unsigned t = atomicAdd(&a.counters[blockIdx.x], 1u);
    is_last = (t == (unsigned)a.splits - 1);
  }
  __syncthreads();
  if (!is_last)
    return;
  __threadfence();
  const int nb = blockIdx.x * kWavesPerBlock * kTileN;
  for (int idx = tid; idx < M * kWavesPerBlock * kTileN; idx += kThreads) {
    const int m = idx / (kWavesPerBlock * kTileN);
    const int nn = nb + idx % (kWavesPerBlock * kTileN);
    if (nn >= a.N || m >= a.rows)
      continue;
    float r0 = 0.f, r1 = 0.f;
    for (int s = 0; s < a.splits; ++s) {
      r0 += __hip_atomic_load(
          &a.partial[((size_t)(s * NMAT + 0) * M + m) * a.np + nn],
          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (DUAL)
        r1 += __hip_atomic_load(
            &a.partial[((size_t)(s * NMAT + 1) * M + m) * a.np + nn],
            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    finish<EPI>(a, m, nn, r0, r1);
  }
  if (tid == 0)
    a.counters[blockIdx.x] = 0; // leave the workspace ready for the next launch
}

template <int M, int EPI, bool NORM>
int launch_one(const KernelArgs &ka, const GemvPlan &p, hipStream_t stream) {
  auto kernel = gemv_w8a32_kernel<M, EPI, NORM>;
  static bool attr_set = false;
  if (!attr_set) {
    BH_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)(kMaxLdsBytes + 1024)));
    attr_set = true;
  }
  hipLaunchKernelGGL(kernel, dim3(p.bx, p.splits), dim3(kThreads), p.lds_bytes,
                     stream, ka);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

template <int M>
int launch_m(const GemvArgs &a, const KernelArgs &ka, const GemvPlan &p,
             hipStream_t stream) {
  const bool norm = a.norm_w != nullptr;
  switch (a.epilogue) {
  case kEpiStore:
    return norm ? launch_one<M, kEpiStore, true>(ka, p, stream)
                : launch_one<M, kEpiStore, false>(ka, p, stream);
  case kEpiAccum:
    return norm ? launch_one<M, kEpiAccum, true>(ka, p, stream)
                : launch_one<M, kEpiAccum, false>(ka, p, stream);
  case kEpiSiluMul:
    return norm ? launch_one<M, kEpiSiluMul, true>(ka, p, stream)
                : launch_one<M, kEpiSiluMul, false>(ka, p, stream);
  }
  return fail(BUDDY_HIP_ERR_ARG, "gemv: unknown epilogue %d", a.epilogue);
}

} // namespace

size_t gemv_workspace_bytes(int64_t M, int64_t K, int64_t N, bool dual) {
  if (M < 1 || K < 1 || N < 1)
    return 0;
  // rows beyond 16 are processed in slabs of at most 16
  const int64_t mc = M > 16 ? 16 : M;
  const int64_t m = mc <= 2 ? mc : mc <= 4 ? 4 : mc <= 8 ? 8 : 16;
  const GemvPlan p = make_plan(m, K, N, dual);
  return kCounterBytes + p.partial_bytes;
}

int launch_gemv(const GemvArgs &a, hipStream_t stream) {
  BH_REQUIRE(a.A && a.W0 && a.s0 && a.C, "gemv: null pointer");
  BH_REQUIRE(a.M >= 1 && a.M <= 16, "gemv: M=%d outside 1..16", a.M);
  BH_REQUIRE(a.K > 0 && a.N > 0 && a.K < (1 << 30) && a.N < (1 << 30),
             "gemv: bad shape K=%lld N=%lld", (long long)a.K, (long long)a.N);
  BH_REQUIRE(a.lda >= a.K && a.ldc >= a.N, "gemv: row stride below row length");
  const bool dual = a.epilogue == kEpiSiluMul;
  BH_REQUIRE(!dual || (a.W1 && a.s1), "gemv: SiLU*mul needs two matrices");
  BH_REQUIRE((reinterpret_cast<uintptr_t>(a.W0) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(a.W1) & 15) == 0,
             "gemv: packed weights must be 16-byte aligned");
  // the kernel is compiled for 1, 2, 4, 8 and 16 rows; extra rows are zero-
  // filled in LDS and never stored
  const int mt = a.M <= 2 ? a.M : a.M <= 4 ? 4 : a.M <= 8 ? 8 : 16;
  const GemvPlan p = make_plan(mt, a.K, a.N, dual);
  if (p.splits > 1) {
    if (!a.workspace || a.workspace_bytes < kCounterBytes + p.partial_bytes)
      return fail(BUDDY_HIP_ERR_WORKSPACE,
                  "gemv: workspace of %zu bytes needed, %zu given",
                  kCounterBytes + p.partial_bytes, a.workspace_bytes);
  }
  KernelArgs ka;
  ka.A = a.A;
  ka.W0 = reinterpret_cast<const int4 *>(a.W0);
  ka.W1 = reinterpret_cast<const int4 *>(a.W1);
  ka.s0 = a.s0;
  ka.s1 = a.s1;
  ka.bias = a.bias;
  ka.norm_w = a.norm_w;
  ka.C = a.C;
  ka.counters = reinterpret_cast<unsigned *>(a.workspace);
  ka.partial = a.workspace ? reinterpret_cast<float *>(
                                 static_cast<char *>(a.workspace) + kCounterBytes)
                           : nullptr;
  ka.lda = a.lda;
  ka.ldc = a.ldc;
  ka.norm_eps = a.norm_eps;
  ka.norm_inv_k = a.norm_inv_k;
  ka.K = (int)a.K;
  ka.N = (int)a.N;
  ka.np = (int)p.np;
  ka.groups = (int)p.groups;
  ka.chunks = (int)p.chunks;
  ka.cps = p.cps;
  ka.splits = p.splits;
  ka.rows = a.M;
  if (a.M == 1) return launch_m<1>(a, ka, p, stream);
  if (a.M == 2) return launch_m<2>(a, ka, p, stream);
  if (a.M <= 4) return launch_m<4>(a, ka, p, stream);
  if (a.M <= 8) return launch_m<8>(a, ka, p, stream);
  if (a.M <= 16) return launch_m<16>(a, ka, p, stream);
  return fail(BUDDY_HIP_ERR_ARG, "gemv: M=%d outside 1..16", a.M);
}

} // namespace bh

extern "C" {

size_t buddy_hip_gemv_workspace_bytes(int64_t M, int64_t K, int64_t N) {
  return bh::gemv_workspace_bytes(M, K, N, true);
}

int buddy_hip_workspace_init(void *workspace, size_t workspace_bytes,
                             buddy_hip_stream stream) {
  BH_REQUIRE(workspace || workspace_bytes == 0, "workspace_init: null pointer");
  if (workspace_bytes == 0)
    return BUDDY_HIP_OK;
  BH_CHECK_HIP(
      hipMemsetAsync(workspace, 0, workspace_bytes, bh::as_stream(stream)));
  return BUDDY_HIP_OK;
}

int buddy_hip_gemv_w8a32(const float *A, const int8_t *packed,
                         const float *scale, float *C, int64_t M, int64_t K,
                         int64_t N, unsigned flags, void *workspace,
                         size_t workspace_bytes, buddy_hip_stream stream) {
  BH_REQUIRE(M >= 1, "gemv_w8a32: M=%lld", (long long)M);
  // rows beyond 16 go in slabs; each slab streams the weights once
  for (int64_t m0 = 0; m0 < M; m0 += 16) {
    bh::GemvArgs a;
    a.A = A + m0 * K;
    a.lda = K;
    a.W0 = packed;
    a.s0 = scale;
    a.C = C + m0 * N;
    a.ldc = N;
    a.M = (int)(M - m0 < 16 ? M - m0 : 16);
    a.K = K;
    a.N = N;
    a.epilogue = (flags & BUDDY_HIP_GEMV_ACCUMULATE) ? bh::kEpiAccum
                                                     : bh::kEpiStore;
    a.workspace = workspace;
    a.workspace_bytes = workspace_bytes;
    int rc = bh::launch_gemv(a, bh::as_stream(stream));
    if (rc)
      return rc;
  }
  return BUDDY_HIP_OK;
}
}
