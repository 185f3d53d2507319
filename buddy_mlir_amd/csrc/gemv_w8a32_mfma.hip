// gemv_w8a32_mfma.hip -- the int8 dequant matmul for small batches (5..16 rows)
// on the bf16 matrix cores: the variant that keeps every bit of the f32
// activations (BUDDY_HIP_GEMV_BATCH=bf16; the default is the int8 matrix-core
// kernel of gemv_w8a32_i8.hip, which rounds them to 2^-23 of the largest of each
// 64 and is quicker).
//
// The reference has no kernel of its own for 1 < M <= 16: its decode patterns
// fire for m == 1 only (DequantMatMulVectorizationDecode.cpp:212-217) and the
// BLIS kernel (MatMulBlisVectorization.cpp:398-986) is the one vectorised
// kernel for M > 1.  On the GPU the f32 FMA pipe cannot keep up with HBM beyond
// a few rows (1 + M instructions per weight byte), so the rows go through
// v_mfma_f32_16x16x32_bf16: the 16 channels of a wave tile are the MFMA's rows,
// the batch rows its columns.
//  * A lane's 16 weight bytes are, as they lie in the tile, two 8-wide operand
//    fragments (exact in bf16).
//  * The other operand of lane l is x[row l % 16][16 consecutive k]: 64
//    contiguous bytes of the activation matrix, loaded straight from L2 and cut
//    into three truncated bf16 terms that add up to the f32 value exactly, so
//    the products are the f32 ones and only the order of summation differs.
//    No LDS staging, no barrier before the stream.
//  * A wavefront converts the activations of a 64-k chunk once and uses them
//    for SPAN channel groups (six MFMAs per 1 KiB tile), so activation traffic
//    from L2 stays below the weight stream.
//  * The weights stream exactly as in the one-row kernel, from the same packed
//    copy; k-slices of a workgroup meet in LDS in slice order.
//  * RMSNorm can be fused in: the weight multiplies the activation before it is
//    cut into terms, each lane gathers the squares of what it loads, and the
//    row's rsqrt factor multiplies the finished sums.
#include "gemv_w8a32.h"

namespace bh {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kMaxWavesMfma = 8; // 512 threads: up to 256 registers per lane

struct MfmaArgs {
  const float *A;
  const int4 *W0, *W1;
  const float *s0, *s1, *bias, *norm_w;
  float *C;
  int64_t lda, ldc;
  float norm_eps, norm_inv_k;
  int K, N, groups, chunks, spans; // spans = ceil(groups / SPAN)
  int GS, KS;                      // spans x k-slices of wavefronts per workgroup
  int rows;
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

// 8 f32 -> three bf16x8 terms, each the truncation of what the ones before it
// left over (8 + 8 + 8 significand bits: the sum is the f32 value).
__device__ __forceinline__ void split3(const float (&x)[8], bf16x8 (&t)[3]) {
  float r[8];
#pragma unroll
  for (int e = 0; e < 8; ++e)
    r[e] = x[e];
#pragma unroll
  for (int term = 0; term < 3; ++term) {
    unsigned h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      h[e] = __float_as_uint(r[e]) & 0xffff0000u;
      r[e] -= __uint_as_float(h[e]);
    }
    union {
      uint4 u;
      bf16x8 v;
    } p;
    p.u = make_uint4((h[0] >> 16) | h[1], (h[2] >> 16) | h[3], (h[4] >> 16) | h[5],
                     (h[6] >> 16) | h[7]);
    t[term] = p.v;
  }
}

// A clamped load near the end of a row is shifted: put the values of the 16-k
// run that starts at k back on their k and zero what lies beyond K.
__device__ __forceinline__ void fix_row_end(float (&v)[16], int k, int K) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int kq = k + 4 * q, sh = kq - min(kq, K - 4);
    if (sh != 0) {
      const float o[4] = {v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float r = 0.f;
#pragma unroll
        for (int d = 1; d < 4; ++d)
          if (e + d < 4 && sh == d)
            r = o[e + d < 4 ? e + d : 0];
        v[4 * q + e] = r;
      }
    }
  }
}

// The loads of the main loop are issued and waited for by hand: the compiler
// sinks ordinary prefetch loads down to their first use and then waits for them
// there.  A fetch is a fixed number of loads in a fixed order, vmcnt counts them
// in order, and each wait names the registers it releases so that nothing reads
// them earlier.
typedef float v4f32 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void issue_load(v4i &dst, const void *p) {
  asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void issue_load(v4f32 &dst, const void *p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}

template <int SPAN, bool DUAL, bool NORM> struct FetchRegs {
  v4i w0[SPAN];
  v4i w1[DUAL ? SPAN : 1];
  v4f32 x[4];  // 16 consecutive k of this lane's row
  v4f32 nw[NORM ? 4 : 1];
};
template <int SPAN, bool DUAL, bool NORM> constexpr int fetch_loads() {
  return SPAN * (DUAL ? 2 : 1) + 4 * (NORM ? 2 : 1);
}

template <int SPAN, bool DUAL, bool NORM>
__device__ __forceinline__ void fetch_chunk(const MfmaArgs &a, const int4 *w0,
                                            const int4 *w1,
                                            const size_t (&gofs)[SPAN],
                                            const float *xrow, int kofs, int c,
                                            FetchRegs<SPAN, DUAL, NORM> &o) {
#pragma unroll
  for (int s = 0; s < SPAN; ++s) {
    issue_load(o.w0[s], w0 + gofs[s] + (size_t)c * 64);
    if (DUAL)
      issue_load(o.w1[s], w1 + gofs[s] + (size_t)c * 64);
  }
  // activations: clamped inside the row; the last chunk of a ragged row is
  // put right when it is consumed
  const int k = c * kTileK + kofs;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int kq = min(k + 4 * q, a.K - 4);
    issue_load(o.x[q], xrow + kq);
    if (NORM)
      issue_load(o.nw[q], a.norm_w + kq);
  }
}

// Waits until at most N loads are in flight; the registers of `f` are valid
// only after it.
template <int N, int SPAN, bool DUAL, bool NORM>
__device__ __forceinline__ void wait_fetch(FetchRegs<SPAN, DUAL, NORM> &f) {
  asm volatile("s_waitcnt vmcnt(%4)"
               : "+v"(f.x[0]), "+v"(f.x[1]), "+v"(f.x[2]), "+v"(f.x[3])
               : "n"(N)
               : "memory");
#pragma unroll
  for (int s = 0; s < SPAN; ++s) {
    asm volatile("" : "+v"(f.w0[s])::"memory");
    if (DUAL)
      asm volatile("" : "+v"(f.w1[DUAL ? s : 0])::"memory");
  }
  if (NORM) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      asm volatile("" : "+v"(f.nw[NORM ? q : 0])::"memory");
  }
}

// Fetches kept in flight: three, two when a fetch is wide (two matrices or a
// fused norm) so that the ring stays inside 256 registers.
template <int SPAN, bool DUAL, bool NORM> constexpr int kRingOf() {
  return (DUAL || NORM || SPAN > 4) ? 2 : 3;
}

template <int EPI, int SPAN, bool NORM>
__global__ void __launch_bounds__(kMaxWavesMfma *kWave)
    gemv_w8a32_mfma_kernel(MfmaArgs a) {
  constexpr bool DUAL = (EPI == kEpiSiluMul);
  constexpr int NA = DUAL ? 2 * SPAN : SPAN; // accumulators per lane
  extern __shared__ __attribute__((aligned(16))) float red[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ksh = shift_of(a.KS);
  const int sl = wave >> ksh, ks = wave & (a.KS - 1);
  const int span = blockIdx.x * a.GS + sl;
  const bool live = span < a.spans;
  const int g0 = (live ? span : 0) * SPAN;
  const int per = (a.chunks + a.KS - 1) >> ksh;
  const int c0 = min(ks * per, a.chunks), c1 = min(c0 + per, a.chunks);
  const int m = lane & 15, kg = lane >> 4;

  f32x4 acc0[SPAN], acc1[DUAL ? SPAN : 1];
#pragma unroll
  for (int s = 0; s < SPAN; ++s) {
    acc0[s] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (DUAL)
      acc1[s] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  float ss = 0.f;
  // groups past the end of the matrix repeat the last one (never stored)
  size_t gofs[SPAN];
#pragma unroll
  for (int s = 0; s < SPAN; ++s)
    gofs[s] = (size_t)min(g0 + s, a.groups - 1) * a.chunks * 64;
  const int4 *w0 = a.W0 + lane;
  const int4 *w1 = (DUAL ? a.W1 : a.W0) + lane;
  const float *xrow = a.A + (int64_t)min(m, a.rows - 1) * a.lda;
  const int kofs = kg * 16;

  constexpr int L = fetch_loads<SPAN, DUAL, NORM>();
  constexpr int R = kRingOf<SPAN, DUAL, NORM>(); // fetches in flight
  FetchRegs<SPAN, DUAL, NORM> ring[R];
  // chunks past the end of the slice are fetched again from its last chunk
  // (never used): every fetch is exactly L loads, which keeps the counts exact
  const int clast = max(c1 - 1, 0);
#pragma unroll
  for (int u = 0; u < R; ++u)
    fetch_chunk<SPAN, DUAL, NORM>(a, w0, w1, gofs, xrow, kofs, min(c0 + u, clast), ring[u]);
  const bool ragged = (a.K & (kTileK - 1)) != 0;
  for (int cb = c0; cb < c1; cb += R) {
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int c = cb + u;
      if (c >= c1)
        continue;
      FetchRegs<SPAN, DUAL, NORM> &cur = ring[u];
      wait_fetch<(R - 1) * L, SPAN, DUAL, NORM>(cur); // chunk c has arrived
    // this lane's 16 activations -> 2 halves x 3 bf16 terms
    float xv[16] = {cur.x[0].x, cur.x[0].y, cur.x[0].z, cur.x[0].w,
                    cur.x[1].x, cur.x[1].y, cur.x[1].z, cur.x[1].w,
                    cur.x[2].x, cur.x[2].y, cur.x[2].z, cur.x[2].w,
                    cur.x[3].x, cur.x[3].y, cur.x[3].z, cur.x[3].w};
    const int k = c * kTileK + kofs;
    if (ragged && c == a.chunks - 1)
      fix_row_end(xv, k, a.K);
    if (NORM) {
      float nv[16] = {cur.nw[0].x, cur.nw[0].y, cur.nw[0].z, cur.nw[0].w,
                      cur.nw[NORM ? 1 : 0].x, cur.nw[NORM ? 1 : 0].y, cur.nw[NORM ? 1 : 0].z, cur.nw[NORM ? 1 : 0].w,
                      cur.nw[NORM ? 2 : 0].x, cur.nw[NORM ? 2 : 0].y, cur.nw[NORM ? 2 : 0].z, cur.nw[NORM ? 2 : 0].w,
                      cur.nw[NORM ? 3 : 0].x, cur.nw[NORM ? 3 : 0].y, cur.nw[NORM ? 3 : 0].z, cur.nw[NORM ? 3 : 0].w};
      if (ragged && c == a.chunks - 1)
        fix_row_end(nv, k, a.K);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        ss = fmaf(xv[e], xv[e], ss);
        xv[e] *= nv[e];
      }
    }
    bf16x8 xlo[3], xhi[3];
    {
      const float lo[8] = {xv[0], xv[1], xv[2], xv[3], xv[4], xv[5], xv[6], xv[7]};
      const float hi[8] = {xv[8], xv[9], xv[10], xv[11], xv[12], xv[13], xv[14], xv[15]};
      split3(lo, xlo);
      split3(hi, xhi);
    }
#pragma unroll
    for (int s = 0; s < SPAN; ++s) {
      const bf16x8 a_lo = frag_from(cur.w0[s].x, cur.w0[s].y);
      const bf16x8 a_hi = frag_from(cur.w0[s].z, cur.w0[s].w);
#pragma unroll
      for (int t = 0; t < 3; ++t) {
        acc0[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, xlo[t], acc0[s], 0, 0, 0);
        acc0[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, xhi[t], acc0[s], 0, 0, 0);
      }
      if (DUAL) {
        const bf16x8 b_lo = frag_from(cur.w1[DUAL ? s : 0].x, cur.w1[DUAL ? s : 0].y);
        const bf16x8 b_hi = frag_from(cur.w1[DUAL ? s : 0].z, cur.w1[DUAL ? s : 0].w);
#pragma unroll
        for (int t = 0; t < 3; ++t) {
          acc1[DUAL ? s : 0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_lo, xlo[t], acc1[DUAL ? s : 0], 0, 0, 0);
          acc1[DUAL ? s : 0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b_hi, xhi[t], acc1[DUAL ? s : 0], 0, 0, 0);
        }
      }
    }
      // the registers of chunk c are free: fetch the chunk R further on
      fetch_chunk<SPAN, DUAL, NORM>(a, w0, w1, gofs, xrow, kofs, min(c + R, clast), cur);
    }
  }
  // repeated last chunks may still be in flight: the ring registers stay
  // allocated until they have landed (without these ties the compiler may put
  // a temporary of the code below into one of them before the wait, and the
  // late load would overwrite it)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int u = 0; u < R; ++u)
    wait_fetch<0, SPAN, DUAL, NORM>(ring[u]);
  if (NORM) { // the four lanes that share a row hold different k
    ss = sum_rows(ss);
  }

  // ---- k-slices meet in LDS, in slice order --------------------------------
  constexpr int kPerWave = (NA * 4 + 1) * kWave; // floats per wavefront
  if (a.KS > 1) {
    float *mine = red + (size_t)wave * kPerWave;
#pragma unroll
    for (int s = 0; s < SPAN; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        mine[(s * 4 + i) * kWave + lane] = acc0[s][i];
        if (DUAL)
          mine[((SPAN + s) * 4 + i) * kWave + lane] = acc1[DUAL ? s : 0][i];
      }
    if (NORM)
      mine[NA * 4 * kWave + lane] = ss;
    __syncthreads();
    if (ks != 0)
      return;
#pragma unroll
    for (int s = 0; s < SPAN; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float r0 = 0.f, r1 = 0.f;
        for (int q = 0; q < a.KS; ++q) {
          const float *o = red + (size_t)(wave + q) * kPerWave;
          r0 += o[(s * 4 + i) * kWave + lane];
          if (DUAL)
            r1 += o[((SPAN + s) * 4 + i) * kWave + lane];
        }
        acc0[s][i] = r0;
        if (DUAL)
          acc1[DUAL ? s : 0][i] = r1;
      }
    if (NORM) {
      float r = 0.f;
      for (int q = 0; q < a.KS; ++q)
        r += red[(size_t)(wave + q) * kPerWave + NA * 4 * kWave + lane];
      ss = r;
    }
  }
  // lane holds batch row m and channels kg*4 .. kg*4+3 of each group
  if (!live || m >= a.rows)
    return;
  const float rn = NORM ? 1.0f / sqrtf(ss * a.norm_inv_k + a.norm_eps) : 1.0f;
#pragma unroll
  for (int s = 0; s < SPAN; ++s) {
    const int g = g0 + s;
    if (g >= a.groups)
      continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = g * kTileN + kg * 4 + i;
      if (n < a.N) {
        float *c = a.C + (int64_t)m * a.ldc + n;
        const float v = acc0[s][i] * rn * a.s0[n];
        if (EPI == kEpiSiluMul)
          *c = silu(v) * (acc1[DUAL ? s : 0][i] * rn * a.s1[n]);
        else if (EPI == kEpiAccum)
          *c = *c + v;
        else
          *c = a.bias ? a.bias[n] + v : v;
      }
    }
  }
}

BH_VARIANT_FAMILY(MfmaFamily, "gemv_w8a32_mfma_kernel");

template <int EPI, int SPAN, bool NORM>
int launch_kernel(const MfmaArgs &ka, int blocks, hipStream_t stream) {
  constexpr int NA = (EPI == kEpiSiluMul) ? 2 * SPAN : SPAN;
  const int waves = ka.GS * ka.KS;
  const size_t lds = ka.KS > 1 ? sizeof(float) * waves * (size_t)(NA * 4 + 1) * kWave : 0;
  auto kernel = gemv_w8a32_mfma_kernel<EPI, SPAN, NORM>;
  static DynLdsOnce dyn_lds;
  BH_CHECK_HIP(ensure_dyn_lds(dyn_lds, reinterpret_cast<const void *>(kernel),
                              144 * 1024));
  BH_NOTE_VARIANT(MfmaFamily, EPI, SPAN, NORM);
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(waves * kWave), lds, stream, ka);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

template <int EPI, int SPAN>
int launch_norm(const MfmaArgs &ka, int blocks, hipStream_t stream) {
  return ka.norm_w ? launch_kernel<EPI, SPAN, true>(ka, blocks, stream)
                   : launch_kernel<EPI, SPAN, false>(ka, blocks, stream);
}

template <int SPAN>
int launch_span(const MfmaArgs &ka, int epilogue, int blocks, hipStream_t stream) {
  switch (epilogue) {
  case kEpiStore: return launch_norm<kEpiStore, SPAN>(ka, blocks, stream);
  case kEpiAccum: return launch_norm<kEpiAccum, SPAN>(ka, blocks, stream);
  case kEpiSiluMul:
    // two matrices with eight groups each do not fit the register file (the
    // fetch ring must never spill), so that variant is not built
    if (SPAN > 4)
      return fail(BUDDY_HIP_ERR_ARG, "gemv: SiLU*mul with %d groups per wavefront", SPAN);
    return launch_norm<kEpiSiluMul, (SPAN > 4 ? 4 : SPAN)>(ka, blocks, stream);
  }
  return fail(BUDDY_HIP_ERR_ARG, "gemv: unknown epilogue %d", epilogue);
}

} // namespace

// Small-batch path of launch_gemv (2 <= M <= 16).
int launch_gemv_mfma(const GemvArgs &a, hipStream_t stream) {
  MfmaArgs ka;
  ka.A = a.A;
  ka.W0 = reinterpret_cast<const int4 *>(a.W0);
  ka.W1 = reinterpret_cast<const int4 *>(a.W1);
  ka.s0 = a.s0;
  ka.s1 = a.s1;
  ka.bias = a.bias;
  ka.norm_w = a.norm_w;
  ka.norm_eps = a.norm_eps;
  ka.norm_inv_k = a.norm_inv_k;
  ka.C = a.C;
  ka.lda = a.lda;
  ka.ldc = a.ldc;
  ka.K = (int)a.K;
  ka.N = (int)a.N;
  ka.groups = (int)ceil_div(a.N, kTileN);
  ka.chunks = (int)ceil_div(a.K, kTileK);
  ka.rows = a.M;
  const bool dual = a.epilogue == kEpiSiluMul;
  // channel groups per wavefront (they share one conversion of the
  // activations): eight for wide single-matrix launches, else four, two when
  // that leaves too few wavefronts to cover the chip even with 8 k-slices.
  // (Measured: fewer, wider spans would cut the L2 -> CU traffic of the
  // activations, but the launches get slower, not faster: 2.9 -> 3.9 ms for the
  // Llama-3-8B sweep at 8 rows.)
  int span = 4;
  if (!dual && ceil_div(ka.groups, 8) >= 1024)
    span = 8;
  else if (ceil_div(ka.groups, 4) * kMaxWavesMfma < 1024)
    span = 2;
  ka.spans = (int)ceil_div(ka.groups, span);
  // k-slices: enough wavefronts for 256 CUs, at least two chunks each; the
  // meeting place of a two-matrix launch must fit in LDS
  int ks = 1;
  const int ks_max = dual && span == 4 ? 8 : kMaxWavesMfma;
  while (ks < ks_max && (int64_t)ka.spans * ks < 2048 && ka.chunks / (ks * 2) >= 2)
    ks *= 2;
  BH_REQUIRE(is_pow2(ks), "gemv: %d k-slices (the kernels shift by their count)", ks);
  ka.KS = ks;
  ka.GS = ks < 4 ? 4 / ks : 1;
  const int blocks = (int)ceil_div(ka.spans, ka.GS);
  if (span == 8)
    return launch_span<8>(ka, a.epilogue, blocks, stream);
  return span == 4 ? launch_span<4>(ka, a.epilogue, blocks, stream)
                   : launch_span<2>(ka, a.epilogue, blocks, stream);
}

} // namespace bh
