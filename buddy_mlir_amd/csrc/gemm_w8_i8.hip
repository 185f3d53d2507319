// gemm_w8_i8.hip -- the prefill matmul on the int8 matrix cores:
// C[M,N] (+)= A[M,K] . (int8 W[K,N] * scale[N]).
//
// Same contract as the bf16 kernels of gemm_w8_mfma.hip (the BLIS-style kernel
// of midend/lib/Conversion/MatMulOptimization/MatMulBlisVectorization.cpp:351-360,
// 398-986), another way to carry the f32 activations.  The int8 weights are used
// as they lie: a lane's 16 bytes of a packed 16 x 64 tile are one operand of
// v_mfma_i32_16x16x64_i8, so nothing is converted in the loop (the bf16 kernels
// spend more VALU time turning int8 into bf16 than the matrix cores spend on the
// products).  The activations become fixed point for that:
//   per row m a power-of-two step s[m] with |A[m,k]| / s[m] < 2^(8D-2),
//   X[m,k] = rint(A[m,k] / s[m])   (an integer of 8D-1 bits with its sign),
//   X = sum_j d_j 256^j with balanced digits d_j in [-128, 127] (each an int8;
//   the last one is what is left, at most 64 in magnitude),
// one integer matmul per digit plane with exact int32 sums, and
//   C[m,n] = s[m] * scale[n] * sum_j 256^j acc_j[m,n].
// The only rounding of the whole product is that of X: at most s/2 per element,
// i.e. 2^-(8D-1) of the row's largest magnitude (D = 3: 2^-23, the rounding an
// f32 sum of the same row makes when it adds the largest term; D = 2: 2^-15).
// The sums themselves are exact and do not depend on any order.  A row that
// holds a NaN or an infinity gets a NaN step, so every result of that row is
// NaN, as a NaN spreads through the reference's f32 multiply-add chain over the
// row (an infinity gives the reference +-inf or NaN per column; here NaN).
// |d q| <= 2^14, so K may not exceed 2^17.
//
// Digit planes lie like the bf16 terms do: [digit][row][k] int8, rows and k zero
// padded, followed by the row steps (f32 [rows_padded]).  A lane's operand is 16
// contiguous bytes of a plane row.
//
// Two workgroup shapes, as for bf16: 64 rows x 64 channels with K split over the
// four wavefronts (narrow matrices), and 64 or 48 rows x 256 or 320 channels with
// the activation fragments shared through LDS (wide matrices).
#include "gemm.h"

#include <algorithm>
#include <cstdlib>
#include <map>
#include <mutex>

namespace bh {
namespace {

constexpr int kSlices = 4;        // wavefronts per workgroup

typedef int v4i32 __attribute__((ext_vector_type(4)));

// ---- f32 rows -> digit planes ------------------------------------------------

// smallest power of two s (not below 2^-126) with mx / s < 2^(8 D - 2)
__device__ __forceinline__ float digit_step(float mx, int D) {
  const int ex = (int)((__float_as_uint(mx) >> 23) & 0xffu) - 127; // floor(log2 mx)
  const int e = max(ex + 1 - (8 * D - 2), -126);
  return __uint_as_float((unsigned)(e + 127) << 23);
}

// Row sources: four consecutive values k0..k0+3 of the row (zero past its end).
__device__ __forceinline__ void load4(const float *p, int k0, int n, float (&v)[4]) {
  if (k0 + 3 < n && (reinterpret_cast<uintptr_t>(p + k0) & 15) == 0) {
    const float4 q = *reinterpret_cast<const float4 *>(p + k0);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      v[e] = k0 + e < n ? p[k0 + e] : 0.f;
  }
}
struct PlainRow {
  const float *a;
  int n;
  __device__ __forceinline__ void operator()(int k0, float (&v)[4]) const {
    load4(a, k0, n, v);
  }
};
struct NormRow { // w * (x * rs)
  const float *x, *w;
  float rs;
  int n;
  __device__ __forceinline__ void operator()(int k0, float (&v)[4]) const {
    float xv[4], wv[4];
    load4(x, k0, n, xv);
    load4(w, k0, n, wv);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      v[e] = wv[e] * (xv[e] * rs);
  }
};
// SiLU(g) * u with the one-instruction exp and reciprocal (1 ulp each)
__device__ __forceinline__ float silu_times(float g, float u) {
  const float sig = fast_rcp(1.0f + fast_exp(-g));
  return (g * sig) * u;
}
struct SiluMulRow { // silu(g) * u
  const float *g, *u;
  int n;
  __device__ __forceinline__ void operator()(int k0, float (&v)[4]) const {
    float gv[4], uv[4];
    load4(g, k0, n, gv);
    load4(u, k0, n, uv);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      v[e] = silu_times(gv[e], uv[e]);
  }
};

// Rows of up to this many values are kept in LDS between the pass that finds the
// row maximum and the pass that writes the digits; longer rows are computed twice.
constexpr int kRowCache = 12288;

constexpr int kRowThreads = 512; // threads of a producer workgroup (one row)

// One workgroup of kRowThreads threads writes row `row` of every plane and its step.
// A thread owns the same groups of four values in both passes.
template <class F>
__device__ __forceinline__ void row_to_digits(const F &f, int n, int row, int D, int Mp,
                                              int Kp, int8_t *planes, float *red,
                                              float *cache) {
  const bool cached = Kp <= kRowCache;
  // the row's largest magnitude as the largest bit pattern of |v|: a NaN or an
  // infinity is then the maximum (fmaxf would drop a NaN) and gives the row a
  // NaN step, so that every result of the row is NaN -- what the reference's f32
  // multiply-add chain makes of such a row (MatMulBlisVectorization.cpp:644-740)
  unsigned mb = 0;
  constexpr unsigned kAbs = 0x7fffffffu;
#pragma unroll 3
  for (int k0 = threadIdx.x * 4; k0 < Kp; k0 += kRowThreads * 4) {
    float v[4];
    f(k0, v);
    mb = max(max(mb, max(__float_as_uint(v[0]) & kAbs, __float_as_uint(v[1]) & kAbs)),
             max(__float_as_uint(v[2]) & kAbs, __float_as_uint(v[3]) & kAbs));
    if (cached)
      *reinterpret_cast<float4 *>(cache + k0) = make_float4(v[0], v[1], v[2], v[3]);
  }
  mb = wave_max_u32(mb);
  __syncthreads(); // red may still be read by the caller's own reduction
  if ((threadIdx.x & 63) == 0)
    red[threadIdx.x >> 6] = __uint_as_float(mb);
  __syncthreads();
  {
    unsigned m2 = __float_as_uint(red[0]);
#pragma unroll
    for (int w = 1; w < kRowThreads / 64; ++w)
      m2 = max(m2, __float_as_uint(red[w]));
    mb = m2;
  }
  const bool finite = mb < 0x7f800000u;
  const float step = finite ? digit_step(__uint_as_float(mb), D) : __uint_as_float(0x7fc00000u);
  // a power of two as well; the digits of a non-finite row are left zero
  const float inv = finite ? 1.0f / step : 0.f;
  float *steps = reinterpret_cast<float *>(planes + (size_t)D * Mp * Kp);
  if (threadIdx.x == 0)
    steps[row] = step;
  const size_t plane = (size_t)Mp * Kp;
  for (int k0 = threadIdx.x * 4; k0 < Kp; k0 += kRowThreads * 4) {
    float v[4];
    if (cached) {
      const float4 q = *reinterpret_cast<const float4 *>(cache + k0);
      v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
    } else {
      f(k0, v);
    }
    int X[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      X[e] = finite ? (int)rintf(v[e] * inv) : 0;
    int8_t *dst = planes + (size_t)row * Kp + k0;
    for (int j = 0; j < D; ++j) {
      unsigned word = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        // the last digit is what is left (|.| <= 64 by the choice of the step)
        const int d = j + 1 < D ? ((X[e] + 128) & 255) - 128 : X[e];
        X[e] = (X[e] - d) >> 8; // exact: X - d is a multiple of 256
        word |= (unsigned)(d & 0xff) << (8 * e);
      }
      *reinterpret_cast<unsigned *>(dst + j * plane) = word;
    }
  }
}

__global__ void __launch_bounds__(kRowThreads)
activations_to_digits_kernel(const float *__restrict__ A, int64_t lda, int M, int K, int D,
                             int Mp, int Kp, int8_t *__restrict__ planes) {
  __shared__ float red[kRowThreads / 64];
  extern __shared__ __attribute__((aligned(16))) float row_cache[];
  const int row = blockIdx.x;
  if (row >= M) { // padding rows: zero digits, step 1
    for (int j = 0; j < D; ++j)
      for (int k0 = threadIdx.x * 4; k0 < Kp; k0 += kRowThreads * 4)
        *reinterpret_cast<unsigned *>(planes + ((size_t)j * Mp + row) * Kp + k0) = 0u;
    if (threadIdx.x == 0)
      reinterpret_cast<float *>(planes + (size_t)D * Mp * Kp)[row] = 1.0f;
    return;
  }
  row_to_digits(PlainRow{A + (int64_t)row * lda, K}, K, row, D, Mp, Kp, planes, red,
                row_cache);
}

__global__ void __launch_bounds__(kRowThreads)
rmsnorm_to_digits_kernel(const float *__restrict__ x, int64_t ldx,
                         const float *__restrict__ w, int n, float inv_n, float eps, int D,
                         int Mp, int Kp, int8_t *__restrict__ planes) {
  __shared__ float red[kRowThreads / 64];
  extern __shared__ __attribute__((aligned(16))) float row_cache[];
  const int row = blockIdx.x;
  const float *xr = x + (int64_t)row * ldx;
  float s = 0.f;
  for (int i = threadIdx.x; i < n; i += kRowThreads)
    s = fmaf(xr[i], xr[i], s);
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0)
    red[threadIdx.x >> 6] = s;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < kRowThreads / 64; w += 2) // pairs first, as four wavefronts did
    tot += red[w] + red[w + 1];
  const float rs = 1.0f / sqrtf(tot * inv_n + eps);
  row_to_digits(NormRow{xr, w, rs, n}, n, row, D, Mp, Kp, planes, red, row_cache);
}

__global__ void __launch_bounds__(kRowThreads)
silu_mul_to_digits_kernel(const float *__restrict__ g, const float *__restrict__ u, int64_t ld,
                          int n, int D, int Mp, int Kp, int8_t *__restrict__ planes) {
  __shared__ float red[kRowThreads / 64];
  extern __shared__ __attribute__((aligned(16))) float row_cache[];
  const int row = blockIdx.x;
  row_to_digits(SiluMulRow{g + (size_t)row * ld, u + (size_t)row * ld, n}, n, row, D, Mp, Kp,
                planes, red, row_cache);
}

// ---- the matmul ----------------------------------------------------------------

struct GemmI8Args {
  const int8_t *planes; // [D][Mp][Kp]
  const float *steps;   // [Mp]
  const int4 *W;
  const float *scale;
  const float *bias;
  float *C;
  int64_t ldc;
  int M, N, Mp, Kp, groups, chunks;
  int ncols;       // column tiles
  int cols_padded; // ids per row tile: column tiles x slices, padded to the XCD count
  // K split over `slices` workgroups per tile, chunks_per_slice chunks each
  // (the last may hold fewer, never none); partial is only used when slices > 1
  int slices, chunks_per_slice;
  float *partial;     // [tile][slice][wavefront][row block][16][16 GPW]
  int accumulate;
  int32_t *sums;      // one plane only: the int32 sums themselves, dense [M, N], or null
  int int_partials;   // one plane, K split: the slices leave their int32 sums as they are
};

// sum_j 256^j acc_j as f32 (each int32 sum is exact; the conversions round to 24
// bits, like an f32 accumulator would)
template <int D> __device__ __forceinline__ float combine(const v4i32 (&acc)[D], int r) {
  float v = (float)acc[D - 1][r];
#pragma unroll
  for (int j = D - 2; j >= 0; --j)
    v = fmaf(v, 256.0f, (float)acc[j][r]);
  return v;
}

// The finished value of one output.  One plane is the w8a8 matmul, whose result
// is f32(sum) * (s_a * s_w[n]) in exactly that order (linalg.py:12833-12845).
template <int D> __device__ __forceinline__ float scaled(float v, float step, float s) {
  return D == 1 ? v * (step * s) : (v * step) * s;
}

constexpr int kSplitGroups = 4; // channel groups of 16 per workgroup of the split kernel

// lane holds channels n..n+3 of row m: C = step[m] * scale[n] * v (+ bias | + C)
__device__ __forceinline__ void store_row(const GemmI8Args &a, int m, int n, float step,
                                          const float (&v)[4], const float (&s)[4],
                                          const float (&b)[4], bool vec) {
  float o[4];
#pragma unroll
  for (int r = 0; r < 4; ++r)
    o[r] = (v[r] * step) * s[r];
  float *c = a.C + (int64_t)m * a.ldc + n;
  if (vec) {
    float4 q = make_float4(o[0], o[1], o[2], o[3]);
    if (a.accumulate) {
      const float4 p = *reinterpret_cast<const float4 *>(c);
      q = make_float4(p.x + q.x, p.y + q.y, p.z + q.z, p.w + q.w);
    } else {
      q = make_float4(b[0] + q.x, b[1] + q.y, b[2] + q.z, b[3] + q.w);
    }
    *reinterpret_cast<float4 *>(c) = q;
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (n + r < a.N)
        c[r] = a.accumulate ? c[r] + o[r] : b[r] + o[r];
  }
}

template <int D> struct ChunkOperands {
  v4i32 w[kSplitGroups];
  v4i32 a[D][4]; // [digit][row block]
};

template <int D>
__device__ __forceinline__ void load_chunk(const v4i32 *const (&wp)[kSplitGroups],
                                           const int8_t *ap, size_t plane, size_t rb_stride,
                                           int c, ChunkOperands<D> &o) {
#pragma unroll
  for (int g = 0; g < kSplitGroups; ++g)
    o.w[g] = wp[g][(size_t)c * 64];
#pragma unroll
  for (int j = 0; j < D; ++j)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
      o.a[j][rb] = *reinterpret_cast<const v4i32 *>(ap + j * plane + rb * rb_stride +
                                                    (size_t)c * kTileK);
}

// 64 rows x 64 channels per workgroup; the four wavefronts split K and meet in
// LDS in slice order.
template <int D>
__global__ void __launch_bounds__(kSlices *kWave) gemm_w8_i8_kernel(
    const int8_t *p_planes, const int4 *p_W, int p_Mp, int p_Kp, int p_groups, int p_chunks,
    int p_ncols, int p_cols_padded, int p_slices, int p_chunks_per_slice, GemmI8Args rest) {
  // what a wavefront needs before its first fetch arrives in SGPRs (this file is
  // built with -amdgpu-kernarg-preload-count); the rest is loaded behind the fetch
  GemmI8Args a = rest;
  a.planes = p_planes;
  a.W = p_W;
  a.Mp = p_Mp;
  a.Kp = p_Kp;
  a.groups = p_groups;
  a.chunks = p_chunks;
  a.ncols = p_ncols;
  a.cols_padded = p_cols_padded;
  a.slices = p_slices;
  a.chunks_per_slice = p_chunks_per_slice;
  extern __shared__ __attribute__((aligned(16))) float red[]; // [slice][64][lane]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = blockIdx.x % a.cols_padded, rbk = blockIdx.x / a.cols_padded;
  if (col >= a.ncols)
    return; // padding id
  const int m0 = rbk * 64, g0 = col * kSplitGroups;
  const int per = (a.chunks + kSlices - 1) / kSlices;
  const int c0 = min(wave * per, a.chunks), c1 = min(c0 + per, a.chunks);

  v4i32 acc[kSplitGroups][4][D];
#pragma unroll
  for (int g = 0; g < kSplitGroups; ++g)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int j = 0; j < D; ++j)
        acc[g][rb][j] = v4i32{0, 0, 0, 0};

  const v4i32 *wp[kSplitGroups];
#pragma unroll
  for (int g = 0; g < kSplitGroups; ++g) // groups past the end repeat the last one
    wp[g] = reinterpret_cast<const v4i32 *>(a.W) +
            ((size_t)min(g0 + g, a.groups - 1) * a.chunks) * 64 + lane;
  const size_t plane = (size_t)a.Mp * a.Kp, rb_stride = (size_t)16 * a.Kp;
  const int8_t *ap = a.planes + (size_t)(m0 + (lane & 15)) * a.Kp + (lane >> 4) * 16;

  ChunkOperands<D> cur, nxt;
  if (c0 < c1)
    load_chunk<D>(wp, ap, plane, rb_stride, c0, cur);
  for (int c = c0; c < c1; ++c) {
    if (c + 1 < c1)
      load_chunk<D>(wp, ap, plane, rb_stride, c + 1, nxt);
#pragma unroll
    for (int j = 0; j < D; ++j)
#pragma unroll
      for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int g = 0; g < kSplitGroups; ++g)
          acc[g][rb][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(cur.w[g], cur.a[j][rb],
                                                                acc[g][rb][j], 0, 0, 0);
    if (c + 1 < c1)
      cur = nxt;
  }

  // wavefront w finishes channel group w: its scales, bias and the steps of the
  // rows are asked for here, ahead of the meeting in LDS, not at their use
  const int g = wave;
  const int n = (g0 + g) * kTileN + (lane >> 4) * 4;
  float s[4], b[4], row_step[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    s[r] = n + r < a.N ? a.scale[n + r] : 0.f;
    b[r] = (a.bias && n + r < a.N) ? a.bias[n + r] : 0.f;
  }
#pragma unroll
  for (int rb = 0; rb < 4; ++rb) {
    const int m = m0 + rb * 16 + (lane & 15);
    row_step[rb] = m < a.M ? a.steps[m] : 0.f;
  }
  float *mine = red + (size_t)wave * 64 * kWave;
#pragma unroll
  for (int gg = 0; gg < kSplitGroups; ++gg)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        mine[((gg * 4 + rb) * 4 + r) * kWave + lane] = combine<D>(acc[gg][rb], r);
  __syncthreads();
  if (g0 + g >= a.groups)
    return;
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
      v[r] = sum;
    }
    if (m >= a.M)
      continue;
    store_row(a, m, n, row_step[rb], v, s, b, vec);
  }
}

// Wide matrices: 16 RB rows x 64 GPW channels per workgroup (GPW channel groups
// per wavefront), every wavefront runs the whole K.  Wavefront w fetches the
// digit fragments of row block w for everyone and leaves them in LDS in fragment
// order (lane l at 16 l: conflict-free).  Weights go from global memory to
// registers to the matrix core.
//
// The loop is a pipeline of three stages so that the matrix cores never wait:
//  * global loads run kRing - 2 chunks ahead.  The compiler sinks ordinary loads
//    down to their first use (and then waits for them there), so they are issued
//    by hand and waited for by hand: a fetch is GPW + D loads in a fixed order,
//    vmcnt counts them in order, and each wait names the registers it releases
//    so that nothing reads them earlier.  The ring registers must never be
//    spilled (a reload would read a register while its load is in flight): the
//    build refuses scratch use in this file;
//  * the fragments of chunk c + 2 go to LDS at the top of chunk c (three
//    buffers), so the barrier that closes chunk c publishes them a whole chunk
//    before they are wanted;
//  * the fragments of the next digit plane (or of the next chunk's first one)
//    are read from LDS into the second half of a two-slot register buffer while
//    the matrix instructions of the current plane run.
//
// Matrices too narrow to fill the chip with such tiles split K over several
// workgroups per tile instead of shrinking the tile (a 64 x 64 tile reads its
// operands four times as often from L2, and that, not the matrix cores, is what
// bounds it).  Every slice writes its unscaled sums to a workspace and a second
// small kernel adds the slices in slice order, applies the scales and writes C.
// (Finishing a tile inside the kernel, by the workgroup that arrives last at a
// counter, needs device-scope fences; on this chip they write back and
// invalidate a whole L2 each time and slowed the running workgroups threefold.)
template <int GPW> struct RingDepth { static constexpr int value = GPW > 4 ? 4 : 5; };

// LDS of the wide kernel: three fragment buffers in the loop, four output tiles in
// the epilogue (and with PAIR the values that cross from wavefronts 2 and 3 to 0
// and 1); behind them, with PAIR, the scales of the workgroup's channels of both
// matrices and the steps of its rows, fetched once as the launch starts (loaded
// at their use, every one of them was an L2 round trip the epilogue waited out).
template <int D, int RB, int GPW, bool PAIR> constexpr size_t wide_main_lds_bytes() {
  const size_t loop = sizeof(v4i32) * 3 * D * RB * kWave;
  const size_t epi = sizeof(float) * kSlices * 16 * (GPW * 16 + 4) +
                     (PAIR ? sizeof(float4) * kSlices * ((RB + 1) / 2) * GPW * kWave : 0);
  return loop > epi ? loop : epi;
}
template <int RB, int GPW> constexpr int wide_epi_scales() { return 2 * 2 * GPW * 16; }
template <int D, int RB, int GPW, bool PAIR> constexpr size_t wide_lds_bytes() {
  return wide_main_lds_bytes<D, RB, GPW, PAIR>() +
         (PAIR ? sizeof(float) * (wide_epi_scales<RB, GPW>() + RB * 16) : 0);
}

__device__ __forceinline__ void issue_load(v4i32 &dst, const void *p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void issue_load_f32(float &dst, const void *p) {
  asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
template <int D, int GPW> struct FetchRegs {
  v4i32 w[GPW];
  v4i32 a[D];
};
// Waits until at most N loads are in flight; the registers of `f` are only valid
// after it.
template <int N, int D, int GPW>
__device__ __forceinline__ void wait_loads(FetchRegs<D, GPW> &f) {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
#pragma unroll
  for (int g = 0; g < GPW; ++g)
    asm volatile("" : "+v"(f.w[g])::"memory");
#pragma unroll
  for (int j = 0; j < D; ++j)
    asm volatile("" : "+v"(f.a[j])::"memory");
}

// PAIR: W holds two matrices of a.groups / 2 channel groups each, one behind the
// other; wavefronts 0 and 1 of a workgroup take 32 GPW channels of the first,
// wavefronts 2 and 3 the same channels of the second, and the result is
// SiLU(first) * second ([M, N / 2]): the two exchange halves of their tiles
// through LDS in the epilogue, so only half as much is stored and no launch
// reads both results again.
template <int D, int RB, int GPW, bool PAIR>
__global__ void __launch_bounds__(kSlices *kWave) gemm_w8_i8_wide_kernel(
    const int8_t *p_planes, const int4 *p_W, int p_Mp, int p_Kp, int p_groups, int p_chunks,
    int p_ncols, int p_cols_padded, int p_slices, int p_chunks_per_slice, GemmI8Args rest) {
  // what a wavefront needs before its first fetch arrives in SGPRs (this file is
  // built with -amdgpu-kernarg-preload-count); the rest is loaded behind the fetch
  GemmI8Args a = rest;
  a.planes = p_planes;
  a.W = p_W;
  a.Mp = p_Mp;
  a.Kp = p_Kp;
  a.groups = p_groups;
  a.chunks = p_chunks;
  a.ncols = p_ncols;
  a.cols_padded = p_cols_padded;
  a.slices = p_slices;
  a.chunks_per_slice = p_chunks_per_slice;
  constexpr int kRing = RingDepth<GPW>::value;
  constexpr int L = GPW + D; // loads per fetch
  // chunks per unrolled pass: a multiple of the ring, and an even number of
  // digit steps so that the two-slot fragment buffer is back where it started
  constexpr int kPass = (kRing * D) % 2 == 0 ? kRing : 2 * kRing;
  extern __shared__ __attribute__((aligned(16))) v4i32 frag_s[]; // [3][D][RB][64]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // ids equal modulo 8 run on the same XCD: the row tiles of one (column tile,
  // K slice) pair do, and share its weights in that XCD's L2
  const int unit = blockIdx.x % a.cols_padded, rbk = blockIdx.x / a.cols_padded;
  if (unit >= a.ncols * a.slices)
    return; // padding id
  const int col = unit % a.ncols, slice = unit / a.ncols;
  const int m0 = rbk * RB * 16;
  const int half_groups = a.groups / 2; // PAIR only
  // first channel group of this wavefront; with PAIR, within its matrix
  const int g0 = PAIR ? (col * 2 + (wave & 1)) * GPW : (col * kSlices + wave) * GPW;
  const int gbase = PAIR ? (wave >> 1) * half_groups : 0;
  const int glast = PAIR ? half_groups - 1 : a.groups - 1;
  const int cb = slice * a.chunks_per_slice;
  const int nch = min(a.chunks_per_slice, a.chunks - cb); // chunks of this slice, >= 1

  v4i32 acc[GPW][RB][D];
#pragma unroll
  for (int g = 0; g < GPW; ++g)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int j = 0; j < D; ++j)
        acc[g][rb][j] = v4i32{0, 0, 0, 0};

  const v4i32 *wp[GPW];
#pragma unroll
  for (int g = 0; g < GPW; ++g) // groups past the end repeat the last one
    wp[g] = reinterpret_cast<const v4i32 *>(a.W) +
            ((size_t)(gbase + min(g0 + g, glast)) * a.chunks + cb) * 64 + lane;
  const size_t plane = (size_t)a.Mp * a.Kp;
  // this wavefront fetches row block `wave` of the activation tile (with three
  // row blocks the fourth wavefront repeats the third's loads and stages nothing)
  const int my_rb = min(wave, RB - 1);
  const int8_t *ap = a.planes + (size_t)(m0 + my_rb * 16 + (lane & 15)) * a.Kp +
                     (size_t)cb * kTileK + (lane >> 4) * 16;

  FetchRegs<D, GPW> ring[kRing];
  // chunks past the end are fetched again from the last chunk (never used):
  // every fetch is exactly L loads, which is what keeps the counts below exact
  auto fetch = [&](int c, FetchRegs<D, GPW> &f) {
    const int cc = min(c, nch - 1);
#pragma unroll
    for (int g = 0; g < GPW; ++g)
      issue_load(f.w[g], wp[g] + (size_t)cc * 64);
#pragma unroll
    for (int j = 0; j < D; ++j)
      issue_load(f.a[j], ap + j * plane + (size_t)cc * kTileK);
  };
  auto stage = [&](const FetchRegs<D, GPW> &f, int buf) { // own row block -> LDS
    if (wave >= RB)
      return;
#pragma unroll
    for (int j = 0; j < D; ++j)
      frag_s[(((size_t)buf * D + j) * RB + wave) * kWave + lane] = f.a[j];
  };
  auto read_frags = [&](v4i32(&dst)[RB], int buf, int j) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
      dst[rb] = frag_s[(((size_t)buf * D + j) * RB + rb) * kWave + lane];
  };
  // PAIR: the epilogue's scales (both matrices, this workgroup's 64 GPW channels)
  // and row steps, two per thread, requested ahead of the stream (so the counted
  // waits below cover them) and parked in LDS for the epilogue
  constexpr int kEpiScales = wide_epi_scales<RB, GPW>(); // [matrix][32 GPW channels]
  float *epi_s = reinterpret_cast<float *>(frag_s) +
                 wide_main_lds_bytes<D, RB, GPW, PAIR>() / sizeof(float);
  float epi_v[2] = {0.f, 0.f};
  bool epi_ok[2] = {false, false};
  if constexpr (PAIR) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int idx = tid + u * kSlices * kWave;
      const float *src = a.scale; // a valid address for the slots past the end
      if (idx < kEpiScales) {
        const int mtx = idx / (kEpiScales / 2), ch = idx % (kEpiScales / 2);
        const int n = col * (kEpiScales / 2) + ch;
        epi_ok[u] = n < a.N;
        if (epi_ok[u])
          src = a.scale + (size_t)mtx * a.N + n;
      } else if (idx < kEpiScales + RB * 16) {
        const int mr = m0 + idx - kEpiScales;
        epi_ok[u] = mr < a.M;
        if (epi_ok[u])
          src = a.steps + mr;
      }
      issue_load_f32(epi_v[u], src);
    }
  }
#pragma unroll
  for (int u = 0; u < kRing; ++u)
    fetch(u, ring[u]);
  wait_loads<(kRing - 1) * L, D, GPW>(ring[0]); // chunk 0 has arrived
  if constexpr (PAIR) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      asm volatile("" : "+v"(epi_v[u])::"memory"); // older than chunk 0: landed
      const int idx = tid + u * kSlices * kWave;
      if (idx < kEpiScales + RB * 16)
        epi_s[idx] = epi_ok[u] ? epi_v[u] : 0.f;
    }
  }
  stage(ring[0], 0);
  wait_loads<(kRing - 2) * L, D, GPW>(ring[1]);
  stage(ring[1], 1);
  __syncthreads();
  v4i32 af[2][RB];
  read_frags(af[0], 0, 0);
  int buf = 0; // LDS buffer of chunk c: c % 3
  for (int c0 = 0; c0 < nch; c0 += kPass) {
#pragma unroll
    for (int u = 0; u < kPass; ++u) {
      const int c = c0 + u;
      if (c < nch) {
        FetchRegs<D, GPW> &cur = ring[u % kRing];
        FetchRegs<D, GPW> &ahead = ring[(u + 2) % kRing];
        const int buf1 = buf == 2 ? 0 : buf + 1, buf2 = buf1 == 2 ? 0 : buf1 + 1;
        // in flight: chunks c+2 .. c+kRing-1.  Release chunk c+2 and put its row
        // block into the buffer that held chunk c-1, whose readers passed the
        // barrier that closed chunk c-1.
        wait_loads<(kRing - 3) * L, D, GPW>(ahead);
        stage(ahead, buf2);
#pragma unroll
        for (int j = 0; j < D; ++j) {
          const int p = (u * D + j) & 1; // slot of this digit step's fragments
          if (j + 1 < D)
            read_frags(af[p ^ 1], buf, j + 1);
          else
            read_frags(af[p ^ 1], buf1, 0);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int g = 0; g < GPW; ++g)
              acc[g][rb][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(cur.w[g], af[p][rb],
                                                                    acc[g][rb][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
        // the matrix cores have read the registers of chunk c when the next
        // instruction issues: fetch the chunk kRing further on into them
        fetch(c + kRing, cur);
        __syncthreads();
        buf = buf1;
      }
    }
  }
  // loads of the repeated last chunk may still be in flight: their registers
  // stay allocated until the wait is over
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int u = 0; u < kRing; ++u)
    wait_loads<0, D, GPW>(ring[u]);

  // ---- epilogue ---------------------------------------------------------
  // A lane's accumulator registers are 4 channels of one row: stored as they are,
  // a store instruction would write 64-byte pieces of 16 rows.  Each wavefront
  // turns its 16 x (16 GPW) tile around in its own part of LDS (free now: every
  // wavefront is past the last barrier of the loop) and writes whole row
  // segments, 64 GPW bytes each.
  constexpr int kPad = GPW * 16 + 4; // floats per tile row in LDS
  float *tile = reinterpret_cast<float *>(frag_s) + wave * (16 * kPad);
  const int n0 = g0 * kTileN;
  const bool vec = (a.ldc & 3) == 0 && (reinterpret_cast<uintptr_t>(a.C) & 15) == 0;
  if (a.slices > 1) {
    // unscaled sums of this slice; reduce_slices_kernel finishes the tile
    constexpr int kSub = 16 * GPW * 16; // floats of one wavefront's row block
    const int tile_id = rbk * a.ncols + col;
    float *mine = a.partial +
                  ((((size_t)tile_id * a.slices + slice) * kSlices + wave) * RB) * kSub;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
      for (int g = 0; g < GPW; ++g) {
        float4 o = make_float4(combine<D>(acc[g][rb], 0), combine<D>(acc[g][rb], 1),
                               combine<D>(acc[g][rb], 2), combine<D>(acc[g][rb], 3));
        if constexpr (D == 1) {
          if (a.int_partials) // exact beyond 2^24: the bits travel as they are
            o = make_float4(__int_as_float(acc[g][rb][0][0]), __int_as_float(acc[g][rb][0][1]),
                            __int_as_float(acc[g][rb][0][2]), __int_as_float(acc[g][rb][0][3]));
        }
        *reinterpret_cast<float4 *>(tile + (lane & 15) * kPad + g * 16 + (lane >> 4) * 4) = o;
      }
#pragma unroll
      for (int i = 0; i < GPW; ++i) {
        const int idx = lane + 64 * i;
        const int row = idx / (GPW * 4), c4 = idx % (GPW * 4);
        *reinterpret_cast<float4 *>(mine + (size_t)rb * kSub + idx * 4) =
            *reinterpret_cast<const float4 *>(tile + row * kPad + c4 * 4);
      }
    }
    return;
  }
  // without PAIR the scales and the bias stay in registers over the row blocks;
  // with it there is no register left for them, and each use loads them again
  float s[PAIR ? 1 : GPW][4], b[PAIR ? 1 : GPW][4];
  if constexpr (!PAIR) {
#pragma unroll
    for (int g = 0; g < GPW; ++g) {
      const int n = (g0 + g) * kTileN + (lane >> 4) * 4;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[g][r] = n + r < a.N ? a.scale[n + r] : 0.f;
        b[g][r] = (a.bias && n + r < a.N) ? a.bias[n + r] : 0.f;
      }
    }
  }
  // finished values of channel group g, row block rb (PAIR: the scales of the
  // second matrix follow those of the first; a.N is a multiple of 16)
  auto finished = [&](int g, int rb, float step) {
    float4 o;
    if constexpr (PAIR) {
      const float4 sc = *reinterpret_cast<const float4 *>(
          epi_s + (wave >> 1) * (kEpiScales / 2) + ((wave & 1) * GPW + g) * kTileN +
          (lane >> 4) * 4);
      o.x = scaled<D>(combine<D>(acc[g][rb], 0), step, sc.x);
      o.y = scaled<D>(combine<D>(acc[g][rb], 1), step, sc.y);
      o.z = scaled<D>(combine<D>(acc[g][rb], 2), step, sc.z);
      o.w = scaled<D>(combine<D>(acc[g][rb], 3), step, sc.w);
    } else {
      o.x = b[g][0] + scaled<D>(combine<D>(acc[g][rb], 0), step, s[g][0]);
      o.y = b[g][1] + scaled<D>(combine<D>(acc[g][rb], 1), step, s[g][1]);
      o.z = b[g][2] + scaled<D>(combine<D>(acc[g][rb], 2), step, s[g][2]);
      o.w = b[g][3] + scaled<D>(combine<D>(acc[g][rb], 3), step, s[g][3]);
    }
    return o;
  };
  // PAIR: the wavefronts of the first matrix finish the upper row blocks of the
  // tile, those of the second the lower ones (each stores half as much as an
  // unpaired wavefront): what a wavefront computed of the other's row blocks
  // crosses over through LDS, same lane, same registers
  constexpr int kUpper = (RB + 1) / 2;
  const bool second = PAIR && wave >= 2;
  float4 *cross = reinterpret_cast<float4 *>(reinterpret_cast<float *>(frag_s) +
                                             kSlices * 16 * kPad);
  if constexpr (PAIR) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      if (second ? rb >= kUpper : rb < kUpper)
        continue; // stays here
      const float step = epi_s[kEpiScales + rb * 16 + (lane & 15)];
      const int slot = rb < kUpper ? rb : rb - kUpper;
#pragma unroll
      for (int g = 0; g < GPW; ++g)
        cross[((wave * kUpper + slot) * GPW + g) * kWave + lane] = finished(g, rb, step);
    }
    __syncthreads();
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    if (PAIR && (second ? rb < kUpper : rb >= kUpper))
      continue; // the partner wavefront finishes this row block
    const int mr = m0 + rb * 16 + (lane & 15);
    float step;
    if constexpr (PAIR)
      step = epi_s[kEpiScales + rb * 16 + (lane & 15)];
    else
      step = mr < a.M ? a.steps[mr] : 0.f;
#pragma unroll
    for (int g = 0; g < GPW; ++g) {
      float4 o = finished(g, rb, step);
      if constexpr (PAIR) {
        const int slot = rb < kUpper ? rb : rb - kUpper;
        const float4 p = cross[(((wave ^ 2) * kUpper + slot) * GPW + g) * kWave + lane];
        const float4 gate = second ? p : o, up = second ? o : p;
        o = make_float4(silu_times(gate.x, up.x), silu_times(gate.y, up.y),
                        silu_times(gate.z, up.z), silu_times(gate.w, up.w));
      }
      *reinterpret_cast<float4 *>(tile + (lane & 15) * kPad + g * 16 + (lane >> 4) * 4) = o;
    }
#pragma unroll
    for (int i = 0; i < GPW; ++i) { // 16 rows x 4 GPW float4 = 64 GPW lanes' worth
      const int idx = lane + 64 * i;
      const int row = idx / (GPW * 4), c4 = idx % (GPW * 4);
      const float4 o = *reinterpret_cast<const float4 *>(tile + row * kPad + c4 * 4);
      const int m = m0 + rb * 16 + row, n = n0 + c4 * 4;
      if (m >= a.M || n >= a.N)
        continue;
      float *c = a.C + (int64_t)m * a.ldc + n;
      if (vec && n + 3 < a.N) {
        float4 q = o;
        if (a.accumulate) {
          const float4 p = *reinterpret_cast<const float4 *>(c);
          q = make_float4(p.x + q.x, p.y + q.y, p.z + q.z, p.w + q.w);
        }
        *reinterpret_cast<float4 *>(c) = q;
      } else {
        const float v[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < a.N)
            c[r] = a.accumulate ? c[r] + v[r] : v[r];
      }
    }
    if constexpr (D == 1) {
      if (a.sums) { // the same turn for the integer sums, carried as float bit patterns
#pragma unroll
        for (int g = 0; g < GPW; ++g)
          *reinterpret_cast<float4 *>(tile + (lane & 15) * kPad + g * 16 + (lane >> 4) * 4) =
              make_float4(__int_as_float(acc[g][rb][0][0]), __int_as_float(acc[g][rb][0][1]),
                          __int_as_float(acc[g][rb][0][2]), __int_as_float(acc[g][rb][0][3]));
        const bool ivec = (a.N & 3) == 0 && (reinterpret_cast<uintptr_t>(a.sums) & 15) == 0;
#pragma unroll
        for (int i = 0; i < GPW; ++i) {
          const int idx = lane + 64 * i;
          const int row = idx / (GPW * 4), c4 = idx % (GPW * 4);
          const float4 q = *reinterpret_cast<const float4 *>(tile + row * kPad + c4 * 4);
          const v4i32 o = {__float_as_int(q.x), __float_as_int(q.y), __float_as_int(q.z),
                           __float_as_int(q.w)};
          const int m = m0 + rb * 16 + row, n = n0 + c4 * 4;
          if (m >= a.M || n >= a.N)
            continue;
          int32_t *c = a.sums + (int64_t)m * a.N + n;
          if (ivec) {
            *reinterpret_cast<v4i32 *>(c) = o;
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (n + r < a.N)
                c[r] = o[r];
          }
        }
      }
    }
  }
}

// Sum of a float4 over the K slices, in slice order, four loads in flight at a
// time (slices past the end repeat the last one and are not added).
__device__ __forceinline__ void sum_slices(const float *p, size_t slice_stride, int slices,
                                           float (&v)[4]) {
  v[0] = v[1] = v[2] = v[3] = 0.f;
  for (int sl = 0; sl < slices; sl += 4) {
    float4 q[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      q[u] = *reinterpret_cast<const float4 *>(p + (size_t)min(sl + u, slices - 1) * slice_stride);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (sl + u < slices) {
        v[0] += q[u].x; v[1] += q[u].y; v[2] += q[u].z; v[3] += q[u].w;
      }
  }
}

// What finishes four neighbouring outputs: scales, bias and (accumulating) the old
// values, asked for in one go before the slices are summed -- loaded at their
// use, each was an L2 round trip of its own behind the sum.
struct FinishOperands {
  float scale[4], bias[4], old[4];
};
__device__ __forceinline__ FinishOperands load_finish_operands(const GemmI8Args &a, const float *c,
                                                              int n) {
  FinishOperands f;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const bool in = n + r < a.N;
    f.scale[r] = in ? a.scale[n + r] : 0.f;
    f.bias[r] = (in && a.bias) ? a.bias[n + r] : 0.f;
    f.old[r] = (in && a.accumulate) ? c[r] : 0.f;
  }
  return f;
}

// C (+)= step[m] * scale[n] * sum over slices of the unscaled sums, slice order.
__global__ void __launch_bounds__(256)
reduce_slices_kernel(GemmI8Args a, int rb_per_tile, int gpw) {
  const int n4 = (a.N + 3) / 4;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)a.M * n4)
    return;
  const int m = (int)(i / n4), n = (int)(i % n4) * 4;
  const int span = 16 * gpw; // channels per wavefront
  const int rbk = m / (16 * rb_per_tile), rb = (m / 16) % rb_per_tile, row = m % 16;
  const int col = n / (kSlices * span), wave = (n / span) % kSlices, ch = n % span;
  const int sub = 16 * span;
  const size_t slice_stride = (size_t)kSlices * rb_per_tile * sub;
  const float *p = a.partial + ((size_t)(rbk * a.ncols + col) * a.slices) * slice_stride +
                   ((size_t)wave * rb_per_tile + rb) * sub + row * span + ch;
  const float step = a.steps[m];
  float *c = a.C + (int64_t)m * a.ldc + n;
  const FinishOperands f = load_finish_operands(a, c, n);
  float v[4];
  sum_slices(p, slice_stride, a.slices, v);
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (n + r < a.N) {
      const float o = f.bias[r] + (v[r] * step) * f.scale[r];
      c[r] = a.accumulate ? f.old[r] + o : o;
    }
}

// One plane (the w8a8 matmul): the slices hold int32 sums, added exactly; then
// C = f32(sum) * (step * scale[n]) in that order (linalg.py:12833-12845), and the
// sums themselves where the caller asked for them.
__global__ void __launch_bounds__(256)
reduce_slices_i32_kernel(GemmI8Args a, int rb_per_tile, int gpw) {
  const int n4 = (a.N + 3) / 4;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)a.M * n4)
    return;
  const int m = (int)(i / n4), n = (int)(i % n4) * 4;
  const int span = 16 * gpw;
  const int rbk = m / (16 * rb_per_tile), rb = (m / 16) % rb_per_tile, row = m % 16;
  const int col = n / (kSlices * span), wave = (n / span) % kSlices, ch = n % span;
  const int sub = 16 * span;
  const size_t slice_stride = (size_t)kSlices * rb_per_tile * sub;
  const float *p = a.partial + ((size_t)(rbk * a.ncols + col) * a.slices) * slice_stride +
                   ((size_t)wave * rb_per_tile + rb) * sub + row * span + ch;
  int v[4] = {0, 0, 0, 0};
  for (int sl = 0; sl < a.slices; sl += 4) {
    v4i32 q[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      q[u] = *reinterpret_cast<const v4i32 *>(p + (size_t)min(sl + u, a.slices - 1) * slice_stride);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (sl + u < a.slices) {
        v[0] += q[u][0]; v[1] += q[u][1]; v[2] += q[u][2]; v[3] += q[u][3];
      }
  }
  const float step = a.steps[m];
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (n + r < a.N) {
      a.C[(int64_t)m * a.ldc + n + r] = scaled<1>((float)v[r], step, a.scale[n + r]);
      if (a.sums)
        a.sums[(int64_t)m * a.N + n + r] = v[r];
    }
}

// The same, one workgroup per row, which then holds the finished row and goes on
// to write RMSNorm(row) * w as the digit planes of the next matmul's input (what
// rmsnorm_to_digits_kernel would read back from C): lds = [Kp2] cache of
// row_to_digits, then [Kp2] the row.
__global__ void __launch_bounds__(kRowThreads)
reduce_slices_norm_kernel(const float *p_partial, const float *p_steps, int p_N, int p_ncols,
                          int p_slices, int rb_per_tile, int gpw, GemmI8Args rest,
                          const float *__restrict__ norm_w, float inv_n, float eps, int D,
                          int Mp2, int Kp2, int8_t *__restrict__ planes) {
  GemmI8Args a = rest; // the leading parameters arrive in SGPRs, ahead of the first load
  a.partial = const_cast<float *>(p_partial);
  a.steps = p_steps;
  a.N = p_N;
  a.ncols = p_ncols;
  a.slices = p_slices;
  __shared__ float red[kRowThreads / 64];
  extern __shared__ __attribute__((aligned(16))) float row_lds[];
  float *xrow = row_lds + Kp2;
  const int m = blockIdx.x;
  const int n4 = (a.N + 3) / 4;
  const int span = 16 * gpw;
  const int rbk = m / (16 * rb_per_tile), rb = (m / 16) % rb_per_tile, row = m % 16;
  const int sub = 16 * span;
  const size_t slice_stride = (size_t)kSlices * rb_per_tile * sub;
  const float step = a.steps[m];
  for (int q4 = threadIdx.x; q4 < n4; q4 += kRowThreads) {
    const int n = q4 * 4;
    const int col = n / (kSlices * span), wave = (n / span) % kSlices, ch = n % span;
    const float *p = a.partial + ((size_t)(rbk * a.ncols + col) * a.slices) * slice_stride +
                     ((size_t)wave * rb_per_tile + rb) * sub + row * span + ch;
    float *c = a.C + (int64_t)m * a.ldc + n;
    const FinishOperands f = load_finish_operands(a, c, n);
    float v[4];
    sum_slices(p, slice_stride, a.slices, v);
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (n + r < a.N) {
        float o = f.bias[r] + (v[r] * step) * f.scale[r];
        if (a.accumulate)
          o += f.old[r];
        c[r] = o;
        xrow[n + r] = o;
      }
  }
  __syncthreads();
  float s = 0.f;
  for (int i = threadIdx.x; i < a.N; i += kRowThreads)
    s = fmaf(xrow[i], xrow[i], s);
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0)
    red[threadIdx.x >> 6] = s;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < kRowThreads / 64; w += 2)
    tot += red[w] + red[w + 1];
  const float rs = 1.0f / sqrtf(tot * inv_n + eps);
  row_to_digits(NormRow{xrow, norm_w, rs, a.N}, a.N, m, D, Mp2, Kp2, planes, red, row_lds);
}

BH_VARIANT_FAMILY(WideFamily, "gemm_w8_i8_wide_kernel");
BH_VARIANT_FAMILY(SplitFamily, "gemm_w8_i8_kernel");

template <int D, int RB, int GPW, bool PAIR = false>
int launch_wide(const GemmI8Args &a, unsigned blocks, hipStream_t stream) {
  constexpr size_t lds = wide_lds_bytes<D, RB, GPW, PAIR>();
  auto kernel = gemm_w8_i8_wide_kernel<D, RB, GPW, PAIR>;
  if (lds > 48 * 1024) {
    static DynLdsOnce dyn_lds;
    BH_CHECK_HIP(ensure_dyn_lds(dyn_lds, reinterpret_cast<const void *>(kernel),
                                (int)lds));
  }
  BH_NOTE_VARIANT(WideFamily, D, RB, GPW, (int)PAIR);
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kSlices * kWave), lds, stream, a.planes, a.W, a.Mp,
                     a.Kp, a.groups, a.chunks, a.ncols, a.cols_padded, a.slices, a.chunks_per_slice,
                     a);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace

namespace {
size_t row_cache_bytes(int cols_padded) {
  return cols_padded <= kRowCache ? sizeof(float) * (size_t)cols_padded : 0;
}
} // namespace

int launch_activations_to_digits(const float *A, int64_t lda, int64_t M, int64_t K,
                                 int digits, void *staged, hipStream_t stream) {
  BH_REQUIRE(A && staged && M > 0 && K > 0 && digits >= 2 && digits <= 3 && lda >= K,
             "activations_to_digits: bad argument");
  const GemmStagingLayout l = gemm_staging_layout(M, K);
  hipLaunchKernelGGL(activations_to_digits_kernel, dim3((unsigned)l.rows_padded), dim3(kRowThreads),
                     row_cache_bytes(l.cols_padded), stream, A, lda, (int)M, (int)K, digits, l.rows_padded,
                     l.cols_padded, static_cast<int8_t *>(staged));
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_rmsnorm_to_digits(const float *x, int64_t ldx, const float *w, int rows, int n,
                             float eps, int digits, void *staged, hipStream_t stream) {
  BH_REQUIRE(x && w && staged && rows > 0 && n > 0 && ldx >= n && digits >= 2 && digits <= 3,
             "rmsnorm_to_digits: bad argument");
  const GemmStagingLayout l = gemm_staging_layout(rows, n);
  hipLaunchKernelGGL(rmsnorm_to_digits_kernel, dim3(rows), dim3(kRowThreads),
                     row_cache_bytes(l.cols_padded), stream, x, ldx, w, n,
                     1.0f / (float)n, eps, digits, l.rows_padded, l.cols_padded,
                     static_cast<int8_t *>(staged));
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_silu_mul_to_digits(const float *g, const float *u, int64_t ld, int rows, int n,
                              int digits, void *staged, hipStream_t stream) {
  BH_REQUIRE(g && u && staged && rows > 0 && n > 0 && ld >= n && digits >= 2 && digits <= 3,
             "silu_mul_to_digits: bad argument");
  const GemmStagingLayout l = gemm_staging_layout(rows, n);
  hipLaunchKernelGGL(silu_mul_to_digits_kernel, dim3(rows), dim3(kRowThreads),
                     row_cache_bytes(l.cols_padded), stream, g, u, ld, n,
                     digits, l.rows_padded, l.cols_padded, static_cast<int8_t *>(staged));
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

namespace {

// Split-K workspace: one grow-only device buffer per stream (calls on one stream
// are ordered; calls on different streams must not share it).
struct Workspace {
  char *ptr = nullptr;
  size_t bytes = 0;
};
std::mutex g_workspace_mutex;
std::map<hipStream_t, Workspace> g_workspace;

int workspace_for(hipStream_t stream, size_t bytes, char **out) {
  std::lock_guard<std::mutex> lock(g_workspace_mutex);
  Workspace &w = g_workspace[stream];
  if (w.bytes < bytes) {
    if (w.ptr) {
      BH_CHECK_HIP(hipStreamSynchronize(stream)); // an earlier matmul may still use it
      BH_CHECK_HIP(hipFree(w.ptr));
      w.ptr = nullptr;
      w.bytes = 0;
    }
    BH_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&w.ptr), bytes));
    w.bytes = bytes;
  }
  *out = w.ptr;
  return BUDDY_HIP_OK;
}

template <int D> int launch_split(const GemmI8Args &a, unsigned blocks, hipStream_t stream) {
  constexpr size_t lds = sizeof(float) * kSlices * 64 * kWave;
  auto kernel = gemm_w8_i8_kernel<D>;
  static DynLdsOnce dyn_lds;
  BH_CHECK_HIP(ensure_dyn_lds(dyn_lds, reinterpret_cast<const void *>(kernel),
                              (int)lds));
  BH_NOTE_VARIANT(SplitFamily, D);
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kSlices * kWave), lds, stream, a.planes, a.W, a.Mp,
                     a.Kp, a.groups, a.chunks, a.ncols, a.cols_padded, a.slices, a.chunks_per_slice,
                     a);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

template <int D, bool PAIR = false>
int launch_shape(int rb, int gpw, const GemmI8Args &a, unsigned blocks, hipStream_t stream) {
  switch (rb * 10 + gpw) {
  case 34: return launch_wide<D, 3, 4, PAIR>(a, blocks, stream);
  case 35: return launch_wide<D, 3, 5, PAIR>(a, blocks, stream);
  case 44: return launch_wide<D, 4, 4, PAIR>(a, blocks, stream);
  default: return launch_wide<D, 4, 5, PAIR>(a, blocks, stream);
  }
}

} // namespace

void release_gemm_i8_workspace(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_workspace_mutex);
  auto it = g_workspace.find(stream);
  if (it == g_workspace.end())
    return;
  if (it->second.ptr) {
    (void)hipStreamSynchronize(stream);
    (void)hipFree(it->second.ptr);
  }
  g_workspace.erase(it);
}

// `planes` holds the digit planes and row steps of the activations (written by
// one of the producers above for exactly this M, K and digit count).
namespace {
template <int D>
int launch_gemm_w8_digits_d(const GemmW8Args &in, const void *planes, hipStream_t stream) {
  GemmI8Args a;
  const GemmStagingLayout layout = gemm_staging_layout(in.M, in.K);
  a.Mp = layout.rows_padded;
  a.Kp = layout.cols_padded;
  a.planes = static_cast<const int8_t *>(planes);
  a.steps = reinterpret_cast<const float *>(a.planes + (size_t)in.digits * a.Mp * a.Kp);
  a.W = reinterpret_cast<const int4 *>(in.W);
  a.scale = in.scale;
  a.bias = in.bias;
  a.C = in.C;
  a.ldc = in.ldc;
  a.M = (int)in.M;
  a.N = (int)in.N;
  a.groups = (int)ceil_div(in.N, kTileN);
  a.chunks = (int)ceil_div(in.K, kTileK);
  a.accumulate = in.accumulate ? 1 : 0;
  a.partial = nullptr;
  a.sums = nullptr;
  a.int_partials = 0;
  a.slices = 1;
  if (in.silu_pair) {
    // two matrices of N / 2 channels, result SiLU(first) * second: wide tiles of
    // 32 GPW channels of both, whole K per workgroup
    BH_REQUIRE(!in.then_norm_w, "gemm_w8: no norm after the SiLU pair");
    BH_REQUIRE(in.N % (2 * kTileN) == 0 && !in.accumulate && !in.bias,
               "gemm_w8: the SiLU pair needs two matrices of a multiple of 16 channels, no "
               "bias, no accumulation");
    a.N = (int)(in.N / 2);
    a.chunks_per_slice = a.chunks;
    const int half_groups = a.groups / 2;
    int best_gpw = 0, best_rb = 0;
    double best_cost = 0;
    for (int gpw : {5, 4})
      for (int rb : {4, 3}) {
        const int64_t ncols = ceil_div(half_groups, 2 * gpw), rows = ceil_div(in.M, 16 * rb);
        const int64_t per_xcd = ceil_div(ncols, 8) * rows;
        const double wg = 0.0125 * (double)(a.chunks * gpw * rb * in.digits) + 7.0;
        const double cost = (double)ceil_div(per_xcd, 32) * wg;
        if (!best_gpw || cost < best_cost - 1e-9) {
          best_gpw = gpw;
          best_rb = rb;
          best_cost = cost;
        }
      }
    a.ncols = (int)ceil_div(half_groups, 2 * best_gpw);
    a.cols_padded = (int)round_up((int64_t)a.ncols, 8);
    const int row_tiles = (int)ceil_div(in.M, 16 * best_rb);
    return launch_shape<D, true>(best_rb, best_gpw, a, (unsigned)(a.cols_padded * row_tiles),
                                 stream);
  }
  // Three schemes, chosen by a model of their cost in microseconds (fitted to
  // measurements at the Qwen2-1.5B shapes and M = 512):
  //  * wide tiles, whole K per workgroup: the chip runs 256 workgroups at a time
  //    (one wavefront per SIMD); a workgroup costs its matrix instructions
  //    (12.5 ns each per SIMD, sustained) plus about 7 us of pipeline fill, drain
  //    and stores; a launch costs rounds x that;
  //  * wide tiles with K split over s workgroups: 2 us more per workgroup for the
  //    partial sums, and the second kernel (3 us + its bytes at 3 TB/s);
  //  * 64 x 64 tiles, K split over the wavefronts: bound by L2 -> CU traffic,
  //    16 KiB per workgroup and chunk at about 6 TB/s.
  // A norm that is to follow (then_norm_w) costs a launch of its own, about
  // 5 us, unless the kernel that adds K slices writes its planes (it holds whole
  // rows, up to kRowCache columns).
  const double pending_norm = in.then_norm_w ? 5.0 : 0.0;
  const bool slices_fuse_norm = gemm_staging_layout(in.M, in.N).cols_padded <= kRowCache;
  int best_gpw = 0, best_rb = 0, best_s = 0;
  double best_cost = 0;
  for (int gpw : {5, 4})
    for (int rb : {4, 3}) {
      const int64_t ncols = ceil_div(a.groups, gpw * kSlices), rows = ceil_div(in.M, 16 * rb);
      for (int s = 1; s <= 16; ++s) {
        // workgroups of the busiest XCD (32 CUs each): the (column tile, slice)
        // pairs are dealt round robin, each with all its row tiles
        const int64_t per_xcd = ceil_div(ncols * s, 8) * rows;
        if (s > 1 && per_xcd > 32)
          break;
        const int64_t cps = ceil_div(a.chunks, s);
        if (ceil_div(a.chunks, cps) != s)
          continue; // the last slice would be empty
        // (with the whole K in one workgroup a chunk of the pipelined loop takes
        // 0.55 us however few matrix instructions it holds -- its barrier, staging
        // and waits: 512 x 1536 x 2048 on two planes as 88 tiles of 48 x 256 took
        // 19.4 us where 24 x 0.3 + 7 would be 14.2)
        const double chunk_us =
            std::max(0.0125 * (double)(gpw * rb * in.digits), s == 1 ? 0.55 : 0.0);
        const double wg = chunk_us * (double)cps + 7.0 + (s > 1 ? 2.0 : 0.0);
        double cost = (double)ceil_div(per_xcd, 32) * wg;
        if (s > 1)
          cost += 3.0 + 4.0 * (double)(ncols * rows * s) * (kSlices * rb * 16 * gpw * 16) / 3e6;
        if (s == 1 || !slices_fuse_norm)
          cost += pending_norm;
        if (!best_gpw || cost < best_cost - 1e-9) {
          best_gpw = gpw;
          best_rb = rb;
          best_s = s;
          best_cost = cost;
        }
      }
    }
  // the RMSNorm of the finished rows into digit planes, where the caller asked
  // for it and no kernel of the matmul holds whole rows
  auto then_norm = [&]() -> int {
    if (!in.then_norm_w)
      return BUDDY_HIP_OK;
    return launch_rmsnorm_to_digits(in.C, in.ldc, in.then_norm_w, (int)in.M, (int)in.N,
                                    in.then_norm_eps, in.digits, in.then_norm_staged, stream);
  };
  // The 64 x 64 kernel: two workgroups fit a compute unit, and a workgroup takes
  // about 6 us for its first chunk per wavefront and 2 us for every further one
  // (measured: 17.3 us for q|k|v, 18.6 us for o_proj at 512 rows, 72 us for
  // down).  Neither it nor the unsplit wide kernel holds whole rows, so a norm
  // that is to follow costs them a launch of its own.
  const int64_t split_wgs = ceil_div(a.groups, kSplitGroups) * (a.Mp / 64);
  const double split_cost =
      1.0 + (double)ceil_div(split_wgs, 512) * (6.2 + 2.0 * (double)(ceil_div(a.chunks, kSlices) - 1)) +
      pending_norm;
  if (split_cost < best_cost) {
    a.ncols = (int)ceil_div(a.groups, kSplitGroups);
    a.cols_padded = (int)round_up(a.ncols, 8);
    const unsigned blocks = (unsigned)(a.cols_padded * (a.Mp / 64));
    if (int rc = launch_split<D>(a, blocks, stream))
      return rc;
    return then_norm();
  }
  a.ncols = (int)ceil_div(a.groups, best_gpw * kSlices);
  a.cols_padded = (int)round_up((int64_t)a.ncols * best_s, 8);
  const int row_tiles = (int)ceil_div(in.M, 16 * best_rb);
  a.slices = best_s;
  a.chunks_per_slice = (int)ceil_div(a.chunks, best_s);
  if (best_s > 1) {
    const size_t tile_floats = (size_t)kSlices * best_rb * 16 * best_gpw * 16;
    const size_t bytes = sizeof(float) * tile_floats * best_s * (size_t)a.ncols * row_tiles;
    char *ws = nullptr;
    if (int rc = workspace_for(stream, bytes, &ws))
      return rc;
    a.partial = reinterpret_cast<float *>(ws);
  }
  const unsigned blocks = (unsigned)(a.cols_padded * row_tiles);
  int rc = launch_shape<D>(best_rb, best_gpw, a, blocks, stream);
  if (rc)
    return rc;
  if (best_s == 1)
    return then_norm();
  const GemmStagingLayout next = gemm_staging_layout(in.M, in.N);
  if (in.then_norm_w && slices_fuse_norm) {
    // the kernel that adds the slices holds whole rows: it writes the planes too
    const size_t row_lds = 2 * sizeof(float) * (size_t)next.cols_padded;
    if (row_lds > 48 * 1024) { // up to 96 KiB at kRowCache columns
      static DynLdsOnce dyn_lds;
      BH_CHECK_HIP(ensure_dyn_lds(dyn_lds,
                                  reinterpret_cast<const void *>(reduce_slices_norm_kernel),
                                  (int)(2 * sizeof(float) * kRowCache)));
    }
    hipLaunchKernelGGL(reduce_slices_norm_kernel, dim3((unsigned)a.M), dim3(kRowThreads),
                       row_lds, stream, a.partial, a.steps, a.N, a.ncols, a.slices, best_rb,
                       best_gpw, a, in.then_norm_w, 1.0f / (float)in.N, in.then_norm_eps,
                       in.digits, next.rows_padded, next.cols_padded,
                       static_cast<int8_t *>(in.then_norm_staged));
    BH_CHECK_HIP(hipGetLastError());
    return BUDDY_HIP_OK;
  }
  const int64_t threads = (int64_t)a.M * ((a.N + 3) / 4);
  hipLaunchKernelGGL(reduce_slices_kernel, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0,
                     stream, a, best_rb, best_gpw);
  BH_CHECK_HIP(hipGetLastError());
  return then_norm();
}
} // namespace

int launch_gemm_w8_digits(const GemmW8Args &in, const void *planes, hipStream_t stream) {
  return in.digits == 2 ? launch_gemm_w8_digits_d<2>(in, planes, stream)
                        : launch_gemm_w8_digits_d<3>(in, planes, stream);
}

// The w8a8 matmul for more than 16 rows: `plane` holds the int8 activations as
// one plane ([rows_padded][cols_padded], zero padded) followed by the row steps,
// every one of them the per-tensor activation scale.  The int32 sums are exact
// whether K stays within one workgroup or is split over several (K <= 2^17:
// 2^17 * 127 * 128 is below 2^31).
int launch_gemm_w8a8_plane(const void *plane, const int8_t *W, const float *wscale, float *C,
                           int32_t *sums, int64_t M, int64_t K, int64_t N,
                           hipStream_t stream) {
  BH_REQUIRE(K <= (1 << 17), "w8a8 matmul: K=%lld above 131072", (long long)K);
  GemmI8Args a;
  const GemmStagingLayout layout = gemm_staging_layout(M, K);
  a.Mp = layout.rows_padded;
  a.Kp = layout.cols_padded;
  a.planes = static_cast<const int8_t *>(plane);
  a.steps = reinterpret_cast<const float *>(a.planes + (size_t)a.Mp * a.Kp);
  a.W = reinterpret_cast<const int4 *>(W);
  a.scale = wscale;
  a.bias = nullptr;
  a.C = C;
  a.ldc = N;
  a.M = (int)M;
  a.N = (int)N;
  a.groups = (int)ceil_div(N, kTileN);
  a.chunks = (int)ceil_div(K, kTileK);
  a.accumulate = 0;
  a.partial = nullptr;
  a.sums = sums;
  a.int_partials = 0;
  // the cost model of the digit-plane launch with one plane; K slices leave int32
  // sums in the workspace (f32 ones would round above 2^24) and a second kernel
  // adds them exactly
  int best_gpw = 0, best_rb = 0, best_s = 0;
  double best_cost = 0;
  const int64_t reduce_wgs = ceil_div(M * ceil_div(N, 4), 256);
  for (int gpw : {5, 4})
    for (int rb : {4, 3}) {
      const int64_t ncols = ceil_div(a.groups, gpw * kSlices), rows = ceil_div(M, 16 * rb);
      for (int s = 1; s <= 16; ++s) {
        const int64_t per_xcd = ceil_div(ncols * s, 8) * rows;
        if (s > 1 && per_xcd > 32)
          break;
        const int64_t cps = ceil_div(a.chunks, s);
        if (ceil_div(a.chunks, cps) != s)
          continue; // the last slice would be empty
        const double chunk_us = std::max(0.0125 * (double)(gpw * rb), s == 1 ? 0.55 : 0.0);
        const double wg = chunk_us * (double)cps + 7.0 + (s > 1 ? 2.0 : 0.0);
        double cost = (double)ceil_div(per_xcd, 32) * wg;
        if (s > 1)
          cost += 3.0 + 4.0 * (double)(ncols * rows * s) * (kSlices * rb * 16 * gpw * 16) / 3e6 +
                  0.002 * (double)reduce_wgs;
        if (!best_gpw || cost < best_cost - 1e-9) {
          best_gpw = gpw;
          best_rb = rb;
          best_s = s;
          best_cost = cost;
        }
      }
    }
  a.ncols = (int)ceil_div(a.groups, best_gpw * kSlices);
  a.cols_padded = (int)round_up((int64_t)a.ncols * best_s, 8);
  const int row_tiles = (int)ceil_div(M, 16 * best_rb);
  a.slices = best_s;
  a.chunks_per_slice = (int)ceil_div(a.chunks, best_s);
  if (best_s > 1) {
    const size_t tile_floats = (size_t)kSlices * best_rb * 16 * best_gpw * 16;
    const size_t bytes = sizeof(float) * tile_floats * best_s * (size_t)a.ncols * row_tiles;
    char *ws = nullptr;
    if (int rc = workspace_for(stream, bytes, &ws))
      return rc;
    a.partial = reinterpret_cast<float *>(ws);
    a.int_partials = 1;
  }
  if (int rc = launch_shape<1>(best_rb, best_gpw, a, (unsigned)(a.cols_padded * row_tiles), stream))
    return rc;
  if (best_s > 1) {
    hipLaunchKernelGGL(reduce_slices_i32_kernel, dim3((unsigned)reduce_wgs), dim3(256), 0, stream, a,
                       best_rb, best_gpw);
    BH_CHECK_HIP(hipGetLastError());
  }
  return BUDDY_HIP_OK;
}

} // namespace bh
