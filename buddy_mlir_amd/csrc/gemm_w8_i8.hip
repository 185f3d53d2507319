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
// The sums themselves are exact and do not depend on any order.  NaN and
// infinity do not survive the conversion to integers: the bf16 modes are the
// ones that propagate them.  |d q| <= 2^14, so K may not exceed 2^17.
//
// Digit planes lie like the bf16 terms do: [digit][row][k] int8, rows and k zero
// padded, followed by the row steps (f32 [rows_padded]).  A lane's operand is 16
// contiguous bytes of a plane row.
//
// Two workgroup shapes, as for bf16: 64 rows x 64 channels with K split over the
// four wavefronts (narrow matrices), and 64 or 48 rows x 256 channels with the
// activation fragments shared through LDS (wide matrices).
#include "gemm.h"

namespace bh {
namespace {

constexpr int kGroupsPerWave = 4; // channel groups of 16 per wavefront
constexpr int kSlices = 4;        // wavefronts per workgroup

typedef int v4i32 __attribute__((ext_vector_type(4)));

// ---- f32 rows -> digit planes ------------------------------------------------

// smallest power of two s (not below 2^-126) with mx / s < 2^(8 D - 2)
__device__ __forceinline__ float digit_step(float mx, int D) {
  const int ex = (int)((__float_as_uint(mx) >> 23) & 0xffu) - 127; // floor(log2 mx)
  const int e = max(ex + 1 - (8 * D - 2), -126);
  return __uint_as_float((unsigned)(e + 127) << 23);
}

struct PlainRow {
  const float *a;
  __device__ __forceinline__ float operator()(int k) const { return a[k]; }
};
struct NormRow { // w * (x * rs)
  const float *x, *w;
  float rs;
  __device__ __forceinline__ float operator()(int k) const { return w[k] * (x[k] * rs); }
};
struct SiluMulRow { // silu(g) * u
  const float *g, *u;
  __device__ __forceinline__ float operator()(int k) const {
    const float gv = g[k];
    const float sig = 1.0f / (1.0f + expf(-gv));
    return (gv * sig) * u[k];
  }
};

// One workgroup of 256 threads writes row `row` of every plane and its step.
template <class F>
__device__ __forceinline__ void row_to_digits(const F &f, int n, int row, int D, int Mp,
                                              int Kp, int8_t *planes, float *red) {
  float mx = 0.f;
  for (int k = threadIdx.x; k < n; k += 256)
    mx = fmaxf(mx, fabsf(f(k)));
  mx = wave_max(mx);
  __syncthreads(); // red may still be read by the caller's own reduction
  if ((threadIdx.x & 63) == 0)
    red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float step = digit_step(mx, D);
  const float inv = 1.0f / step; // a power of two as well
  float *steps = reinterpret_cast<float *>(planes + (size_t)D * Mp * Kp);
  if (threadIdx.x == 0)
    steps[row] = step;
  const size_t plane = (size_t)Mp * Kp;
  for (int k0 = threadIdx.x * 4; k0 < Kp; k0 += 256 * 4) {
    int X[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      X[e] = k0 + e < n ? (int)rintf(f(k0 + e) * inv) : 0;
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

__global__ void __launch_bounds__(256)
activations_to_digits_kernel(const float *__restrict__ A, int64_t lda, int M, int K, int D,
                             int Mp, int Kp, int8_t *__restrict__ planes) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  if (row >= M) { // padding rows: zero digits, step 1
    for (int j = 0; j < D; ++j)
      for (int k0 = threadIdx.x * 4; k0 < Kp; k0 += 256 * 4)
        *reinterpret_cast<unsigned *>(planes + ((size_t)j * Mp + row) * Kp + k0) = 0u;
    if (threadIdx.x == 0)
      reinterpret_cast<float *>(planes + (size_t)D * Mp * Kp)[row] = 1.0f;
    return;
  }
  row_to_digits(PlainRow{A + (int64_t)row * lda}, K, row, D, Mp, Kp, planes, red);
}

__global__ void __launch_bounds__(256)
rmsnorm_to_digits_kernel(const float *__restrict__ x, const float *__restrict__ w, int n,
                         float inv_n, float eps, int D, int Mp, int Kp,
                         int8_t *__restrict__ planes) {
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
  row_to_digits(NormRow{xr, w, rs}, n, row, D, Mp, Kp, planes, red);
}

__global__ void __launch_bounds__(256)
silu_mul_to_digits_kernel(const float *__restrict__ g, const float *__restrict__ u, int n,
                          int D, int Mp, int Kp, int8_t *__restrict__ planes) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  row_to_digits(SiluMulRow{g + (size_t)row * n, u + (size_t)row * n}, n, row, D, Mp, Kp,
                planes, red);
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
  int ncols, cols_padded; // column tiles; ids padded to the XCD count
  int accumulate;
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
  v4i32 w[kGroupsPerWave];
  v4i32 a[D][4]; // [digit][row block]
};

template <int D>
__device__ __forceinline__ void load_chunk(const v4i32 *const (&wp)[kGroupsPerWave],
                                           const int8_t *ap, size_t plane, size_t rb_stride,
                                           int c, ChunkOperands<D> &o) {
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g)
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
__global__ void __launch_bounds__(kSlices *kWave) gemm_w8_i8_kernel(GemmI8Args a) {
  extern __shared__ __attribute__((aligned(16))) float red[]; // [slice][64][lane]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = blockIdx.x % a.cols_padded, rbk = blockIdx.x / a.cols_padded;
  if (col >= a.ncols)
    return; // padding id
  const int m0 = rbk * 64, g0 = col * kGroupsPerWave;
  const int per = (a.chunks + kSlices - 1) / kSlices;
  const int c0 = min(wave * per, a.chunks), c1 = min(c0 + per, a.chunks);

  v4i32 acc[kGroupsPerWave][4][D];
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int j = 0; j < D; ++j)
        acc[g][rb][j] = v4i32{0, 0, 0, 0};

  const v4i32 *wp[kGroupsPerWave];
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g) // groups past the end repeat the last one
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
        for (int g = 0; g < kGroupsPerWave; ++g)
          acc[g][rb][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(cur.w[g], cur.a[j][rb],
                                                                acc[g][rb][j], 0, 0, 0);
    if (c + 1 < c1)
      cur = nxt;
  }

  float *mine = red + (size_t)wave * 64 * kWave;
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g)
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        mine[((g * 4 + rb) * 4 + r) * kWave + lane] = combine<D>(acc[g][rb], r);
  __syncthreads();
  const int g = wave; // wavefront w finishes channel group w
  if (g0 + g >= a.groups)
    return;
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
      v[r] = sum;
    }
    if (m >= a.M)
      continue;
    store_row(a, m, n, a.steps[m], v, s, b, vec);
  }
}

// Wide matrices: 16 RB rows x 256 channels per workgroup, one 64-channel span per
// wavefront, every wavefront runs the whole K.  Wavefront w fetches the digit
// fragments of row block w for everyone and leaves them in LDS in fragment order
// (lane l at 16 l: conflict-free).  Weights go from global memory to registers
// to the matrix core.
//
// Global loads run kRing - 2 chunks ahead of the matrix cores.  The compiler
// sinks ordinary loads down to their first use (and then waits for them there),
// so the loads of this loop are issued by hand and waited for by hand: a fetch
// is 4 + D loads in a fixed order, vmcnt counts them in order, and each wait
// names the registers it releases so that nothing reads them earlier.  The ring
// registers must never be spilled (a reload would read a register while its load
// is in flight): the build refuses scratch use in this file.
constexpr int kRing = 5;

__device__ __forceinline__ void issue_load(v4i32 &dst, const void *p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
template <int D> struct FetchRegs {
  v4i32 w[kGroupsPerWave];
  v4i32 a[D];
};
template <int N, int D> __device__ __forceinline__ void wait_loads(FetchRegs<D> &f) {
  static_assert(kGroupsPerWave == 4, "operand list below");
  asm volatile("s_waitcnt vmcnt(%4)"
               : "+v"(f.w[0]), "+v"(f.w[1]), "+v"(f.w[2]), "+v"(f.w[3])
               : "n"(N)
               : "memory");
#pragma unroll
  for (int j = 0; j < D; ++j)
    asm volatile("" : "+v"(f.a[j])::"memory");
}

template <int D, int RB>
__global__ void __launch_bounds__(kSlices *kWave) gemm_w8_i8_wide_kernel(GemmI8Args a) {
  constexpr int L = kGroupsPerWave + D; // loads per fetch
  extern __shared__ __attribute__((aligned(16))) v4i32 frag_s[]; // [2][D][RB][64]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = blockIdx.x % a.cols_padded, rbk = blockIdx.x / a.cols_padded;
  if (col >= a.ncols)
    return; // padding id
  const int m0 = rbk * RB * 16;
  const int g0 = (col * kSlices + wave) * kGroupsPerWave;

  v4i32 acc[kGroupsPerWave][RB][D];
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int j = 0; j < D; ++j)
        acc[g][rb][j] = v4i32{0, 0, 0, 0};

  const v4i32 *wp[kGroupsPerWave];
#pragma unroll
  for (int g = 0; g < kGroupsPerWave; ++g) // groups past the end repeat the last one
    wp[g] = reinterpret_cast<const v4i32 *>(a.W) +
            ((size_t)min(g0 + g, a.groups - 1) * a.chunks) * 64 + lane;
  const size_t plane = (size_t)a.Mp * a.Kp;
  // this wavefront fetches row block `wave` of the activation tile (with three
  // row blocks the fourth wavefront repeats the third's loads and stages nothing)
  const int my_rb = min(wave, RB - 1);
  const int8_t *ap = a.planes + (size_t)(m0 + my_rb * 16 + (lane & 15)) * a.Kp + (lane >> 4) * 16;

  FetchRegs<D> ring[kRing];
  // chunks past the end are fetched again from the last chunk (never used):
  // every fetch is exactly L loads, which is what keeps the counts below exact
  auto fetch = [&](int c, FetchRegs<D> &f) {
    const int cc = min(c, a.chunks - 1);
#pragma unroll
    for (int g = 0; g < kGroupsPerWave; ++g)
      issue_load(f.w[g], wp[g] + (size_t)cc * 64);
#pragma unroll
    for (int j = 0; j < D; ++j)
      issue_load(f.a[j], ap + j * plane + (size_t)cc * kTileK);
  };
  auto stage = [&](const FetchRegs<D> &f, int buf) { // own row block -> LDS
    if (wave >= RB)
      return;
#pragma unroll
    for (int j = 0; j < D; ++j)
      frag_s[(((size_t)buf * D + j) * RB + wave) * kWave + lane] = f.a[j];
  };
#pragma unroll
  for (int u = 0; u < kRing; ++u)
    fetch(u, ring[u]);
  wait_loads<(kRing - 1) * L, D>(ring[0]); // chunk 0 has arrived
  stage(ring[0], 0);
  __syncthreads();
  for (int c0 = 0; c0 < a.chunks; c0 += kRing) {
#pragma unroll
    for (int u = 0; u < kRing; ++u) {
      const int c = c0 + u;
      if (c < a.chunks) {
        const int buf = c & 1;
        FetchRegs<D> &cur = ring[u];
        FetchRegs<D> &nxt = ring[(u + 1) % kRing];
        // in flight: chunks c+1 .. c+kRing-1 (chunk c was waited for when it was
        // staged).  Release chunk c+1 and put its row block into the other
        // buffer, whose readers passed the barrier that closed chunk c-1.
        wait_loads<(kRing - 2) * L, D>(nxt);
        stage(nxt, buf ^ 1);
        // all fragments of the chunk first, one wait, then nothing but matrix
        // instructions (left alone the compiler reads two fragments at a time
        // and the matrix cores idle through every LDS round trip)
        v4i32 af[D][RB];
#pragma unroll
        for (int j = 0; j < D; ++j)
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
            af[j][rb] = frag_s[(((size_t)buf * D + j) * RB + rb) * kWave + lane];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < D; ++j)
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int g = 0; g < kGroupsPerWave; ++g)
              acc[g][rb][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(cur.w[g], af[j][rb],
                                                                    acc[g][rb][j], 0, 0, 0);
        // the matrix cores have read the registers of chunk c when the next
        // instruction issues: fetch the chunk kRing further on into them
        fetch(c + kRing, cur);
        __syncthreads();
      }
    }
  }
  // loads of the repeated last chunk may still be in flight: their registers
  // stay allocated until the wait is over
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int u = 0; u < kRing; ++u)
    wait_loads<0, D>(ring[u]);

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
        v[r] = combine<D>(acc[g][rb], r);
      store_row(a, m, n, a.steps[m], v, s, b, vec);
    }
  }
}

template <int D, int RB>
int launch_wide(const GemmI8Args &a, unsigned blocks, hipStream_t stream) {
  constexpr size_t lds = sizeof(v4i32) * 2 * D * RB * kWave;
  hipLaunchKernelGGL((gemm_w8_i8_wide_kernel<D, RB>), dim3(blocks), dim3(kSlices * kWave),
                     lds, stream, a);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

template <int D> int launch_split(const GemmI8Args &a, unsigned blocks, hipStream_t stream) {
  constexpr size_t lds = sizeof(float) * kSlices * 64 * kWave;
  auto kernel = gemm_w8_i8_kernel<D>;
  static bool attr_set = false;
  if (!attr_set) {
    BH_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kSlices * kWave), lds, stream, a);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace

int launch_activations_to_digits(const float *A, int64_t lda, int64_t M, int64_t K,
                                 int digits, void *staged, hipStream_t stream) {
  BH_REQUIRE(A && staged && M > 0 && K > 0 && digits >= 2 && digits <= 3 && lda >= K,
             "activations_to_digits: bad argument");
  const GemmStagingLayout l = gemm_staging_layout(M, K);
  hipLaunchKernelGGL(activations_to_digits_kernel, dim3((unsigned)l.rows_padded), dim3(256),
                     0, stream, A, lda, (int)M, (int)K, digits, l.rows_padded,
                     l.cols_padded, static_cast<int8_t *>(staged));
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_rmsnorm_to_digits(const float *x, const float *w, int rows, int n, float eps,
                             int digits, void *staged, hipStream_t stream) {
  BH_REQUIRE(x && w && staged && rows > 0 && n > 0 && digits >= 2 && digits <= 3,
             "rmsnorm_to_digits: bad argument");
  const GemmStagingLayout l = gemm_staging_layout(rows, n);
  hipLaunchKernelGGL(rmsnorm_to_digits_kernel, dim3(rows), dim3(256), 0, stream, x, w, n,
                     1.0f / (float)n, eps, digits, l.rows_padded, l.cols_padded,
                     static_cast<int8_t *>(staged));
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_silu_mul_to_digits(const float *g, const float *u, int rows, int n, int digits,
                              void *staged, hipStream_t stream) {
  BH_REQUIRE(g && u && staged && rows > 0 && n > 0 && digits >= 2 && digits <= 3,
             "silu_mul_to_digits: bad argument");
  const GemmStagingLayout l = gemm_staging_layout(rows, n);
  hipLaunchKernelGGL(silu_mul_to_digits_kernel, dim3(rows), dim3(256), 0, stream, g, u, n,
                     digits, l.rows_padded, l.cols_padded, static_cast<int8_t *>(staged));
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

// `planes` holds the digit planes and row steps of the activations (written by
// one of the producers above for exactly this M, K and digit count).
int launch_gemm_w8_digits(const GemmW8Args &in, const void *planes, hipStream_t stream) {
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
  // wide matrices: a workgroup per 64 (48) rows x 256 channels, no split of K
  const int wide_cols = (int)ceil_div(a.groups, kGroupsPerWave * kSlices);
  if ((int64_t)wide_cols * (a.Mp / 64) >= 200) {
    // the chip runs 256 workgroups at a time (one wavefront per SIMD), so the
    // time is rounds x rows; ties go to 64 rows
    const int64_t wg4 = wide_cols * ceil_div(in.M, 64), wg3 = wide_cols * ceil_div(in.M, 48);
    const bool three = ceil_div(wg3, 256) * 3 < ceil_div(wg4, 256) * 4;
    a.ncols = wide_cols;
    a.cols_padded = (int)round_up(wide_cols, 8);
    const unsigned wb = (unsigned)(a.cols_padded * ceil_div(in.M, three ? 48 : 64));
    if (three) {
      if (in.digits == 2)
        return launch_wide<2, 3>(a, wb, stream);
      return launch_wide<3, 3>(a, wb, stream);
    }
    if (in.digits == 2)
      return launch_wide<2, 4>(a, wb, stream);
    return launch_wide<3, 4>(a, wb, stream);
  }
  a.ncols = (int)ceil_div(a.groups, kGroupsPerWave);
  a.cols_padded = (int)round_up(a.ncols, 8);
  const unsigned blocks = (unsigned)(a.cols_padded * (a.Mp / 64));
  if (in.digits == 2)
    return launch_split<2>(a, blocks, stream);
  return launch_split<3>(a, blocks, stream);
}

} // namespace bh
