// gemv_w8a32_i8.hip -- the int8 dequant matmul for small batches (5..16 rows) on
// the int8 matrix cores.
//
// The reference has no kernel of its own for 1 < M <= 16 (its decode patterns
// fire for m == 1 only, DequantMatMulVectorizationDecode.cpp:212-217; the BLIS
// kernel of MatMulBlisVectorization.cpp:398-986 is the one vectorised kernel for
// M > 1).  Here the weights stream exactly as in the one-row kernel, from the same
// packed copy, and go into v_mfma_i32_16x16x64_i8 as they lie: a lane's 16 bytes
// of a 16-channel x 64-k tile are that instruction's operand, so the loop spends
// no instruction on a weight.  The f32 activations become fixed point for it, 64
// k at a time:
//   * a wavefront reads its 16 rows x 64 k of activations from L2 as whole
//     256-byte row pieces (four rows per load instruction) and turns them through
//     a private 4 KiB of LDS into operand order: lane l holds x[row l % 16][16
//     consecutive k].  (Reading them in operand order directly makes every load
//     instruction touch 64 cache lines; that, not the weight stream, then bounds
//     the kernel.)
//   * the four lanes of a row find the largest magnitude of the row's 64 values
//     and from it a power-of-two step s with |x| / s < 2^22;
//   * X = rint(x / s) is cut into three balanced int8 digits, X = d0 + 256 d1 +
//     65536 d2 (the bytes of X + 0x8080, the lower two with their top bit
//     flipped), and a byte transpose puts each digit plane into operand order;
//   * three matrix instructions per tile give exact int32 sums r0, r1, r2, and
//     acc += s * (r0 + 256 r1 + 65536 r2) in f32.
// The only rounding of a product is that of X: at most 2^-23 of the largest of
// the 64 activations it is summed with -- what an f32 sum of the same terms does
// when it adds the largest one.  A row whose chunk holds a NaN or an infinity
// gets a NaN step and with it NaN results, so non-finite activations still show.
//   * A wavefront converts a chunk once and uses it for SPAN channel groups.
//   * Up to 8 rows (T2): the 16 columns of the activation operand are 8 rows of
//     two consecutive tiles, so that one conversion serves two tiles; each tile's
//     weights are multiplied with the whole operand and a lane keeps the product
//     that belongs to its own tile (columns 0-7 the first, 8-15 the second); the
//     two halves are added at the end.
//   * k-slices of a workgroup meet in LDS in slice order.
//   * RMSNorm can be fused in: the norm weight multiplies the activation before
//     it is converted, each lane gathers the squares of what it loads, and the
//     row's rsqrt factor multiplies the finished sums.
#include "gemv_w8a32.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>

namespace bh {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kMaxWavesI8 = 8; // 512 threads: up to 256 registers per lane

struct I8Args {
  const float *A;
  const int4 *W0, *W1;
  const float *s0, *s1, *bias, *norm_w;
  float *C;
  int64_t lda, ldc;
  float norm_eps, norm_inv_k;
  int K, N, groups, chunks, spans; // spans = ceil(groups / SPAN)
  int GS, KS;                      // spans x k-slices of wavefronts per workgroup
  int rows;
  bool two_tiles; // up to 8 rows: the variant that converts two tiles at a time
  // 9..16 rows of a narrow matrix: two workgroups per span, rows 0..7 and 8..15,
  // each on the two-tile variant (neighbouring workgroup ids, so that the second
  // reads the weights while the first's requests have them on their way)
  bool row_split;
};

__device__ __forceinline__ float silu(float g) {
  const float sig = 1.0f / (1.0f + expf(-g));
  return g * sig;
}

// Largest magnitude of 16 values; a NaN among them gives NaN (v_maximum3_f32, the
// IEEE-754-2019 maximum, which does not drop NaNs the way fmaxf does).
__device__ __forceinline__ float max_magnitude(const float (&v)[16]) {
  float m = __builtin_fabsf(v[0]);
#pragma unroll
  for (int e = 1; e < 16; ++e)
    m = __builtin_elementwise_maximum(m, __builtin_fabsf(v[e]));
  return m;
}

// 16 values of one row -> this lane's operand of each of the three digit planes.
__device__ __forceinline__ void to_digits(const float (&x)[16], float inv, v4i (&d)[3]) {
  // x * inv + 1.5 * 2^23 is rounded to an integer by the addition itself and
  // leaves 0x4B400000 + X in the word
  constexpr float kMagic = 12582912.0f;
  constexpr int kBias = 0x8080 - 0x4B400000;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    unsigned y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      y[e] = (unsigned)(__float_as_int(fmaf(x[4 * q + e], inv, kMagic)) + kBias);
    // 4 x 4 byte transpose, three rows of it
    const unsigned ta = __builtin_amdgcn_perm(y[1], y[0], 0x05010400u);
    const unsigned tb = __builtin_amdgcn_perm(y[3], y[2], 0x05010400u);
    const unsigned tc = __builtin_amdgcn_perm(y[1], y[0], 0x00000602u);
    const unsigned td = __builtin_amdgcn_perm(y[3], y[2], 0x00000602u);
    d[0][q] = (int)(__builtin_amdgcn_perm(tb, ta, 0x05040100u) ^ 0x80808080u);
    d[1][q] = (int)(__builtin_amdgcn_perm(tb, ta, 0x07060302u) ^ 0x80808080u);
    d[2][q] = (int)__builtin_amdgcn_perm(td, tc, 0x05040100u);
  }
}

// acc += step * (r0 + 256 r1 + 65536 r2); step65536 = 65536 * step
__device__ __forceinline__ void combine(f32x4 &acc, const v4i &r0, const v4i &r1,
                                        const v4i &r2, float step, float step65536) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int u = r0[i] + (r1[i] << 8); // |r0| <= 2^20, |r1| <= 2^20: exact
    acc[i] = fmaf((float)r2[i], step65536, fmaf((float)u, step, acc[i]));
  }
}

// The loads of the main loop are issued and waited for by hand: the compiler
// sinks ordinary prefetch loads down to their first use and then waits for them
// there.  A fetch is a fixed number of loads in a fixed order, vmcnt counts them
// in order, and each wait names the registers it releases so that nothing reads
// them earlier.
__device__ __forceinline__ void issue_load(v4i &dst, const void *p) {
  asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void issue_load(f32x4 &dst, const void *p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}

template <int SPAN, bool DUAL, bool NORM, bool T2> struct FetchRegs {
  static constexpr int W = SPAN * (T2 ? 2 : 1); // weight tiles per matrix: [group][tile of the pair]
  v4i w0[W];
  v4i w1[DUAL ? W : 1];
  f32x4 x[4]; // k kcol .. kcol+3 of rows lane/16, 4 + lane/16, 8 + lane/16, 12 + lane/16
              // (T2: of rows lane/16, 4 + lane/16 of the first tile, then of the second)
  f32x4 nw[NORM ? 4 : 1];
};
template <int SPAN, bool DUAL, bool NORM, bool T2> constexpr int fetch_loads() {
  return SPAN * (T2 ? 2 : 1) * (DUAL ? 2 : 1) + 4 * (NORM ? 2 : 1);
}
// Fetches kept in flight: as many as fit in about 64 registers, two at least.
// Without the fused norm the kernels then stay within 128 registers (a compute
// unit holds 16 of their wavefronts); with it they take up to 147 (12).
template <int SPAN, bool DUAL, bool NORM, bool T2> constexpr int ring_depth() {
  constexpr int regs = 4 * SPAN * (T2 ? 2 : 1) * (DUAL ? 2 : 1) + 16 * (NORM ? 2 : 1);
  return 64 / regs < 2 ? 2 : 64 / regs;
}

// `c` counts chunks, or pairs of chunks with T2 (`upper`: this lane's operand
// column belongs to the pair's second tile).
template <int SPAN, bool DUAL, bool NORM, bool T2>
__device__ __forceinline__ void fetch_chunk(const I8Args &a, const int4 *w0, const int4 *w1,
                                            const size_t (&gofs)[SPAN],
                                            const float *const (&xrow)[4], int kcol,
                                            int kofs, int c, bool real, int upper,
                                            FetchRegs<SPAN, DUAL, NORM, T2> &o) {
  // a fetch past the end of the slice (issued only to keep the load counts
  // fixed, never used) reads the first tile of the matrix, which stays in cache:
  // a streaming load of a tile of its own would go to HBM again
  constexpr int TP = T2 ? 2 : 1;
  // the chunks of this fetch; a second tile past the end of the matrix repeats
  // the last one and meets zero digits
  const int ca = TP * c, cb = min(TP * c + 1, a.chunks - 1);
#pragma unroll
  for (int s = 0; s < SPAN; ++s)
#pragma unroll
    for (int t = 0; t < TP; ++t) {
      const size_t ofs = real ? gofs[s] + (size_t)(t ? cb : ca) * 64 : (size_t)0;
      issue_load(o.w0[s * TP + t], w0 + ofs);
      if (DUAL)
        issue_load(o.w1[DUAL ? s * TP + t : 0], w1 + ofs);
    }
  // activations: load q takes 256 bytes of each of rows 4q .. 4q+3 (this lane:
  // four k of one of them); clamped inside the row, what lies past the end of a
  // ragged row is zeroed when it is consumed (K is a multiple of four).  T2:
  // loads 0 and 1 take rows 0..7 of the first tile, loads 2 and 3 of the second.
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int tile = T2 ? ca + (q >> 1) : ca;
    issue_load(o.x[q], xrow[q] + min(tile * kTileK + kcol, a.K - 4));
  }
  if (NORM) { // norm weights in operand order: 16 consecutive k, the same for all rows
    const int k = (ca + (T2 ? upper : 0)) * kTileK + kofs;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      issue_load(o.nw[NORM ? q : 0], a.norm_w + min(k + 4 * q, a.K - 4));
  }
}

// Waits until at most N loads are in flight; the registers of `f` are valid only
// after it.
template <int N, int SPAN, bool DUAL, bool NORM, bool T2>
__device__ __forceinline__ void wait_fetch(FetchRegs<SPAN, DUAL, NORM, T2> &f) {
  asm volatile("s_waitcnt vmcnt(%4)"
               : "+v"(f.x[0]), "+v"(f.x[1]), "+v"(f.x[2]), "+v"(f.x[3])
               : "n"(N)
               : "memory");
#pragma unroll
  for (int s = 0; s < FetchRegs<SPAN, DUAL, NORM, T2>::W; ++s) {
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

constexpr int kTurnStride = 68;               // floats between rows of the turning area
constexpr int kTurnFloats = 16 * kTurnStride; // per wavefront

template <int EPI, int SPAN, bool NORM, bool T2>
__global__ void __launch_bounds__(kMaxWavesI8 *kWave, 3) // 3 wavefronts per SIMD at least
    gemv_w8a32_i8_kernel(I8Args a) {
  constexpr bool DUAL = (EPI == kEpiSiluMul);
  constexpr int NA = DUAL ? 2 * SPAN : SPAN; // accumulators per lane
  extern __shared__ __attribute__((aligned(16))) float red[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ksh = shift_of(a.KS);
  const int sl = wave >> ksh, ks = wave & (a.KS - 1);
  const int row_half = a.row_split ? blockIdx.x & 1 : 0;
  if (a.row_split) { // this workgroup's rows: the first eight or the rest
    a.A += (int64_t)row_half * 8 * a.lda;
    a.C += (int64_t)row_half * 8 * a.ldc;
    a.rows = row_half ? a.rows - 8 : 8;
  }
  const int span = (a.row_split ? blockIdx.x >> 1 : blockIdx.x) * a.GS + sl;
  const bool live = span < a.spans;
  const int g0 = (live ? span : 0) * SPAN;
  // what a wavefront's slice is cut from and a fetch brings: chunks, or pairs of
  // chunks with T2
  const int units = T2 ? (a.chunks + 1) / 2 : a.chunks;
  const int per = (units + a.KS - 1) >> ksh;
  const int c0 = min(ks * per, units), c1 = min(c0 + per, units);
  const int kg = lane >> 4;
  const int col = lane & 15;          // column of the activation operand
  const int m = T2 ? col & 7 : col;   // its batch row
  const int upper = T2 ? col >> 3 : 0; // T2: the column belongs to the pair's second tile

  f32x4 acc0[SPAN], acc1[DUAL ? SPAN : 1];
#pragma unroll
  for (int s = 0; s < SPAN; ++s) {
    acc0[s] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (DUAL)
      acc1[DUAL ? s : 0] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  float ss = 0.f;
  // groups past the end of the matrix repeat the last one (never stored)
  size_t gofs[SPAN];
#pragma unroll
  for (int s = 0; s < SPAN; ++s)
    gofs[s] = (size_t)min(g0 + s, a.groups - 1) * a.chunks * 64;
  const int4 *w0 = a.W0 + lane;
  const int4 *w1 = (DUAL ? a.W1 : a.W0) + lane;
  const float *xrow[4]; // rows past the batch repeat its last row (never stored)
#pragma unroll
  for (int q = 0; q < 4; ++q)
    xrow[q] = a.A + (int64_t)min(T2 ? (4 * q + kg) & 7 : 4 * q + kg, a.rows - 1) * a.lda;
  const int kcol = (lane & 15) * 4, kofs = kg * 16;
  // this wavefront's 16 x 64 activations on their way into operand order; rows
  // are 68 floats apart so that the 16 lanes of an operand read hit 64 banks
  float *xt = red + (size_t)wave * kTurnFloats;
  float *meet = red + (size_t)(a.GS * a.KS) * kTurnFloats;

  // Per-channel operands of the epilogue, requested before the stream starts so
  // that their latency hides behind it (they are older than every fetch, so the
  // counted waits cover them).
  // With four groups per wavefront the registers are worth more than the
  // latency, and they are loaded after the stream.
  constexpr bool EARLY = SPAN <= 2;
  const bool writer = live && ks == 0 && col < a.rows; // (T2: rows <= 8, the lower columns)
  float e_s0[SPAN][4], e_s1[SPAN][4], e_c[SPAN][4];
  auto load_epilogue = [&]() {
#pragma unroll
    for (int s = 0; s < SPAN; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = (g0 + s) * kTileN + kg * 4 + i;
        const bool in = writer && g0 + s < a.groups && n < a.N;
        e_s0[s][i] = in ? a.s0[n] : 0.f;
        e_s1[s][i] = (DUAL && in) ? a.s1[n] : 0.f;
        e_c[s][i] = 0.f;
        if (in && EPI == kEpiAccum)
          e_c[s][i] = a.C[(int64_t)m * a.ldc + n];
        if (in && EPI == kEpiStore && a.bias)
          e_c[s][i] = a.bias[n];
      }
  };
  if (EARLY)
    load_epilogue();

  constexpr int L = fetch_loads<SPAN, DUAL, NORM, T2>();
  constexpr int R = ring_depth<SPAN, DUAL, NORM, T2>(); // fetches in flight
  FetchRegs<SPAN, DUAL, NORM, T2> ring[R];
  // every fetch is exactly L loads, also one past the end of the slice, which
  // keeps the counts exact
  const int clast = max(c1 - 1, 0);
#pragma unroll
  for (int u = 0; u < R; ++u)
    fetch_chunk<SPAN, DUAL, NORM, T2>(a, w0, w1, gofs, xrow, kcol, kofs, min(c0 + u, clast),
                                      c0 + u < c1, upper, ring[u]);
  // the last fetch of the matrix may bring a ragged tile or (T2) no second tile
  const bool ragged = (a.K & (kTileK - 1)) != 0 || (T2 && (a.chunks & 1));
  const v4i zero = v4i{0, 0, 0, 0};
  for (int cb = c0; cb < c1; cb += R) {
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int c = cb + u;
      if (c >= c1)
        continue;
      FetchRegs<SPAN, DUAL, NORM, T2> &cur = ring[u];
      wait_fetch<(R - 1) * L, SPAN, DUAL, NORM, T2>(cur); // chunk c has arrived
      // rows 4q + kg, k kcol..kcol+3  ->  column col, k kofs..kofs+15
      if (ragged && c == units - 1) { // only the last chunk of a ragged row has a tail
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int tile = T2 ? 2 * c + (q >> 1) : c;
          const bool past = tile * kTileK + kcol >= a.K;
          *reinterpret_cast<f32x4 *>(xt + (4 * q + kg) * kTurnStride + kcol) =
              past ? f32x4{0.f, 0.f, 0.f, 0.f} : cur.x[q];
        }
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<f32x4 *>(xt + (4 * q + kg) * kTurnStride + kcol) = cur.x[q];
      }
      float xv[16];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const f32x4 t = *reinterpret_cast<const f32x4 *>(xt + col * kTurnStride + kofs + 4 * q);
        xv[4 * q] = t.x;
        xv[4 * q + 1] = t.y;
        xv[4 * q + 2] = t.z;
        xv[4 * q + 3] = t.w;
      }
      if (NORM) {
        float nv[16] = {cur.nw[0].x, cur.nw[0].y, cur.nw[0].z, cur.nw[0].w,
                        cur.nw[NORM ? 1 : 0].x, cur.nw[NORM ? 1 : 0].y, cur.nw[NORM ? 1 : 0].z, cur.nw[NORM ? 1 : 0].w,
                        cur.nw[NORM ? 2 : 0].x, cur.nw[NORM ? 2 : 0].y, cur.nw[NORM ? 2 : 0].z, cur.nw[NORM ? 2 : 0].w,
                        cur.nw[NORM ? 3 : 0].x, cur.nw[NORM ? 3 : 0].y, cur.nw[NORM ? 3 : 0].z, cur.nw[NORM ? 3 : 0].w};
#pragma unroll
        for (int e = 0; e < 16; ++e) { // past the end of a ragged row x is zero
          ss = fmaf(xv[e], xv[e], ss);
          xv[e] *= nv[e];
        }
      }
      // the row's step for these 64 k: the smallest power of two s (not below
      // 2^-126) with |x| / s < 2^22
      float mx = max_magnitude(xv);
      mx = __builtin_elementwise_maximum(mx, __shfl_xor(mx, 16, 64));
      mx = __builtin_elementwise_maximum(mx, __shfl_xor(mx, 32, 64));
      const unsigned mb = __float_as_uint(mx) & 0x7fffffffu;
      const int ex = (int)(mb >> 23) - 127; // floor(log2 max), -127 for zero and subnormals
      const int e2 = max(ex + 1 - 22, -126);
      const bool finite = mb < 0x7f800000u;
      const float step = finite ? __uint_as_float((unsigned)(e2 + 127) << 23)
                                : __uint_as_float(0x7fc00000u);
      const float inv = __uint_as_float((unsigned)(127 - e2) << 23);
      const float step65536 = step * 65536.0f;
      v4i d[3];
      to_digits(xv, inv, d);
      // the three exact sums of one weight tile with the operand; T2: of both
      // tiles of the pair, each lane keeping those of its own tile
      auto products = [&](const v4i *w, v4i &r0, v4i &r1, v4i &r2) {
        r0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[0], d[0], zero, 0, 0, 0);
        r1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[0], d[1], zero, 0, 0, 0);
        r2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[0], d[2], zero, 0, 0, 0);
        if constexpr (T2) {
          const v4i u0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[1], d[0], zero, 0, 0, 0);
          const v4i u1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[1], d[1], zero, 0, 0, 0);
          const v4i u2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[1], d[2], zero, 0, 0, 0);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            r0[i] = upper ? u0[i] : r0[i];
            r1[i] = upper ? u1[i] : r1[i];
            r2[i] = upper ? u2[i] : r2[i];
          }
        }
      };
      constexpr int TP = T2 ? 2 : 1;
#pragma unroll
      for (int s = 0; s < SPAN; ++s) {
        v4i r0, r1, r2;
        products(&cur.w0[s * TP], r0, r1, r2);
        combine(acc0[s], r0, r1, r2, step, step65536);
        if (DUAL) {
          products(&cur.w1[DUAL ? s * TP : 0], r0, r1, r2);
          combine(acc1[DUAL ? s : 0], r0, r1, r2, step, step65536);
        }
      }
      // the registers of chunk c are free: fetch the chunk R further on
      fetch_chunk<SPAN, DUAL, NORM, T2>(a, w0, w1, gofs, xrow, kcol, kofs, min(c + R, clast),
                                        c + R < c1, upper, cur);
    }
  }
  // repeated last chunks may still be in flight: the ring registers stay
  // allocated until they have landed (without these ties the compiler may put a
  // temporary of the code below into one of them before the wait, and the late
  // load would overwrite it)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int u = 0; u < R; ++u)
    wait_fetch<0, SPAN, DUAL, NORM, T2>(ring[u]);
  if (EARLY) {
    // nothing that depends on the epilogue operands moves above this point
#pragma unroll
    for (int s = 0; s < SPAN; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        asm volatile("" : "+v"(e_s0[s][i]));
        if (DUAL)
          asm volatile("" : "+v"(e_s1[s][i]));
        else
          asm volatile("" : "+v"(e_c[s][i]));
      }
  } else {
    load_epilogue();
  }
  if constexpr (T2) { // columns col and col + 8 hold the two tiles' shares of a row
#pragma unroll
    for (int s = 0; s < SPAN; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc0[s][i] += dpp_f<0x128>(acc0[s][i]); // row_ror:8
        if (DUAL)
          acc1[DUAL ? s : 0][i] += dpp_f<0x128>(acc1[DUAL ? s : 0][i]);
      }
    if (NORM)
      ss += dpp_f<0x128>(ss);
  }
  if (NORM) { // the four lanes that share a row hold different k
    ss = sum_rows(ss);
  }

  // ---- k-slices meet in LDS, in slice order --------------------------------
  constexpr int kPerWave = (NA * 4 + 1) * kWave; // floats per wavefront
  if (a.KS > 1) {
    float *mine = meet + (size_t)wave * kPerWave;
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
    // four slices at a time, all their reads in flight together (KS is a power
    // of two; with two slices the reads past them repeat the last and are dropped)
    float r[NA][4], rs = 0.f;
#pragma unroll
    for (int t = 0; t < NA; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        r[t][i] = 0.f;
    for (int q0 = 0; q0 < a.KS; q0 += 4) {
      float v[4][NA][4], vs[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float *o = meet + (size_t)(wave + min(q0 + j, a.KS - 1)) * kPerWave + lane;
#pragma unroll
        for (int t = 0; t < NA; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            v[j][t][i] = o[(t * 4 + i) * kWave];
        vs[j] = NORM ? o[NA * 4 * kWave] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool has = q0 + j < a.KS;
#pragma unroll
        for (int t = 0; t < NA; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            r[t][i] += has ? v[j][t][i] : 0.f;
        rs += has ? vs[j] : 0.f;
      }
    }
#pragma unroll
    for (int s = 0; s < SPAN; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc0[s][i] = r[s][i];
        if (DUAL)
          acc1[DUAL ? s : 0][i] = r[DUAL ? SPAN + s : 0][i];
      }
    if (NORM)
      ss = rs;
  }
  // lane holds batch row m and channels kg*4 .. kg*4+3 of each group
  if (!writer)
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
        const float v = acc0[s][i] * rn * e_s0[s][i];
        if (EPI == kEpiSiluMul)
          *c = silu(v) * (acc1[DUAL ? s : 0][i] * rn * e_s1[s][i]);
        else // the residual row (accumulate) or the bias (or 0)
          *c = e_c[s][i] + v;
      }
    }
  }
}

BH_VARIANT_FAMILY(I8Family, "gemv_w8a32_i8_kernel");

// Workgroups of `waves` wavefronts of this variant that one compute unit holds
// (asked of the runtime once per variant and size: it knows the registers the
// compiler used).
template <int EPI, int SPAN, bool NORM, bool T2> int workgroups_per_cu(int waves, size_t lds) {
  static int cached[kMaxWavesI8 + 1] = {};
  if (!cached[waves]) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &n, reinterpret_cast<const void *>(gemv_w8a32_i8_kernel<EPI, SPAN, NORM, T2>),
            waves * kWave, lds) != hipSuccess ||
        n < 1)
      n = 1;
    cached[waves] = n;
  }
  return cached[waves];
}

template <int EPI, int SPAN, bool NORM, bool T2>
int launch_kernel(I8Args ka, int ks_forced, hipStream_t stream) {
  constexpr int NA = (EPI == kEpiSiluMul) ? 2 * SPAN : SPAN;
  auto kernel = gemv_w8a32_i8_kernel<EPI, SPAN, NORM, T2>;
  static DynLdsOnce dyn_lds;
  BH_CHECK_HIP(ensure_dyn_lds(dyn_lds, reinterpret_cast<const void *>(kernel),
                              144 * 1024));
  auto lds_bytes = [&](int ks, int waves) {
    return sizeof(float) * waves *
           ((size_t)kTurnFloats + (ks > 1 ? (size_t)(NA * 4 + 1) * kWave : 0));
  };
  // k-slices per workgroup: as many as give every wavefront two chunks at least
  // and still let every workgroup of the launch run at once (the chip has 256
  // compute units) -- a second round of workgroups costs far more than longer
  // slices do (1536 -> 2 x 8960 at 16 rows: 16.2 us with 280 workgroups of 8
  // wavefronts, of which 256 fit, 12.8 us with 280 of 4)
  // (chunks, or with T2 the pairs of chunks a fetch brings)
  const int units = T2 ? (ka.chunks + 1) / 2 : ka.chunks;
  int ks = kMaxWavesI8;
  for (; ks > 1; ks /= 2) {
    if (units / ks < 2)
      continue;
    const int gs = ks < 4 ? 4 / ks : 1, waves = gs * ks;
    const int64_t blocks = ceil_div(ka.spans, gs) * (ka.row_split ? 2 : 1);
    if (blocks <=
        256 * (int64_t)workgroups_per_cu<EPI, SPAN, NORM, T2>(waves, lds_bytes(ks, waves)))
      break;
  }
  if (ks_forced)
    ks = ks_forced;
  BH_REQUIRE(is_pow2(ks), "gemv: %d k-slices (the kernels shift by their count)", ks);
  ka.KS = ks;
  ka.GS = ks < 4 ? 4 / ks : 1;
  const int waves = ka.GS * ka.KS;
  const int blocks = (int)ceil_div(ka.spans, ka.GS) * (ka.row_split ? 2 : 1);
  BH_NOTE_VARIANT(I8Family, EPI, SPAN, NORM, T2);
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(waves * kWave), lds_bytes(ks, waves), stream, ka);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

template <int EPI, int SPAN>
int launch_norm(const I8Args &ka, int ks_forced, hipStream_t stream) {
  // up to 8 rows: two tiles per conversion of the activations (built for the
  // group counts whose two weight tiles per group fit the registers)
  if (ka.two_tiles) {
    if constexpr (EPI == kEpiSiluMul ? SPAN == 1 : SPAN <= 2)
      return ka.norm_w ? launch_kernel<EPI, SPAN, true, true>(ka, ks_forced, stream)
                       : launch_kernel<EPI, SPAN, false, true>(ka, ks_forced, stream);
    else
      return fail(BUDDY_HIP_ERR_ARG, "gemv: no two-tile variant for %d groups per wavefront",
                  SPAN);
  }
  return ka.norm_w ? launch_kernel<EPI, SPAN, true, false>(ka, ks_forced, stream)
                   : launch_kernel<EPI, SPAN, false, false>(ka, ks_forced, stream);
}

template <int SPAN>
int launch_span(const I8Args &ka, int epilogue, int ks_forced, hipStream_t stream) {
  switch (epilogue) {
  case kEpiStore: return launch_norm<kEpiStore, SPAN>(ka, ks_forced, stream);
  case kEpiAccum: return launch_norm<kEpiAccum, SPAN>(ka, ks_forced, stream);
  case kEpiSiluMul:
    if (SPAN > 2)
      return fail(BUDDY_HIP_ERR_ARG, "gemv: SiLU*mul with %d groups per wavefront", SPAN);
    return launch_norm<kEpiSiluMul, (SPAN > 2 ? 2 : SPAN)>(ka, ks_forced, stream);
  }
  return fail(BUDDY_HIP_ERR_ARG, "gemv: unknown epilogue %d", epilogue);
}

// measurement only: BUDDY_HIP_I8_NO_ROW_SPLIT (any value) keeps 9..16 rows in one
// workgroup per span (read once per process)
bool no_row_split() {
  static bool v = getenv("BUDDY_HIP_I8_NO_ROW_SPLIT") != nullptr;
  return v;
}

} // namespace

// Small-batch path of launch_gemv (5 <= M <= 16) on the int8 matrix cores.
int launch_gemv_i8(const GemvArgs &a, hipStream_t stream) {
  I8Args ka;
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
  // Channel groups per wavefront (they share one conversion of the activations
  // and one read of them from L2): as many as still leave the chip a workgroup
  // per compute unit.
  int span = 1;
  if (!dual && ka.groups >= 4 * 512)
    span = 4;
  else if (ka.groups >= 2 * 256)
    span = 2;
  // Between 257 and 1024 channel groups: the fewest groups per wavefront that
  // bring the launch down to one workgroup of 8 k-slices per compute unit (all
  // of them resident at once) beat more, shorter workgroups (4096 -> 6144 at 8
  // rows: 13.5 us as 384 workgroups of 4 wavefronts, 10.3 us as 192 of 8).
  if (ka.groups > 256 && ka.chunks >= 2 * kMaxWavesI8) {
    if (ka.groups <= 2 * 256)
      span = 2;
    else if (!dual && ka.groups <= 4 * 256)
      span = 4;
  }
  // Up to 8 rows: two tiles per conversion, with at most two groups per
  // wavefront.  Two matrices with two groups each stay on the one-tile variant
  // (the same four weight tiles per conversion; 4096 -> 2 x 14336 at 8 rows:
  // 26.0 us against 29.0).
  // 9..16 rows of a matrix so narrow that at most half of the compute units
  // would have a workgroup: the rows go to two workgroups of up to 8 rows (each
  // converts half as much, two tiles at a time; the weights are read twice, the
  // second time from cache)
  ka.row_split = a.M > 8 && ka.groups <= 128 && !no_row_split();
  ka.two_tiles = (a.M <= 8 || ka.row_split) && !(dual && span == 2);
  if (ka.two_tiles && span == 4)
    span = 2;
  ka.spans = (int)ceil_div(ka.groups, span);
  int ks_forced = 0;
  if (const char *e = getenv("BUDDY_HIP_I8_PLAN")) { // measurement only: "span,ks"
    int s_ = 0, k_ = 0;
    if (sscanf(e, "%d,%d", &s_, &k_) == 2 &&
        (s_ == 1 || (ka.two_tiles ? s_ == 2 && !dual : s_ == 2 || (s_ == 4 && !dual))) &&
        (k_ == 1 || k_ == 2 || k_ == 4 || k_ == kMaxWavesI8)) {
      span = s_;
      ks_forced = k_;
      ka.spans = (int)ceil_div(ka.groups, span);
    }
  }
  if (span == 4)
    return launch_span<4>(ka, a.epilogue, ks_forced, stream);
  return span == 2 ? launch_span<2>(ka, a.epilogue, ks_forced, stream)
                   : launch_span<1>(ka, a.epilogue, ks_forced, stream);
}

} // namespace bh
