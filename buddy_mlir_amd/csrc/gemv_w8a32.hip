// gemv_w8a32.hip -- int8 weight-only decode GEMV / small-batch matmul.
//
// Replaces the loop nest that
// midend/lib/Conversion/MatMulOptimization/DequantMatMulVectorizationDecode.cpp
// :250-321 generates (parallel over 32-wide n panels, sequential k, scale
// applied once after the reduction, result added to C).
//
// The kernels are HBM-bound, so their shape follows the memory system:
//  * weights live in 1 KiB wave tiles (16 channels x 64 k); one wavefront
//    streams a contiguous run of tiles of one channel group with 128-bit
//    loads, 1 KiB per instruction, several tiles in flight;
//  * a workgroup is G channel groups x KS k-slices of wavefronts.  Wide
//    matrices (lm_head) use G=4, KS=1; narrow ones (down/o_proj) put up to 16
//    wavefronts on one channel group so that 96 groups still keep ~1500
//    wavefronts streaming.  The k-slices meet in LDS, in slice order, so the
//    sum is deterministic and no workgroup ever waits for another one (cross-
//    XCD traffic inside a kernel costs an L2 write-back on this part);
//  * one to four rows (gemv_w8a32_digits_kernel): a wavefront turns the
//    activations of its run of tiles into four int8 digit planes of a 31-bit
//    fixed-point value per row, leaves them in a private corner of LDS and
//    feeds weight tiles and planes to the int8 matrix cores (exact int32 sums);
//  * runs too long for one batch of loads, or rows that are not 16-byte aligned
//    (gemv_w8a32_bcast_kernel): activations never pass through LDS, a lane
//    loads the one activation whose k equals its position in the tile and the
//    f32 multiply-add reads its neighbours' values through DPP row broadcasts;
//  * RMSNorm is fused in (weight multiplied while consuming, the row's sum of
//    squares gathered on the way, the common rsqrt factor applied to the
//    finished sums), as is folding the attention partials (o_proj);
//  * scale, bias, residual add and SiLU*up are applied to the finished sums in
//    the same kernel; their operands are requested before the stream starts.
// The 8- and 4-channel tile layouts keep the older kernel that stages the
// activations in LDS (gemv_w8a32_kernel).
#include "gemv_w8a32.h"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <utility>

namespace bh {
namespace {


constexpr int kMaxWaves = 16;            // wavefronts per workgroup
constexpr int kXStride = 20;             // floats per (tile, k-group) in LDS:
                                         // 16 used + 4 pad, conflict-free b128
// LDS floats per staged tile: one padded run per 16 k values
constexpr int tile_floats(int tn) { return (1024 / tn / 16) * kXStride; }
constexpr size_t kMaxLdsBytes = 144 * 1024; // hard limit of one workgroup
constexpr size_t kLdsBudget = 40 * 1024;    // preferred, keeps ~4 workgroups per CU

struct GemvPlan {
  int64_t chunks, groups;
  int G, KS, waves, tiles_per_round, blocks;
  // 1: two workgroups per channel group, each streaming the bytes of 8 of its 16
  // channels (narrow, long matrices: 96 channel groups would otherwise keep
  // only 96 of the 256 compute units streaming)
  int half_split = 0;
  // planned for (and checked against the variants of) the digit-plane kernel
  bool on_digits = false;
  size_t lds_bytes;
};

int target_waves() {
  static int v = [] {
    const char *e = getenv("BUDDY_HIP_GEMV_TARGET_WAVES");
    int t = e ? atoi(e) : 0;
    return t > 0 ? t : 4096;
  }();
  return v;
}

bool no_half_split() {
  static bool v = getenv("BUDDY_HIP_GEMV_NO_HALF_SPLIT") != nullptr;
  return v;
}

GemvPlan make_plan(int64_t M, int64_t K, int64_t N, bool dual, int tn, bool fold = false) {
  GemvPlan p;
  p.chunks = ceil_div(K, 1024 / tn);
  p.groups = ceil_div(N, tn);
  // k-slices per channel group: enough wavefronts to cover 256 CUs several
  // times, but at least two tiles per wavefront (one when the input is folded
  // from attention partials: that prologue is a chain of dependent loads per
  // tile, and more, shorter wavefronts shorten it)
  // (one row: 16 wavefronts per CU's worth of them measured best; with more
  // rows per wavefront, half as many)
  const int target = M == 1 ? target_waves() : target_waves() / 2;
  int ks = 1;
  while (ks < kMaxWaves && p.groups * ks < target &&
         p.chunks / (ks * 2) >= (fold ? 1 : 2))
    ks *= 2;
  // four staged tiles per wavefront must fit in LDS for every row
  auto red_bytes = [&](int waves) {
    return sizeof(float) * waves * (size_t)M * (2 * 16 + 1);
  };
  auto round_bytes = [&](int waves, int64_t tiles) {
    return sizeof(float) * tile_floats(tn) * (size_t)M * waves * (size_t)tiles;
  };
  while (ks > 1 && round_bytes(ks < 4 ? 4 : ks, 4) + red_bytes(ks < 4 ? 4 : ks) >
                       kMaxLdsBytes)
    ks /= 2;
  p.KS = ks;
  p.waves = ks < 4 ? 4 : ks;
  while (p.waves > ks && round_bytes(p.waves, 4) + red_bytes(p.waves) > kMaxLdsBytes)
    p.waves /= 2; // fewer channel groups per workgroup
  p.G = p.waves / ks;
  p.blocks = (int)ceil_div(p.groups, p.G);
  const int64_t tiles = ceil_div(p.chunks, ks);
  int64_t cap = (int64_t)(kLdsBudget / round_bytes(p.waves, 1));
  cap = cap / 4 * 4; // rounds are whole batches of four tiles
  if (cap < 4)
    cap = 4;
  p.tiles_per_round = (int)(tiles < cap ? round_up(tiles, 4) : cap);
  p.lds_bytes = round_bytes(p.waves, p.tiles_per_round) + red_bytes(p.waves);
  // One row, 16-channel tiles, at most half of the compute units busy and enough
  // bytes per channel group (>= 64 KiB) for the stream, not latency, to decide
  // the launch: measured 6.6 -> 5.x us for 8960 -> 1536.
  if (M == 1 && tn == 16 && !dual && !fold && p.G == 1 && p.blocks <= 128 &&
      p.chunks >= 64 && !no_half_split())
    p.half_split = 1;
  return p;
}

struct KernelArgs {
  const float *A;
  const int4 *W0, *W1;
  const float *s0, *s1, *bias, *norm_w;
  float *C;
  int64_t lda, ldc;
  float norm_eps, norm_inv_k;
  int K, N, groups, chunks;
  int G, KS, tiles_per_round, tile_n;
  int rows; // valid rows; the kernel is compiled for the next power of two
  // activation provider 2: fold flash-decoding partials while staging
  const float *attn_acc, *attn_ml;
  const int *pos_ptr;
  int attn_nchunks, attn_chunk, head_dim, attn_used;
  // one row, STORE: per channel group the first maximum of its results, or null
  float *cand_v;
  int *cand_i;
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

// acc[m] += sum_j x[m][j] * w[j] for the lane's 16 k values of one tile.
template <int M>
__device__ __forceinline__ void fma_tile(const int4 &w, const float *xl,
                                         int row_stride, float (&acc)[M]) {
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
    const float4 *xv = reinterpret_cast<const float4 *>(xl + m * row_stride);
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
  const float sig = fast_rcp(1.0f + fast_exp(-g));
  return g * sig;
}

// Per-channel operands of the epilogue.  They are fetched when the kernel
// starts, so that their memory latency is hidden behind the weight stream
// instead of following the reduction.
template <int M>
struct EpilogueOperands {
  float s0, s1, bias;
  float c[M];
};

// stores one result and returns it
template <int M, int EPI>
__device__ __forceinline__ float finish(const KernelArgs &a, int m, int n, float raw0,
                                        float raw1, const EpilogueOperands<M> &e) {
  float *c = a.C + (int64_t)m * a.ldc + n;
  const float v = raw0 * e.s0;
  float y;
  if (EPI == kEpiSiluMul) {
    const float u = raw1 * e.s1;
    y = silu(v) * u;
  } else if (EPI == kEpiAccum) {
    y = e.c[m] + v;
  } else {
    y = a.bias ? e.bias + v : v;
  }
  *c = y;
  return y;
}

// The first maximum of the 16 results of a channel group (lanes 0..15 of the
// wavefront that finished it; `y` of a lane without a result is ignored):
// larger value first, then smaller index, NaNs never -- the order of
// std::max_element over the row.  Lane 0 writes (value, index) for the group.
__device__ __forceinline__ void emit_group_maximum(const KernelArgs &a, int g, int lane,
                                                   bool has, float y, int n) {
  float v = -INFINITY;
  int i = 0x7fffffff;
  if (has && y == y) {
    v = y;
    i = n;
  }
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, 16);
    const int oi = __shfl_xor(i, o, 16);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
  if (lane == 0) {
    a.cand_v[g] = v;
    a.cand_i[g] = i;
  }
}

// Combined attention output for 4 consecutive k of one head, from the
// flash-decoding partials (m, l, acc) of the chunks used so far:
//   w_s = exp(m_s - max m); x = sum_s w_s acc_s / sum_s w_s l_s
// (the combine of frontend/Python/ops/tosa.py:14485-14594, eight chunks at a
// time so that their loads are in flight together).
__device__ __forceinline__ float4 attn_combined(const KernelArgs &a, int k) {
  constexpr int B = 9; // partials fetched per batch (two batches at 18 chunks)
  const int h = k >> shift_of(a.head_dim), d = k & (a.head_dim - 1); // a power of two
  // every chunk the launch was given is folded: the ones beyond the position
  // hold (m, l, acc) = (-1e30, 0, 0) and drop out with weight exp(-1e30 - m) = 0,
  // so the loop does not have to wait for the position
  const int used = a.attn_used;
  const float2 *ml = reinterpret_cast<const float2 *>(a.attn_ml) +
                     (size_t)h * a.attn_nchunks;
  const float *acc = a.attn_acc + (size_t)h * a.attn_nchunks * a.head_dim + d;
  float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
  float m = -1.0e30f, l = 0.f;
  for (int s0 = 0; s0 < used; s0 += B) {
    float2 mlv[B];
    float4 v[B];
#pragma unroll
    for (int j = 0; j < B; ++j) {
      const int s = min(s0 + j, used - 1);
      mlv[j] = ml[s];
      v[j] = *reinterpret_cast<const float4 *>(acc + (size_t)s * a.head_dim);
    }
    float mb = m;
#pragma unroll
    for (int j = 0; j < B; ++j)
      if (s0 + j < used)
        mb = fmaxf(mb, mlv[j].x);
    const float al = fast_exp(m - mb); // rescale what was gathered so far
    r.x *= al;
    r.y *= al;
    r.z *= al;
    r.w *= al;
    l *= al;
    m = mb;
#pragma unroll
    for (int j = 0; j < B; ++j) {
      if (s0 + j < used) {
        const float w = fast_exp(mlv[j].x - m);
        l = fmaf(mlv[j].y, w, l);
        r.x = fmaf(v[j].x, w, r.x);
        r.y = fmaf(v[j].y, w, r.y);
        r.z = fmaf(v[j].z, w, r.z);
        r.w = fmaf(v[j].w, w, r.w);
      }
    }
  }
  const float inv = fast_rcp(l);
  return make_float4(r.x * inv, r.y * inv, r.z * inv, r.w * inv);
}

enum { kProPlain = 0, kProNorm = 1, kProAttn = 2 };

template <int M, int EPI, int PRO, int U, int TN>
__global__ void __launch_bounds__(kMaxWaves *kWave)
    gemv_w8a32_kernel(KernelArgs a) {
  constexpr int TK = 1024 / TN;           // k values per tile
  constexpr int kTileFloats = tile_floats(TN);
  constexpr bool DUAL = (EPI == kEpiSiluMul);
  constexpr bool NORM = (PRO == kProNorm);
  // U = weight loads in flight per matrix
  extern __shared__ float lds[];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int nwaves = a.G * a.KS;
  const int ksh = shift_of(a.KS);
  const int gl = wave >> ksh, ks = wave & (a.KS - 1);
  const int g = blockIdx.x * a.G + gl;
  const bool live = g < a.groups;
  // this wavefront's contiguous run of tiles
  const int per = (a.chunks + a.KS - 1) >> ksh;
  const int t0 = min(ks * per, a.chunks);
  const int t1 = min(t0 + per, a.chunks);
  const int TR = a.tiles_per_round;
  const int row_stride = TR * kTileFloats;
  float *xs = lds + (size_t)wave * M * row_stride;
  float *red = lds + (size_t)nwaves * M * row_stride;

  float acc0[M], acc1[M], ss[M]; // acc1 is dead code unless DUAL
#pragma unroll
  for (int m = 0; m < M; ++m) {
    acc0[m] = 0.f;
    acc1[m] = 0.f;
    ss[m] = 0.f;
  }
  const size_t wbase = ((size_t)(live ? g : 0) * a.chunks) * 64 + lane;
  const int4 *w0 = a.W0 + wbase;
  const int4 *w1 = DUAL ? a.W1 + wbase : a.W0 + wbase;
  // where this lane's float4 of a 256-float staging load lands in LDS
  const int st_off = (lane >> 2) * kXStride + (lane & 3) * 4;
  const float *xl = xs + (lane / TN) * kXStride; // this lane's k sub-range

  const int n = g * TN + lane;
  const bool writer = ks == 0 && lane < TN && live && n < a.N;
  EpilogueOperands<M> epi;

  const int nrounds = (per + TR - 1) / TR; // same for every wavefront
  const int kend = min(a.K, t1 * TK);       // this wavefront's k range ends here
  for (int rd = 0; rd < nrounds; ++rd) {
    const int r0 = t0 + rd * TR;
    const int r1 = min(r0 + TR, t1);
    // ---- first batch of weight loads goes out before anything else -------
    int4 wa[U], wb[U];
    if (r0 < r1) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (r0 + u < r1) { // never fetch a tile this wavefront will not use
          wa[u] = load_stream(w0 + (size_t)(r0 + u) * 64);
          if (DUAL)
            wb[u] = load_stream(w1 + (size_t)(r0 + u) * 64);
        }
      }
    }
    if (rd == 0 && writer) {
      epi.s0 = a.s0[n];
      if (DUAL)
        epi.s1 = a.s1[n];
      if (EPI == kEpiStore && a.bias)
        epi.bias = a.bias[n];
      if (EPI == kEpiAccum) {
#pragma unroll
        for (int m = 0; m < M; ++m)
          if (m < a.rows)
            epi.c[m] = a.C[(int64_t)m * a.ldc + n];
      }
    }
    // ---- stage this wavefront's slice of the activations -----------------
    if (rd != 0)
      __syncthreads(); // everyone is done with the previous round's LDS
    for (int i = 0; i < ((r1 - r0) * TK + 255) / 256; ++i) {
      const int k = r0 * TK + i * 256 + lane * 4;
      float4 nw = make_float4(1.f, 1.f, 1.f, 1.f);
      const bool in = k + 3 < kend;
      if (NORM) {
        if (in)
          nw = *reinterpret_cast<const float4 *>(a.norm_w + k);
        else
          nw = make_float4(k < kend ? a.norm_w[k] : 0.f,
                           k + 1 < kend ? a.norm_w[k + 1] : 0.f,
                           k + 2 < kend ? a.norm_w[k + 2] : 0.f, 0.f);
      }
#pragma unroll
      for (int m = 0; m < M; ++m) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (PRO == kProAttn) {
          if (m == 0 && in)
            v = attn_combined(a, k);
        } else if (m < a.rows) {
          const float *src = a.A + (int64_t)m * a.lda + k;
          if (in && ((reinterpret_cast<uintptr_t>(src) & 15) == 0))
            v = *reinterpret_cast<const float4 *>(src);
          else
            v = make_float4(k < kend ? src[0] : 0.f, k + 1 < kend ? src[1] : 0.f,
                            k + 2 < kend ? src[2] : 0.f,
                            k + 3 < kend ? src[3] : 0.f);
        }
        if (NORM) {
          ss[m] = fmaf(v.x, v.x, ss[m]);
          ss[m] = fmaf(v.y, v.y, ss[m]);
          ss[m] = fmaf(v.z, v.z, ss[m]);
          ss[m] = fmaf(v.w, v.w, ss[m]);
          v.x *= nw.x;
          v.y *= nw.y;
          v.z *= nw.z;
          v.w *= nw.w;
        }
        *reinterpret_cast<float4 *>(xs + m * row_stride + i * 16 * kXStride +
                                    st_off) = v;
      }
    }
    __syncthreads();
    // ---- stream the tiles, next batch in flight while this one is used ----
    for (int t = r0; t < r1; t += U) {
      int4 na[U], nb[U];
      const bool more = t + U < r1;
      if (more) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (t + U + u < r1) {
            na[u] = load_stream(w0 + (size_t)(t + U + u) * 64);
            if (DUAL)
              nb[u] = load_stream(w1 + (size_t)(t + U + u) * 64);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (t + u < r1) {
          const float *x = xl + (t + u - r0) * kTileFloats;
          fma_tile<M>(wa[u], x, row_stride, acc0);
          if (DUAL)
            fma_tile<M>(wb[u], x, row_stride, acc1);
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

  // lanes TN apart hold different k sub-ranges of the same channel
#pragma unroll
  for (int m = 0; m < M; ++m) {
#pragma unroll
    for (int o = TN; o < 64; o <<= 1) {
      acc0[m] += __shfl_xor(acc0[m], o, 64);
      if (DUAL)
        acc1[m] += __shfl_xor(acc1[m], o, 64);
    }
    if (NORM)
      ss[m] = wave_sum(ss[m]);
  }

  // ---- k-slices of one channel group meet in LDS, in slice order ----------
  if (a.KS > 1) {
    float *mine = red + (size_t)wave * M * 33;
    if (lane < TN) {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        mine[m * 33 + lane] = acc0[m];
        if (DUAL)
          mine[m * 33 + 16 + lane] = acc1[m];
      }
    }
    if (NORM && lane == 0) {
#pragma unroll
      for (int m = 0; m < M; ++m)
        mine[m * 33 + 32] = ss[m];
    }
    __syncthreads();
    if (ks != 0)
      return;
    if (lane < TN) {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        float r0 = 0.f, r1 = 0.f, rs = 0.f;
        for (int s = 0; s < a.KS; ++s) {
          const float *o = red + (size_t)(wave + s) * M * 33 + m * 33;
          r0 += o[lane];
          if (DUAL)
            r1 += o[16 + lane];
          if (NORM)
            rs += o[32];
        }
        acc0[m] = r0;
        acc1[m] = r1;
        ss[m] = rs;
      }
    }
  }
  if (writer) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      if (m < a.rows) {
        float v0 = acc0[m], v1 = acc1[m];
        if (NORM) {
          // x' = w (.) (x * r) with r = rsqrt(mean(x^2) + eps): r is common to
          // the whole row, so it multiplies the finished sum
          // (subgraph0_decode_simplify.mlir:60-72)
          const float r = fast_rsqrt(ss[m] * a.norm_inv_k + a.norm_eps);
          v0 *= r;
          v1 *= r;
        }
        finish<M, EPI>(a, m, n, v0, v1, epi);
      }
    }
  }
}


// ---------------------------------------------------------------------------
// 16-channel tiles: activations stay in registers.
//
// In a 16 x 64 tile the 16 lanes of a DPP row (lanes 16r .. 16r+15) hold 16
// different channels of the same 16 k values, k = 64c + 16r + j.  A lane that
// loads x[64c + lane] therefore holds, for its row, exactly the 16 activations
// the row needs, and `v_fmac_f32 ... row_newbcast:j` multiplies every lane's
// j-th weight with the activation held by lane j of its own row.  No LDS
// staging, no barrier before the stream, and the VALU issues two instructions
// per weight (SDWA convert + DPP multiply-add) and nothing else.
// ---------------------------------------------------------------------------

// acc += sum_j x(lane j of this row) * (float)(int8 byte j of w), bytes in the
// order x, y, z, w of the 16-byte word.  Convert and multiply-add are
// interleaved over four rotating temporaries so that a tile in flight costs
// four registers, not sixteen.  The leading wait states cover a preceding VALU
// write of x (2) or of EXEC (5) before the first DPP read.
__device__ __forceinline__ void fma_tile_row_bcast(float &acc, float x, const int4 &w) {
  float t0, t1, t2, t3;
  asm volatile(
      "s_nop 4\n\t"
      "v_cvt_f32_i32_sdwa %1, sext(%6) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0\n\t"
      "v_cvt_f32_i32_sdwa %2, sext(%6) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1\n\t"
      "v_cvt_f32_i32_sdwa %3, sext(%6) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2\n\t"
      "v_cvt_f32_i32_sdwa %4, sext(%6) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3\n\t"
      "v_fmac_f32_dpp %0, %5, %1 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %1, sext(%7) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0\n\t"
      "v_fmac_f32_dpp %0, %5, %2 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %2, sext(%7) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1\n\t"
      "v_fmac_f32_dpp %0, %5, %3 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %3, sext(%7) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2\n\t"
      "v_fmac_f32_dpp %0, %5, %4 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %4, sext(%7) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3\n\t"
      "v_fmac_f32_dpp %0, %5, %1 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %1, sext(%8) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0\n\t"
      "v_fmac_f32_dpp %0, %5, %2 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %2, sext(%8) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1\n\t"
      "v_fmac_f32_dpp %0, %5, %3 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %3, sext(%8) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2\n\t"
      "v_fmac_f32_dpp %0, %5, %4 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %4, sext(%8) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3\n\t"
      "v_fmac_f32_dpp %0, %5, %1 row_newbcast:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %1, sext(%9) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0\n\t"
      "v_fmac_f32_dpp %0, %5, %2 row_newbcast:9 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %2, sext(%9) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1\n\t"
      "v_fmac_f32_dpp %0, %5, %3 row_newbcast:10 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %3, sext(%9) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2\n\t"
      "v_fmac_f32_dpp %0, %5, %4 row_newbcast:11 row_mask:0xf bank_mask:0xf\n\t"
      "v_cvt_f32_i32_sdwa %4, sext(%9) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3\n\t"
      "v_fmac_f32_dpp %0, %5, %1 row_newbcast:12 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %5, %2 row_newbcast:13 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %5, %3 row_newbcast:14 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %5, %4 row_newbcast:15 row_mask:0xf bank_mask:0xf"
      : "+v"(acc), "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3)
      : "v"(x), "v"(w.x), "v"(w.y), "v"(w.z), "v"(w.w));
}

// acc[m] += ... for M rows that share the converted weights.
__device__ __forceinline__ void fma16_row_bcast(float &acc, float x,
                                                const float (&w)[16]) {
  asm volatile(
      "s_nop 4\n\t"
      "v_fmac_f32_dpp %0, %1, %2 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %3 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %4 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %5 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %6 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %7 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %8 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %9 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %10 row_newbcast:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %11 row_newbcast:9 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %12 row_newbcast:10 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %13 row_newbcast:11 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %14 row_newbcast:12 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %15 row_newbcast:13 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %16 row_newbcast:14 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f32_dpp %0, %1, %17 row_newbcast:15 row_mask:0xf bank_mask:0xf"
      : "+v"(acc)
      : "v"(x), "v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3]), "v"(w[4]), "v"(w[5]),
        "v"(w[6]), "v"(w[7]), "v"(w[8]), "v"(w[9]), "v"(w[10]), "v"(w[11]),
        "v"(w[12]), "v"(w[13]), "v"(w[14]), "v"(w[15]));
}

__device__ __forceinline__ void tile_to_float(const int4 &w, float (&wf)[16]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    wf[j] = byte_to_float(w.x, j);
    wf[4 + j] = byte_to_float(w.y, j);
    wf[8 + j] = byte_to_float(w.z, j);
    wf[12 + j] = byte_to_float(w.w, j);
  }
}

// Combined attention output (see attn_combined) for the k = 64 t + lane of U
// consecutive tiles of a wavefront.  A tile lies inside one head, so the chunk
// weights exp(m_s - max m) are common to the wavefront: lane s computes the
// weight of chunk s (one exp for up to 64 chunks) and the sum over the chunks
// reads it from there.  The partials of all U tiles are requested together, 18
// chunks at a time.
template <int U>
__device__ __forceinline__ void attn_fold_tiles(const KernelArgs &a, int t0, int t1,
                                                int lane, float (&x)[U]) {
  constexpr int B = 18;
  const int used = a.attn_used;
  const float2 *ml[U];
  const float *acc[U];
  float r[U], m[U], l[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int t = min(t0 + u, t1 - 1); // slots past the run repeat its last tile
    const int k = min(t * kTileK + lane, a.K - 1);
    const int h = __builtin_amdgcn_readfirstlane(k >> shift_of(a.head_dim)),
              d = k & (a.head_dim - 1); // a power of two
    ml[u] = reinterpret_cast<const float2 *>(a.attn_ml) + (size_t)h * a.attn_nchunks;
    acc[u] = a.attn_acc + (size_t)h * a.attn_nchunks * a.head_dim + d;
    r[u] = 0.f;
    m[u] = -1.0e30f;
    l[u] = 0.f;
  }
  // The usual case (up to 18 chunks: a cache of 1152 positions, or a step whose
  // chunks are 128 or 256 positions), and up to 36: one batch, and nothing in it
  // depends on anything loaded -- the (max, sum) pair of every chunk and the
  // partial sums of every tile are requested together, so the fold costs one trip
  // to memory, not two.  Slots past the last chunk repeat it (a valid, finite
  // partial) and get weight 0.
  auto one_batch = [&](auto batch) {
    constexpr int BB = decltype(batch)::value;
    float2 mine[U];
    float v[U][BB];
#pragma unroll
    for (int u = 0; u < U; ++u)
      mine[u] = ml[u][min(lane, used - 1)];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int j = 0; j < BB; ++j)
        v[u][j] = acc[u][(size_t)min(j, used - 1) * a.head_dim];
    const bool valid = lane < used;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float mb = wave_max(valid ? mine[u].x : -1.0e30f);
      const float w = valid ? fast_exp(mine[u].x - mb) : 0.f;
      l[u] = wave_sum(mine[u].y * w);
#pragma unroll
      for (int j = 0; j < BB; ++j)
        r[u] = fmaf(v[u][j], lane_f(w, j), r[u]);
    }
  };
  if (used <= B) {
    one_batch(std::integral_constant<int, B>{});
  } else if (used <= 2 * B && U <= 2) {
    one_batch(std::integral_constant<int, 2 * B>{});
  } else {
  for (int c0 = 0; c0 < used; c0 += kWave) { // 64 chunks per pass
    const int cnt = min(kWave, used - c0);
    float w[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float2 mine = ml[u][c0 + min(lane, cnt - 1)];
      const bool valid = lane < cnt;
      const float mb = fmaxf(m[u], wave_max(valid ? mine.x : -1.0e30f));
      const float al = fast_exp(m[u] - mb); // rescale what earlier passes gathered
      w[u] = valid ? fast_exp(mine.x - mb) : 0.f;
      l[u] = fmaf(l[u], al, wave_sum(mine.y * w[u]));
      r[u] *= al;
      m[u] = mb;
    }
    for (int s0 = 0; s0 < cnt; s0 += B) {
      float v[U][B];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int j = 0; j < B; ++j)
          v[u][j] = acc[u][(size_t)(c0 + min(s0 + j, cnt - 1)) * a.head_dim];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int j = 0; j < B; ++j)
          if (s0 + j < cnt)
            r[u] = fmaf(v[u][j], lane_f(w[u], s0 + j), r[u]);
    }
  }
  } // longer caches
#pragma unroll
  for (int u = 0; u < U; ++u)
    x[u] = r[u] * fast_rcp(l[u]);
}

// One tile's worth of operands of one wavefront.
template <int M> struct TileOperands {
  int4 w0, w1;
  float x[M];
  float nw;
};

template <int M, int PRO, bool DUAL, bool FOLD_LATER = false>
__device__ __forceinline__ void fetch_tile(const KernelArgs &a, const int4 *w0,
                                           const int4 *w1, int t, int lane,
                                           TileOperands<M> &o) {
  o.w0 = load_stream(w0 + (size_t)t * 64);
  if (DUAL)
    o.w1 = load_stream(w1 + (size_t)t * 64);
  // out-of-range lanes and rows read a valid address; the value is dropped when
  // the tile is consumed.  Branch-free loads whose results are not touched here
  // let the compiler keep an exact count of the loads in flight.
  const int k = t * kTileK + lane;
  const int kc = k < a.K ? k : a.K - 1;
  if (PRO == kProNorm)
    o.nw = a.norm_w[kc];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    if (PRO == kProAttn) {
      if (!FOLD_LATER) {
        float x1[1] = {0.f};
        if (m == 0)
          attn_fold_tiles<1>(a, t, t + 1, lane, x1);
        o.x[m] = x1[0];
      }
    } else {
      if (M == 1) {
        o.x[m] = a.A[kc];
      } else {
        const int mc = m < a.rows ? m : a.rows - 1;
        o.x[m] = a.A[(int64_t)mc * a.lda + kc];
      }
    }
  }
}

// Everything a wavefront needs before it can request its tiles -- four
// pointers and six integers, 14 argument words -- are separate leading
// parameters: this file is built with -amdgpu-kernarg-preload-count=14, so the
// command processor hands them to every wavefront in SGPRs and the first loads
// do not wait for a scalar load of the argument block.  The remaining fields
// travel in `rest` and are loaded as usual, behind the stream.
template <int M, int EPI, int PRO, int U>
__global__ void __launch_bounds__(kMaxWaves *kWave)
    gemv_w8a32_bcast_kernel(const int4 *pW0, const int4 *pW1, const float *pA,
                            const float *pnorm_w, int p_chunks, int p_KS, int p_G,
                            int p_groups, int p_K, int p_rows, KernelArgs rest) {
  KernelArgs a = rest;
  a.W0 = pW0;
  a.W1 = pW1;
  a.A = pA;
  a.norm_w = pnorm_w;
  a.chunks = p_chunks;
  a.KS = p_KS;
  a.G = p_G & 0xffff;
  const int hs = p_G >> 16; // 1: this workgroup takes 8 of its group's 16 channels
  a.groups = p_groups;
  a.K = p_K;
  a.rows = p_rows;
  constexpr bool DUAL = (EPI == kEpiSiluMul);
  constexpr bool NORM = (PRO == kProNorm);
  extern __shared__ float lds[]; // only the meeting place of the k-slices
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int ksh = shift_of(a.KS);
  const int gl = wave >> ksh, ks = wave & (a.KS - 1);
  const int gi = blockIdx.x * a.G + gl;
  const int g = gi >> hs, half = gi & hs;
  const bool live = g < a.groups;
  const int per = (a.chunks + a.KS - 1) >> ksh;
  const int t0 = min(ks * per, a.chunks);
  const int t1 = min(t0 + per, a.chunks);

  float acc0[M], acc1[M], ss[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    acc0[m] = 0.f;
    acc1[m] = 0.f;
    ss[m] = 0.f;
  }
  // With the channel group split over two workgroups, the lanes of the other
  // half read their partner's 16 bytes (lane ^ 8: the same cache line, no extra
  // traffic) and compute a copy of its sums that nobody stores: every load
  // instruction then moves four whole 128-byte lines, half a tile.
  const int wlane = hs ? ((lane & ~8) | (half << 3)) : lane;
  const size_t wbase = ((size_t)(live ? g : 0) * a.chunks) * 64 + wlane;
  const int4 *w0 = a.W0 + wbase;
  const int4 *w1 = DUAL ? a.W1 + wbase : a.W0 + wbase;

  // a ring of U tiles in flight: a slot is refilled as soon as it is consumed
  TileOperands<M> slot[U];
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (t0 + u < t1)
      fetch_tile<M, PRO, DUAL, true>(a, w0, w1, t0 + u, lane, slot[u]);
  if (PRO == kProAttn && t0 < t1) {
    // at most four tiles per fold keep the partials of a batch in registers
    constexpr int FB = U < 4 ? U : 4;
    float xf[(U + FB - 1) / FB][FB];
#pragma unroll
    for (int q = 0; q < (U + FB - 1) / FB; ++q)
      if (t0 + FB * q < t1)
        attn_fold_tiles<FB>(a, t0 + FB * q, t1, lane, xf[q]);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      slot[u].x[0] = xf[u / FB][u % FB];
#pragma unroll
      for (int m = 1; m < M; ++m)
        slot[u].x[m] = 0.f;
    }
  }

  const int n = g * kTileN + lane;
  const bool writer = ks == 0 && lane < kTileN && live && n < a.N &&
                      (!hs || (lane >> 3) == half);
  EpilogueOperands<M> epi;
  if (writer) {
    epi.s0 = a.s0[n];
    if (DUAL)
      epi.s1 = a.s1[n];
    if (EPI == kEpiStore && a.bias)
      epi.bias = a.bias[n];
    if (EPI == kEpiAccum) {
#pragma unroll
      for (int m = 0; m < M; ++m)
        if (m < a.rows)
          epi.c[m] = a.C[(int64_t)m * a.ldc + n];
    }
  }

  for (int t = t0; t < t1; t += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (t + u < t1) {
        const TileOperands<M> &o = slot[u];
        const bool in = (t + u) * kTileK + lane < a.K;
        if (M == 1) {
          float x = in ? o.x[0] : 0.f;
          if (NORM) {
            ss[0] = fmaf(x, x, ss[0]);
            x *= o.nw;
          }
          fma_tile_row_bcast(acc0[0], x, o.w0);
          if (DUAL)
            fma_tile_row_bcast(acc1[0], x, o.w1);
        } else {
          float wf0[16], wf1[16];
          tile_to_float(o.w0, wf0);
          if (DUAL)
            tile_to_float(o.w1, wf1);
#pragma unroll
          for (int m = 0; m < M; ++m) {
            float x = (in && m < a.rows) ? o.x[m] : 0.f;
            if (NORM) {
              ss[m] = fmaf(x, x, ss[m]);
              x *= o.nw;
            }
            fma16_row_bcast(acc0[m], x, wf0);
            if (DUAL)
              fma16_row_bcast(acc1[m], x, wf1);
          }
        }
        if (t + U + u < t1)
          fetch_tile<M, PRO, DUAL>(a, w0, w1, t + U + u, lane, slot[u]);
      }
    }
  }

  // the four rows of a wavefront hold different k sub-ranges of the same channels
#pragma unroll
  for (int m = 0; m < M; ++m) {
    acc0[m] = sum_rows(acc0[m]);
    if (DUAL)
      acc1[m] = sum_rows(acc1[m]);
    if (NORM)
      ss[m] = wave_sum(ss[m]);
  }

  // ---- k-slices of one channel group meet in LDS, in slice order ----------
  if (a.KS > 1) {
    float *mine = lds + (size_t)wave * M * 33;
    if (lane < kTileN) {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        mine[m * 33 + lane] = acc0[m];
        if (DUAL)
          mine[m * 33 + 16 + lane] = acc1[m];
      }
    }
    if (NORM && lane == 0) {
#pragma unroll
      for (int m = 0; m < M; ++m)
        mine[m * 33 + 32] = ss[m];
    }
    __syncthreads();
    if (ks != 0)
      return;
    if (lane < kTileN) {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        float r0 = 0.f, r1 = 0.f, rs = 0.f;
        for (int s = 0; s < a.KS; ++s) {
          const float *o = lds + (size_t)(wave + s) * M * 33 + m * 33;
          r0 += o[lane];
          if (DUAL)
            r1 += o[16 + lane];
          if (NORM)
            rs += o[32];
        }
        acc0[m] = r0;
        acc1[m] = r1;
        ss[m] = rs;
      }
    }
  }
  float y_row = 0.f; // one row: its result of this lane's channel
  if (writer) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      if (m < a.rows) {
        float v0 = acc0[m], v1 = acc1[m];
        if (NORM) {
          // x' = w (.) (x * r) with r = rsqrt(mean(x^2) + eps): r is common to
          // the whole row, so it multiplies the finished sum
          // (subgraph0_decode_simplify.mlir:60-72)
          const float r = fast_rsqrt(ss[m] * a.norm_inv_k + a.norm_eps);
          v0 *= r;
          v1 *= r;
        }
        const float y = finish<M, EPI>(a, m, n, v0, v1, epi);
        if (M == 1)
          y_row = y;
      }
    }
  }
  if (M == 1 && EPI == kEpiStore && a.cand_v && live)
    emit_group_maximum(a, g, lane, writer, y_row, n);
}

// ---------------------------------------------------------------------------
// One to four rows on the int8 matrix cores, no VALU instruction per weight.
//
// A wavefront turns the activations of its own run of tiles into fixed point,
// X = rint(x / s) with s the smallest power of two that keeps |X| < 2^30 over
// the run (one s per row), cuts X into four balanced int8 digits
// (X = d0 + 256 d1 + 65536 d2 + 2^24 d3) and leaves each digit plane in its own
// corner of LDS in k order.  A weight tile as it lies in its registers is the A
// operand of v_mfma_i32_16x16x64_i8 (16 channels x 64 k); the 4 M digit planes
// of the tile are columns of B, of which lane (k / 16, column) reads its 16
// bytes with one ds_read_b128.  One matrix instruction per tile and matrix
// multiplies every row and digit.  The int32 sums are exact; the only rounding
// is that of X, 2^-31 of the row's largest activation in the run, so that an
// activation within 2^7 of that largest one enters with all its 24 bits.
// Nothing waits for another wavefront before the stream: the planes are private
// to the wavefront that wrote them.
// ---------------------------------------------------------------------------
constexpr int kDigits = 4;                            // int8 digits per activation
constexpr int kDigitBytesPerTile = kDigits * kTileK;  // the planes of one tile and row

// HS (a channel group split over two workgroups): a load instruction covers the
// workgroup's 8 channels of two consecutive tiles -- the lanes that would hold
// the other workgroup's channels take the second tile instead -- so it moves
// 1 KiB of weights that nobody else reads, in whole 128-byte lines.  The rows
// of such an A operand belong to two tiles: it is multiplied once with each
// tile's planes and every row keeps the product that is its own.
template <int M, int EPI, int PRO, int U, bool HS>
__global__ void __launch_bounds__(kMaxWaves *kWave)
    gemv_w8a32_digits_kernel(const int4 *pW0, const int4 *pW1, const float *pA,
                           const float *pnorm_w, int p_chunks, int p_KS, int p_G,
                           int p_groups, int p_K, int p_rows, KernelArgs rest) {
  KernelArgs a = rest;
  a.W0 = pW0;
  a.W1 = pW1;
  a.A = pA;
  a.norm_w = pnorm_w;
  a.chunks = p_chunks;
  a.KS = p_KS;
  a.G = p_G & 0xffff;
  const int hs = p_G >> 16; // 1: this workgroup takes 8 of its group's 16 channels
  a.groups = p_groups;
  a.K = p_K;
  a.rows = p_rows;
  constexpr bool DUAL = (EPI == kEpiSiluMul);
  constexpr bool NORM = (PRO == kProNorm);
  static_assert(M == 1 || PRO != kProAttn, "the attention fold feeds one row");
  extern __shared__ float lds[];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int nwaves = a.G * a.KS;
  const int ksh = shift_of(a.KS);
  const int gl = wave >> ksh, ks = wave & (a.KS - 1);
  const int gi = blockIdx.x * a.G + gl;
  const int g = gi >> hs, half = gi & hs;
  const bool live = g < a.groups;
  const int per = (a.chunks + a.KS - 1) >> ksh;
  const int t0 = min(ks * per, a.chunks);
  const int t1 = min(t0 + per, a.chunks);

  // ---- activations first: their use must not wait for the weights ----------
  // A lane takes four consecutive k of the run per load (64 lanes: four tiles),
  // so that it can cut their digits and write whole dwords of the planes.  The
  // 16 bytes start inside the row and are aligned, so they never leave the page
  // the row ends in; values past the row or the run are dropped below.  When
  // the input is folded from attention partials a lane holds one k per tile.
  constexpr bool VEC = PRO != kProAttn;
  constexpr int XV = VEC ? (U + 3) / 4 : U; // activation slots per row
  constexpr int XE = VEC ? 4 : 1;           // values per slot
  float x[M][XV][XE], nw[XV][XE];
  if constexpr (VEC) {
    // lanes past the run repeat its last 16 bytes (a line this wavefront reads
    // anyway, not one that every wavefront of the launch would share)
    const int klast = max(min(((a.K + 3) & ~3), t1 * kTileK) - 4, 0);
#pragma unroll
    for (int q = 0; q < XV; ++q) {
      const int kc = min(t0 * kTileK + q * 256 + 4 * lane, klast);
      if (NORM) {
        // (the weight's last 16 bytes may reach past its end, where anything
        // lies -- a NaN there would turn the zero it meets into a NaN)
        const float4 v = *reinterpret_cast<const float4 *>(a.norm_w + kc);
        nw[q][0] = v.x;
        nw[q][1] = kc + 1 < a.K ? v.y : 0.f;
        nw[q][2] = kc + 2 < a.K ? v.z : 0.f;
        nw[q][3] = kc + 3 < a.K ? v.w : 0.f;
      }
#pragma unroll
      for (int m = 0; m < M; ++m) { // rows past the batch repeat its last row; never stored
        const float4 v = *reinterpret_cast<const float4 *>(
            a.A + (int64_t)(M == 1 ? 0 : min(m, a.rows - 1)) * a.lda + kc);
        x[m][q][0] = v.x, x[m][q][1] = v.y, x[m][q][2] = v.z, x[m][q][3] = v.w;
      }
    }
  }
  static_assert(!HS || (!DUAL && U % 2 == 0), "split groups: one matrix, tiles in pairs");
  constexpr int P = HS ? U / 2 : U; // weight loads per matrix
  const int wlane = HS ? ((lane & ~8) | (half << 3)) : lane;
  const int second = HS ? (((lane >> 3) & 1) ^ half) : 0; // this lane takes the pair's second tile
  const size_t wbase = ((size_t)(live ? g : 0) * a.chunks) * 64 + wlane;
  const int4 *w0 = a.W0 + wbase;
  const int4 *w1 = DUAL ? a.W1 + wbase : a.W0 + wbase;
  int4 wa[P], wb[P];
#pragma unroll
  for (int u = 0; u < P; ++u) {
    // Every load is issued whatever the run's length, so that the wait for the
    // activations can name the exact number of weight loads behind them.  A
    // slot past the run repeats the run's last tile (lines this wavefront has
    // just asked for) and meets zero digits (the second tile of a last pair) or
    // is not used; the slot counts are dense so that few runs have such a slot.
    const int t = min(t0 + (HS ? 2 * u + second : u), max(t1 - 1, 0));
    wa[u] = load_stream(w0 + (size_t)t * 64);
    if (DUAL)
      wb[u] = load_stream(w1 + (size_t)t * 64);
  }
  if constexpr (PRO == kProAttn) {
    if (t0 < t1) {
      constexpr int FB = U < 4 ? U : 4;
      float xf[(U + FB - 1) / FB][FB];
#pragma unroll
      for (int q = 0; q < (U + FB - 1) / FB; ++q)
        if (t0 + FB * q < t1)
          attn_fold_tiles<FB>(a, t0 + FB * q, t1, lane, xf[q]);
#pragma unroll
      for (int u = 0; u < U; ++u)
        x[0][u][0] = xf[u / FB][u % FB];
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u)
        x[0][u][0] = 0.f;
    }
  }

  const int n = g * kTileN + lane;
  const bool writer = ks == 0 && lane < kTileN && live && n < a.N &&
                      (!hs || (lane >> 3) == half);
  EpilogueOperands<M> epi;
  if (writer) {
    epi.s0 = a.s0[n];
    if (DUAL)
      epi.s1 = a.s1[n];
    if (EPI == kEpiStore && a.bias)
      epi.bias = a.bias[n];
    if (EPI == kEpiAccum) {
#pragma unroll
      for (int m = 0; m < M; ++m)
        if (m < a.rows)
          epi.c[m] = a.C[(int64_t)m * a.ldc + n];
    }
  }

  // ---- this wavefront's activations -> digit planes in LDS -----------------
  // Four digits: X = rint(x / s) with |X| < 2^30, so that an activation within
  // 2^7 of the row's largest in the run keeps every one of its 24 bits.
  // Per row the run's largest magnitude first (a NaN or infinity is the
  // largest bit pattern), then the step.
  float ss[M], step[M], inv[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    ss[m] = 0.f;
    unsigned mb = 0;
#pragma unroll
    for (int q = 0; q < XV; ++q) {
#pragma unroll
      for (int e = 0; e < XE; ++e) {
        // VEC: k = 64 t0 + 256 q + 4 lane + e; otherwise k = 64 (t0 + q) + lane
        const int k = VEC ? t0 * kTileK + q * 256 + 4 * lane + e : (t0 + q) * kTileK + lane;
        const bool in = k < t1 * kTileK && k < a.K;
        float v = in ? x[m][q][e] : 0.f;
        if (NORM) {
          ss[m] = fmaf(v, v, ss[m]);
          v *= nw[q][e];
        }
        x[m][q][e] = v;
        mb = max(mb, __float_as_uint(v) & 0x7fffffffu);
      }
    }
    mb = wave_max_u32(mb);
    const int ex = (int)(mb >> 23) - 127; // floor(log2 max), -127 for zero and subnormals
    const int e2 = max(ex + 1 - 30, -126);
    const bool finite = mb < 0x7f800000u;
    step[m] = finite ? __uint_as_float((unsigned)(e2 + 127) << 23)
                     : __uint_as_float(0x7fc00000u);
    inv[m] = __uint_as_float((unsigned)(127 - e2) << 23);
  }
  // The planes of four tiles at a time, [tile][row][digit][64 k] bytes, in a
  // corner of LDS private to the wavefront (after the meeting place of the
  // k-slices): group q + 1 is cut and written once the reads of group q have
  // been issued (LDS serves a wavefront's requests in order).
  constexpr int NG = VEC ? XV : 1;      // groups of tiles
  constexpr int TG = VEC ? 4 : U;       // tiles per group
  static_assert(TG <= 4, "a group of planes holds four tiles");
  unsigned char *planes =
      reinterpret_cast<unsigned char *>(lds + (size_t)nwaves * M * 33) +
      (size_t)wave * (4 * M * kDigitBytesPerTile);
  auto cut_group = [&](int q) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      if constexpr (VEC) {
        // X + 0x00808080: the low three bytes are the balanced digits with their
        // sign bits flipped, the top byte is the fourth digit as it is
        unsigned y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = (int)__builtin_rintf(x[m][q][e] * inv[m]); // exact: |.| < 2^30
          y[e] = (unsigned)r + 0x00808080u;
        }
        // 4 x 4 byte transpose: a dword per plane
        const unsigned ta = __builtin_amdgcn_perm(y[1], y[0], 0x05010400u);
        const unsigned tb = __builtin_amdgcn_perm(y[3], y[2], 0x05010400u);
        const unsigned tc = __builtin_amdgcn_perm(y[1], y[0], 0x07030602u);
        const unsigned td = __builtin_amdgcn_perm(y[3], y[2], 0x07030602u);
        const unsigned d0 = __builtin_amdgcn_perm(tb, ta, 0x05040100u) ^ 0x80808080u;
        const unsigned d1 = __builtin_amdgcn_perm(tb, ta, 0x07060302u) ^ 0x80808080u;
        const unsigned d2 = __builtin_amdgcn_perm(td, tc, 0x05040100u) ^ 0x80808080u;
        const unsigned d3 = __builtin_amdgcn_perm(td, tc, 0x07060302u);
        // tile lane / 16 of the group, bytes 4 (lane % 16) .. + 3 of its planes
        unsigned *p = reinterpret_cast<unsigned *>(planes +
                                                   ((lane >> 4) * M + m) * kDigitBytesPerTile) +
                      (lane & 15);
        p[0] = d0;
        p[kTileK / 4] = d1;
        p[2 * kTileK / 4] = d2;
        p[3 * kTileK / 4] = d3;
      } else {
#pragma unroll
        for (int t = 0; t < U; ++t) { // one k per tile and lane
          const int r = (int)__builtin_rintf(x[m][t][0] * inv[m]);
          const unsigned z = ((unsigned)r + 0x00808080u) ^ 0x00808080u;
          unsigned char *p = planes + (t * M + m) * kDigitBytesPerTile + lane;
          p[0] = (unsigned char)z;
          p[kTileK] = (unsigned char)(z >> 8);
          p[2 * kTileK] = (unsigned char)(z >> 16);
          p[3 * kTileK] = (unsigned char)(z >> 24);
        }
      }
    }
  };
  auto lds_turn = [] { // this wavefront's LDS writes before its LDS reads that follow
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  // ---- the matrix cores: a weight tile as it lies is the A operand (16
  // channels x 64 k), the 4 M digit planes of the tile are columns of B: column
  // 4 m + d, lane (k / 16, column) reading 16 bytes.  One instruction per tile
  // and matrix multiplies every row and digit; the int32 sums stay exact over
  // the run (at most 16 x 64 products of 2^14).
  typedef int v4i32 __attribute__((ext_vector_type(4)));
  constexpr int COLS = kDigits * M;
  static_assert(COLS <= 16, "the digit planes of all rows are the 16 columns of one B operand");
  const int col = lane & 15, kq = lane >> 4;
  const unsigned char *my_b = planes + min(col, COLS - 1) * kTileK + 16 * kq;
  v4i32 c0 = {0, 0, 0, 0}, c1 = {0, 0, 0, 0}; // HS: c1 collects the pairs' second tiles
  cut_group(0);
#pragma unroll
  for (int q = 0; q < NG; ++q) {
    lds_turn();
    v4i32 b[TG];
#pragma unroll
    for (int t = 0; t < TG; ++t)
      b[t] = *reinterpret_cast<const v4i32 *>(my_b + t * (M * kDigitBytesPerTile));
    if (q + 1 < NG) {
      lds_turn();
      cut_group(q + 1);
    }
    if constexpr (HS) {
#pragma unroll
      for (int jp = 0; jp < 2; ++jp) { // the pairs 2 q and 2 q + 1
        const int u = 2 * q + jp;
        if (u < P) {
          if (t0 + 2 * u < t1) {
            const v4i32 wv = {wa[u < P ? u : 0].x, wa[u < P ? u : 0].y, wa[u < P ? u : 0].z,
                              wa[u < P ? u : 0].w};
            // rows of the other half of the lanes belong to the pair's second tile
            c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv, b[2 * jp], c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv, b[2 * jp + 1], c1, 0, 0, 0);
          }
        }
      }
    } else {
#pragma unroll
      for (int t = 0; t < TG; ++t) {
        const int u = TG * q + t;
        if (u < U) {
          if (t0 + u < t1) {
            const v4i32 wv = {wa[u < U ? u : 0].x, wa[u < U ? u : 0].y, wa[u < U ? u : 0].z,
                              wa[u < U ? u : 0].w};
            c0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv, b[t], c0, 0, 0, 0);
            if (DUAL) {
              const int ud = DUAL && u < U ? u : 0;
              const v4i32 wu = {wb[ud].x, wb[ud].y, wb[ud].z, wb[ud].w};
              c1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wu, b[t], c1, 0, 0, 0);
            }
          }
        }
      }
    }
  }
  // Lane (kq, col) holds the sums of channels 4 kq + i for its column.  Scale
  // by the column's step (step of row col / 4 times 256^(col % 4)), then the
  // four digits of a row, which sit in neighbouring lanes, are added up in the
  // lane of digit 0.
  float colscale = 0.f;
#pragma unroll
  for (int m = 0; m < M; ++m) {
    colscale = col == 4 * m ? step[m] : colscale;
    colscale = col == 4 * m + 1 ? step[m] * 256.0f : colscale;
    colscale = col == 4 * m + 2 ? step[m] * 65536.0f : colscale;
    colscale = col == 4 * m + 3 ? step[m] * 16777216.0f : colscale;
  }
  auto digits_sum = [](float v) { // row_shl:1..3: lanes col + 1, col + 2, col + 3
    return (v + dpp_f<0x101>(v)) + (dpp_f<0x102>(v) + dpp_f<0x103>(v));
  };
  float f0[4], f1[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (HS) {
      // channels 8 half + j: row j of the first tiles' product and row 8 + j of
      // the second tiles' (or the other way round for the other half)
      const bool first = (kq >> 1) == half;
      f0[i] = sum_xor<32>(digits_sum((float)(first ? c0[i] : c1[i]) * colscale));
      f1[i] = 0.f;
    } else {
      f0[i] = digits_sum((float)c0[i] * colscale);
      f1[i] = DUAL ? digits_sum((float)c1[i] * colscale) : 0.f;
    }
  }
#pragma unroll
  for (int m = 0; m < M; ++m)
    if (NORM)
      ss[m] = wave_sum(ss[m]);

  // ---- hand the sums over in LDS: [row][channel], the layout the k-slices
  // meet in; lane (kq, 4 m) has row m of channels 4 kq .. 4 kq + 3 -------------
  float acc0[M], acc1[M];
  {
    float *mine = lds + (size_t)wave * M * 33;
    const int mrow = col >> 2;
    if (col < COLS && (col & 3) == 0 && (!HS || kq < 2)) {
      const int ch = HS ? 8 * half + 4 * kq : 4 * kq;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        mine[mrow * 33 + ch + i] = f0[i];
        if (DUAL)
          mine[mrow * 33 + 16 + ch + i] = f1[i];
      }
    }
    if (NORM && lane == 0) {
#pragma unroll
      for (int m = 0; m < M; ++m)
        mine[m * 33 + 32] = ss[m];
    }
  }
  if (a.KS > 1) {
    __syncthreads();
    if (ks != 0)
      return;
  } else {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  if (lane < kTileN) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float r0 = 0.f, r1 = 0.f, rs = 0.f;
      for (int s = 0; s < a.KS; ++s) {
        const float *o = lds + (size_t)(wave + s) * M * 33 + m * 33;
        r0 += o[lane];
        if (DUAL)
          r1 += o[16 + lane];
        if (NORM)
          rs += o[32];
      }
      acc0[m] = r0;
      acc1[m] = r1;
      ss[m] = rs;
    }
  }
  if (writer) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      if (m < a.rows) {
        float v0 = acc0[m], v1 = acc1[m];
        if (NORM) {
          const float r = fast_rsqrt(ss[m] * a.norm_inv_k + a.norm_eps);
          v0 *= r;
          v1 *= r;
        }
        finish<M, EPI>(a, m, n, v0, v1, epi);
      }
    }
  }
}

BH_VARIANT_FAMILY(DigitsFamily, "gemv_w8a32_digits_kernel");

// the meeting place of the k-slices and, per wavefront, the planes of four tiles
constexpr size_t digits_lds_bytes(int waves, int M) {
  return sizeof(float) * waves * (size_t)M * 33 + (size_t)waves * 4 * M * kDigitBytesPerTile;
}

template <int M, int EPI, int PRO, int U, bool HS = false>
int launch_digits(const KernelArgs &ka, const GemvPlan &p, hipStream_t stream) {
  BH_NOTE_VARIANT(DigitsFamily, M, EPI, PRO, U, HS ? 1 : 0);
  auto kernel = gemv_w8a32_digits_kernel<M, EPI, PRO, U, HS>;
  const size_t lds = digits_lds_bytes(p.waves, M);
  if constexpr (digits_lds_bytes(kMaxWaves, M) > 48 * 1024) {
    static DynLdsOnce dyn_lds;
    BH_CHECK_HIP(ensure_dyn_lds(dyn_lds, reinterpret_cast<const void *>(kernel),
                                (int)digits_lds_bytes(kMaxWaves, M)));
  }
  hipLaunchKernelGGL(kernel, dim3(p.blocks << p.half_split), dim3(p.waves * kWave), lds,
                     stream, ka.W0, ka.W1, ka.A, ka.norm_w, ka.chunks, ka.KS,
                     ka.G | (p.half_split << 16), ka.groups, ka.K, ka.rows, ka);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

constexpr int kNoFit = -1000; // no compiled slot count holds the run

// the smallest compiled slot count that holds `tpw` tiles per wavefront
template <int M, int EPI, int PRO, bool HS, int... Us>
int launch_digits_fit(std::integer_sequence<int, Us...>, int64_t tpw, const KernelArgs &ka,
                    const GemvPlan &p, hipStream_t stream) {
  int rc = kNoFit;
  bool done = false;
  ((done || tpw > Us ? 0
                     : (done = true, rc = launch_digits<M, EPI, PRO, Us, HS>(ka, p, stream))),
   ...);
  return rc;
}

// Slot counts compiled per form: dense for one row, where a spare slot is a
// large part of a short run; coarser for 2 and 4 rows, and only as far as the
// activations (M per slot) and the weights fit in 128 registers.
template <int M> struct DigitSlots { // M = 4
  using Single = std::integer_sequence<int, 2, 3, 4, 6, 8>;
  using Dual = std::integer_sequence<int, 2, 3, 4, 6>;
};
template <> struct DigitSlots<2> {
  using Single = std::integer_sequence<int, 2, 3, 4, 6, 8, 10, 12>;
  using Dual = std::integer_sequence<int, 2, 3, 4, 6, 8>;
};
template <> struct DigitSlots<1> {
  using Single = std::integer_sequence<int, 2, 3, 4, 5, 6, 7, 8, 9, 10, 12, 14, 16>;
  using Dual = std::integer_sequence<int, 2, 3, 4, 5, 6, 7, 8, 9>;
};
using DigitSlotsSplit = std::integer_sequence<int, 4, 6, 8, 10>;
using DigitSlotsFold = std::integer_sequence<int, 2, 3, 4>; // 18 partials per tile in registers

// the slot count a run of `tpw` tiles gets from a list, 0 if none holds it
template <int... Us> int slots_for(std::integer_sequence<int, Us...>, int64_t tpw) {
  int v = 0;
  ((v = (v == 0 && tpw <= Us) ? Us : v), ...);
  return v;
}

int digit_slots(int M, const GemvPlan &p, bool dual, bool fold);

// Does a plan made for the digit-plane kernel have a compiled variant?
bool digits_fit(int M, const GemvPlan &p, bool dual, bool fold) {
  return digit_slots(M, p, dual, fold) != 0;
}

bool rows_on_digits() {
  static bool v = [] {
    const char *e = getenv("BUDDY_HIP_GEMV_ROW");
    return !(e && strcmp(e, "f32") == 0);
  }();
  return v;
}

template <int M, int EPI, int PRO, int U>
int launch_bcast(const KernelArgs &ka, const GemvPlan &p, hipStream_t stream) {
  auto kernel = gemv_w8a32_bcast_kernel<M, EPI, PRO, U>;
  hipLaunchKernelGGL(kernel, dim3(p.blocks << p.half_split), dim3(p.waves * kWave),
                     sizeof(float) * p.waves * (size_t)M * 33, stream, ka.W0, ka.W1, ka.A,
                     ka.norm_w, ka.chunks, ka.KS, ka.G | (p.half_split << 16), ka.groups,
                     ka.K, ka.rows, ka);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

template <int M, int EPI, int PRO, int U, int TN>
int launch_tn(const KernelArgs &ka, const GemvPlan &p, hipStream_t stream) {
  auto kernel = gemv_w8a32_kernel<M, EPI, PRO, U, TN>;
  static DynLdsOnce dyn_lds;
  BH_CHECK_HIP(ensure_dyn_lds(dyn_lds, reinterpret_cast<const void *>(kernel),
                              (int)(kMaxLdsBytes + 4096)));
  hipLaunchKernelGGL(kernel, dim3(p.blocks), dim3(p.waves * kWave), p.lds_bytes,
                     stream, ka);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

// 16-channel tiles run on the register-resident kernel; the 8- and 4-channel
// layouts (one row, one matrix) on the LDS-staged one.
template <int M, int EPI, int PRO>
int launch_one(const KernelArgs &ka, const GemvPlan &p, hipStream_t stream) {
  constexpr bool kDual = EPI == kEpiSiluMul;
  if (ka.tile_n != 16) {
    constexpr bool kNarrowOk = M == 1 && !kDual;
    if (!kNarrowOk)
      return fail(BUDDY_HIP_ERR_ARG, "gemv: %d-channel tiles need M = 1 and one matrix",
                  ka.tile_n);
    if (ka.tile_n == 8)
      return launch_tn<kNarrowOk ? 1 : M, kNarrowOk ? EPI : kEpiStore, PRO, 4, kNarrowOk ? 8 : 16>(ka, p, stream);
    return launch_tn<kNarrowOk ? 1 : M, kNarrowOk ? EPI : kEpiStore, PRO, 4, kNarrowOk ? 4 : 16>(ka, p, stream);
  }
  if constexpr (M <= 4) {
    if (p.on_digits) {
      // every tile of a wavefront's run is requested at once
      const int64_t tpw = ceil_div(p.chunks, p.KS); // tiles per wavefront
      int rc = kNoFit;
      if (p.half_split) {
        if constexpr (!kDual && PRO != kProAttn)
          rc = launch_digits_fit<M, EPI, PRO, true>(DigitSlotsSplit{}, tpw, ka, p, stream);
      } else if constexpr (PRO == kProAttn) {
        if constexpr (M == 1)
          rc = launch_digits_fit<1, EPI, PRO, false>(DigitSlotsFold{}, tpw, ka, p, stream);
      } else if constexpr (kDual) {
        rc = launch_digits_fit<M, EPI, PRO, false>(typename DigitSlots<M>::Dual{}, tpw, ka, p,
                                                 stream);
      } else {
        rc = launch_digits_fit<M, EPI, PRO, false>(typename DigitSlots<M>::Single{}, tpw, ka, p,
                                                 stream);
      }
      if (rc != kNoFit)
        return rc;
      return fail(BUDDY_HIP_ERR_ARG, "gemv: no digit-plane variant for %lld tiles per wavefront",
                  (long long)tpw);
    }
  }
  constexpr int kRing = M == 1 ? (kDual ? 6 : 8) : M <= 4 ? 4 : M == 8 ? 2 : 1;
  return launch_bcast<M, EPI, PRO, kRing>(ka, p, stream);
}

template <int M>
int launch_m(const GemvArgs &a, const KernelArgs &ka, const GemvPlan &p,
             hipStream_t stream) {
  const bool norm = a.norm_w != nullptr;
  if (a.attn_acc) { // only the o_proj of a decode step: M = 1, residual add
    if (M == 1 && a.epilogue == kEpiAccum)
      return launch_one<1, kEpiAccum, kProAttn>(ka, p, stream);
    return fail(BUDDY_HIP_ERR_ARG, "gemv: attention input needs M=1 + ACCUM");
  }
  switch (a.epilogue) {
  case kEpiStore:
    return norm ? launch_one<M, kEpiStore, kProNorm>(ka, p, stream)
                : launch_one<M, kEpiStore, kProPlain>(ka, p, stream);
  case kEpiAccum:
    return norm ? launch_one<M, kEpiAccum, kProNorm>(ka, p, stream)
                : launch_one<M, kEpiAccum, kProPlain>(ka, p, stream);
  case kEpiSiluMul:
    return norm ? launch_one<M, kEpiSiluMul, kProNorm>(ka, p, stream)
                : launch_one<M, kEpiSiluMul, kProPlain>(ka, p, stream);
  }
  return fail(BUDDY_HIP_ERR_ARG, "gemv: unknown epilogue %d", a.epilogue);
}

// Which matrix-core kernel takes batches of 5..16 rows: 0 = int8 (default),
// 1 = bf16 (three bf16 terms per activation: every f32 bit).  The environment
// variable BUDDY_HIP_GEMV_BATCH=bf16 sets the default, read once per process;
// buddy_hip_set_gemv_batch_kernel changes it between calls.
std::atomic<int> g_batch_kernel{-1};
bool batch_bf16() {
  int k = g_batch_kernel.load(std::memory_order_relaxed);
  if (k < 0) {
    const char *e = getenv("BUDDY_HIP_GEMV_BATCH");
    k = e && strcmp(e, "bf16") == 0;
    int expected = -1; // a setter that ran meanwhile wins
    if (!g_batch_kernel.compare_exchange_strong(expected, k))
      k = expected;
  }
  return k == 1;
}
// The cut of a launch of up to four rows (or of the f32 kernel for more): the
// digit-plane kernel, cut as for one row, when it has a variant for the run a
// wavefront gets; otherwise the f32 kernel with its own cut.
GemvPlan choose_plan(int mt, int64_t K, int64_t N, bool dual, int tile_n, bool fold,
                     bool rows_aligned) {
  GemvPlan p = make_plan(mt, K, N, dual, tile_n, fold);
  if (mt <= 4 && tile_n == 16 && rows_aligned && rows_on_digits()) {
    GemvPlan q = make_plan(1, K, N, dual, tile_n, fold);
    if (digits_fit(mt, q, dual, fold)) {
      q.on_digits = true;
      p = q;
    }
  }
  return p;
}

// the slot count the digit-plane kernel is launched with for a plan, 0 if none
int digit_slots(int M, const GemvPlan &p, bool dual, bool fold) {
  const int64_t tpw = ceil_div(p.chunks, p.KS);
  if (p.half_split)
    return (dual || fold) ? 0 : slots_for(DigitSlotsSplit{}, tpw);
  if (fold)
    return M == 1 ? slots_for(DigitSlotsFold{}, tpw) : 0;
  if (dual)
    return M == 1   ? slots_for(DigitSlots<1>::Dual{}, tpw)
           : M == 2 ? slots_for(DigitSlots<2>::Dual{}, tpw)
                    : slots_for(DigitSlots<4>::Dual{}, tpw);
  return M == 1   ? slots_for(DigitSlots<1>::Single{}, tpw)
         : M == 2 ? slots_for(DigitSlots<2>::Single{}, tpw)
                  : slots_for(DigitSlots<4>::Single{}, tpw);
}

bool force_valu() {
  static bool v = getenv("BUDDY_HIP_GEMV_FORCE_VALU") != nullptr;
  return v;
}

int compiled_rows(int64_t M) {
  return M <= 2 ? (int)M : M <= 4 ? 4 : M <= 8 ? 8 : 16;
}

} // namespace

int launch_gemv(const GemvArgs &a, hipStream_t stream) {
  BH_REQUIRE((a.A || a.attn_acc) && a.W0 && a.s0 && a.C, "gemv: null pointer");
  BH_REQUIRE(!a.attn_acc || (a.attn_ml && a.pos_ptr && a.attn_nchunks > 0 &&
                             a.attn_chunk > 0 && a.head_dim > 0 &&
                             a.head_dim % 4 == 0 && is_pow2(a.head_dim) &&
                             a.K % a.head_dim == 0),
             "gemv: incomplete attention-partials input");
  BH_REQUIRE(a.M >= 1 && a.M <= 16, "gemv: M=%d outside 1..16", a.M);
  BH_REQUIRE(a.K > 0 && a.N > 0 && a.K < (1 << 30) && a.N < (1 << 30),
             "gemv: bad shape K=%lld N=%lld", (long long)a.K, (long long)a.N);
  BH_REQUIRE((a.attn_acc || a.lda >= a.K) && a.ldc >= a.N,
             "gemv: row stride below row length");
  const bool dual = a.epilogue == kEpiSiluMul;
  BH_REQUIRE(!dual || (a.W1 && a.s1), "gemv: SiLU*mul needs two matrices");
  BH_REQUIRE((reinterpret_cast<uintptr_t>(a.W0) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(a.W1) & 15) == 0,
             "gemv: packed weights must be 16-byte aligned");
  BH_REQUIRE(!a.norm_w || (reinterpret_cast<uintptr_t>(a.norm_w) & 15) == 0,
             "gemv: norm weight must be 16-byte aligned");
  // batches of 5..16 rows go to the matrix cores (int8 ones by default) when the
  // activations can be read as aligned 16-byte pieces; up to four rows the f32
  // FMA kernel (1 + M instructions per weight) is quicker, and it takes whatever
  // is unaligned
  if (a.M >= 5 && !a.attn_acc && !force_valu() && a.tile_n == 16 && a.K >= 4 &&
      (a.K & 3) == 0 && (a.lda & 3) == 0 &&
      (reinterpret_cast<uintptr_t>(a.A) & 15) == 0 &&
      (!a.norm_w || (reinterpret_cast<uintptr_t>(a.norm_w) & 15) == 0))
  {
    if (a.argmax_groups)
      *a.argmax_groups = 0;
    return batch_bf16() ? launch_gemv_mfma(a, stream) : launch_gemv_i8(a, stream);
  }
  // the kernel is compiled for 1, 2, 4, 8 and 16 rows; extra rows are zero-
  // filled in LDS and never stored
  const int mt = compiled_rows(a.M);
  BH_REQUIRE(a.tile_n == 16 || a.tile_n == 8 || a.tile_n == 4,
             "gemv: tile_n=%d (16, 8 or 4)", a.tile_n);
  const bool fold = a.attn_acc != nullptr;
  // (its activation rows are read as aligned 16-byte pieces; the norm weight,
  // read the same way, was required to be 16-byte aligned above, so that a
  // piece that starts inside the array ends inside its last 16-byte line)
  const bool rows_aligned =
      fold || ((reinterpret_cast<uintptr_t>(a.A) & 15) == 0 && (a.M == 1 || (a.lda & 3) == 0));
  const GemvPlan p = choose_plan(mt, a.K, a.N, dual, a.tile_n, fold, rows_aligned);
  KernelArgs ka;
  ka.A = a.A;
  ka.W0 = reinterpret_cast<const int4 *>(a.W0);
  ka.W1 = reinterpret_cast<const int4 *>(a.W1);
  ka.s0 = a.s0;
  ka.s1 = a.s1;
  ka.bias = a.bias;
  ka.norm_w = a.norm_w;
  ka.C = a.C;
  ka.lda = a.lda;
  ka.ldc = a.ldc;
  ka.norm_eps = a.norm_eps;
  ka.norm_inv_k = a.norm_inv_k;
  ka.K = (int)a.K;
  ka.N = (int)a.N;
  ka.groups = (int)p.groups;
  ka.chunks = (int)p.chunks;
  ka.G = p.G;
  BH_REQUIRE(is_pow2(p.KS), "gemv: %d k-slices (the kernels shift by their count)", p.KS);
  ka.KS = p.KS;
  ka.tiles_per_round = p.tiles_per_round;
  ka.tile_n = a.tile_n;
  ka.rows = a.M;
  // the per-group maxima come from the f32 kernel of one row (whole groups per
  // workgroup); other cuts leave the row to the caller
  const bool emit = a.argmax_v && a.argmax_i && mt == 1 && a.tile_n == 16 && !p.on_digits &&
                    !p.half_split && !fold && a.epilogue == kEpiStore;
  ka.cand_v = emit ? a.argmax_v : nullptr;
  ka.cand_i = emit ? a.argmax_i : nullptr;
  if (a.argmax_groups)
    *a.argmax_groups = emit ? (int)p.groups : 0;
  ka.attn_acc = a.attn_acc;
  ka.attn_ml = a.attn_ml;
  ka.pos_ptr = a.pos_ptr;
  ka.attn_nchunks = a.attn_nchunks;
  ka.attn_chunk = a.attn_chunk;
  ka.attn_used = a.attn_used > 0 ? std::min(a.attn_used, a.attn_nchunks) : a.attn_nchunks;
  ka.head_dim = a.head_dim;
  switch (mt) {
  case 1: return launch_m<1>(a, ka, p, stream);
  case 2: return launch_m<2>(a, ka, p, stream);
  case 4: return launch_m<4>(a, ka, p, stream);
  case 8: return launch_m<8>(a, ka, p, stream);
  default: return launch_m<16>(a, ka, p, stream);
  }
}

} // namespace bh

extern "C" {

int buddy_hip_set_gemv_batch_kernel(int kernel) try {
  BH_REQUIRE(kernel == BUDDY_HIP_GEMV_BATCH_INT8 || kernel == BUDDY_HIP_GEMV_BATCH_BF16,
             "set_gemv_batch_kernel: %d (0 = int8, 1 = bf16)", kernel);
  bh::g_batch_kernel.store(kernel, std::memory_order_relaxed);
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_set_gemv_batch_kernel")

int buddy_hip_gemv_w8a32_plan(int64_t M, int64_t K, int64_t N, unsigned flags,
                              buddy_hip_gemv_plan *out) try {
  BH_REQUIRE(out, "gemv_w8a32_plan: null result");
  BH_REQUIRE(M >= 1 && M <= 16, "gemv_w8a32_plan: M=%lld outside 1..16", (long long)M);
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30),
             "gemv_w8a32_plan: bad shape K=%lld N=%lld", (long long)K, (long long)N);
  const bool dual = flags & BUDDY_HIP_PLAN_TWO_MATRICES, fold = flags & BUDDY_HIP_PLAN_FOLD_INPUT;
  BH_REQUIRE(!(fold && (M != 1 || dual)), "gemv_w8a32_plan: folded input is one row, one matrix");
  *out = buddy_hip_gemv_plan{};
  const bool aligned = !(flags & BUDDY_HIP_PLAN_UNALIGNED_ROWS);
  if (M >= 5 && !fold && !bh::force_valu() && (K & 3) == 0 && aligned) {
    out->kernel = bh::batch_bf16() ? BUDDY_HIP_PLAN_BATCH_BF16 : BUDDY_HIP_PLAN_BATCH_INT8;
    out->rows_compiled = 16;
    return BUDDY_HIP_OK; // those kernels cut their launch by what the device holds
  }
  const int mt = bh::compiled_rows(M);
  const bh::GemvPlan p = bh::choose_plan(mt, K, N, dual, 16, fold, aligned);
  out->kernel = p.on_digits ? BUDDY_HIP_PLAN_DIGITS : BUDDY_HIP_PLAN_F32;
  out->rows_compiled = mt;
  out->channel_groups = (int32_t)p.groups;
  out->tiles = (int32_t)p.chunks;
  out->groups_per_workgroup = p.G;
  out->k_slices = p.KS;
  out->wavefronts = p.waves;
  out->workgroups = p.blocks << p.half_split;
  out->split = p.half_split;
  out->tiles_per_wavefront = (int32_t)bh::ceil_div(p.chunks, p.KS);
  out->slots = p.on_digits ? bh::digit_slots(mt, p, dual, fold) : 0;
  out->lds_bytes = p.on_digits ? (int64_t)bh::digits_lds_bytes(p.waves, mt)
                               : (int64_t)(sizeof(float) * p.waves * (size_t)mt * 33);
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_gemv_w8a32_plan")

int buddy_hip_linear_w8a32(const buddy_hip_linear_desc *d,
                           buddy_hip_stream stream) try {
  BH_REQUIRE(d, "linear_w8a32: null descriptor");
  bh::GemvArgs a;
  a.A = d->A;
  a.lda = d->lda;
  a.W0 = d->W0;
  a.W1 = d->W1;
  a.s0 = d->scale0;
  a.s1 = d->scale1;
  a.bias = d->bias;
  a.norm_w = d->norm_w;
  a.norm_eps = d->norm_eps;
  a.norm_inv_k = d->K > 0 ? 1.0f / (float)d->K : 0.f;
  a.C = d->C;
  a.ldc = d->ldc;
  a.M = (int)d->M;
  a.K = d->K;
  a.N = d->N;
  a.epilogue = d->epilogue;
  a.tile_n = d->tile_n ? d->tile_n : 16;
  BH_REQUIRE(d->M >= 1 && d->M <= 16, "linear_w8a32: M=%lld outside 1..16",
             (long long)d->M);
  BH_REQUIRE(!(d->bias && d->epilogue != BUDDY_HIP_EPI_STORE),
             "linear_w8a32: bias only with the STORE epilogue");
  return bh::launch_gemv(a, bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_linear_w8a32")

size_t buddy_hip_mlp_block_workspace_bytes(int64_t M, int64_t inter) {
  if (M < 1 || M > 16 || inter < 1)
    return 0;
  return (sizeof(float) * (size_t)M * (size_t)inter + 255) & ~(size_t)255;
}

int buddy_hip_mlp_block_w8a32(const buddy_hip_mlp_block_desc *d, buddy_hip_stream stream) try {
  BH_REQUIRE(d, "mlp_block_w8a32: null descriptor");
  BH_REQUIRE(d->x && d->gate && d->gate_scale && d->up && d->up_scale && d->down &&
                 d->down_scale && d->y && d->workspace,
             "mlp_block_w8a32: null pointer");
  BH_REQUIRE(d->M >= 1 && d->M <= 16, "mlp_block_w8a32: M=%lld outside 1..16", (long long)d->M);
  BH_REQUIRE(d->hidden > 0 && d->inter > 0 && d->ldx >= d->hidden && d->ldy >= d->hidden,
             "mlp_block_w8a32: bad shape or row stride");
  BH_REQUIRE(d->workspace_bytes >= buddy_hip_mlp_block_workspace_bytes(d->M, d->inter) &&
                 (reinterpret_cast<uintptr_t>(d->workspace) & 15) == 0,
             "mlp_block_w8a32: workspace of %zu bytes (16-byte aligned) needed, %zu given",
             buddy_hip_mlp_block_workspace_bytes(d->M, d->inter), d->workspace_bytes);
  hipStream_t s = bh::as_stream(stream);
  float *h = static_cast<float *>(d->workspace); // [M, inter] between the two launches
  bh::GemvArgs g;
  g.A = d->x;
  g.lda = d->ldx;
  g.W0 = d->gate;
  g.s0 = d->gate_scale;
  g.W1 = d->up;
  g.s1 = d->up_scale;
  g.norm_w = d->norm_w;
  g.norm_eps = d->norm_eps;
  g.norm_inv_k = 1.0f / (float)d->hidden;
  g.C = h;
  g.ldc = d->inter;
  g.M = (int)d->M;
  g.K = d->hidden;
  g.N = d->inter;
  g.epilogue = bh::kEpiSiluMul;
  int rc = bh::launch_gemv(g, s);
  if (rc)
    return rc;
  bh::GemvArgs w;
  w.A = h;
  w.lda = d->inter;
  w.W0 = d->down;
  w.s0 = d->down_scale;
  w.C = d->y;
  w.ldc = d->ldy;
  w.M = (int)d->M;
  w.K = d->inter;
  w.N = d->hidden;
  w.epilogue = (d->flags & BUDDY_HIP_GEMV_ACCUMULATE) ? bh::kEpiAccum : bh::kEpiStore;
  return bh::launch_gemv(w, s);
} BH_CATCH_INT("buddy_hip_mlp_block_w8a32")

int buddy_hip_gemv_w8a32(const float *A, const int8_t *packed,
                         const float *scale, float *C, int64_t M, int64_t K,
                         int64_t N, unsigned flags, buddy_hip_stream stream) try {
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
    int rc = bh::launch_gemv(a, bh::as_stream(stream));
    if (rc)
      return rc;
  }
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_gemv_w8a32")
}
