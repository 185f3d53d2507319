// attn_prefill.hip -- causal GQA attention over a block of prompt tokens, and
// the RoPE + KV-cache write in front of it.
//
// Replaces flash_attention_for_cpu_prefill_op
// (frontend/Python/ops/tosa.py:4326-4810: q-blocks of 16, kv-blocks of 64,
// online softmax with m seeded at -1e30, out = acc / l) and, for a block of
// tokens, the RoPE / cache write of
// examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:51-59,88-142.
//
// The reference kernel is handed K and V already repeated to one copy per query
// head (tosa.py:4578-4579,4700); here the KV head is h / group, so the cache is
// read in place.  The causal structure is exploited: key blocks that lie wholly
// in a query block's future are skipped (they are exactly zero after softmax).
// Arithmetic is f32 throughout, on the f32 matrix cores.
#include "attn.h"

#include <type_traits>

namespace bh {
namespace {

constexpr int kD = 128;
constexpr int kQB = 16;            // query rows per block
constexpr int kKB = 16;            // key positions per step of a wavefront
constexpr int kKPitch = kD + 4;    // floats per key row in LDS (fragment reads hit every bank once)
constexpr int kOutPitch = kWave + 1;      // floats per accumulator register row of a partial output in LDS
constexpr int kSlotFloats = kKB * kKPitch; // a wavefront's part of LDS: a K block, later its partial output
static_assert(32 * kOutPitch <= kSlotFloats, "partial output must fit the slot");
constexpr float kSeedM = -1.0e30f; // tosa.py:4383

typedef float f32x4 __attribute__((ext_vector_type(4)));

struct PrefillArgs {
  const float *q;   // token t, head h at q + t*q_stride + h*q_hstride
  const float *k, *v; // [kv_heads, kv_stride rows, D]
  const float *mask;  // additive [q_len, k_len] or null (causal)
  float *out;         // token t, head h at out + t*o_stride + h*o_hstride
  int64_t q_stride, q_hstride, o_stride, o_hstride, kv_stride;
  int heads, group, q_len, k_len, q_offset; // query i sits at key position q_offset + i
  int nqb;                                  // query blocks of kQB rows
  int paired;                               // a workgroup takes a query block and its mirror image
  float scale;
};

// LDS of a workgroup, in floats: the Q fragments of its two query blocks, one
// slot per wavefront, the (max, sum) pairs of the partial results and which part
// each wavefront worked on.
constexpr int kQFloats = 2 * 8 * kWave * 4;
constexpr int lds_floats(int waves) { return kQFloats + waves * kSlotFloats + 2 * waves * kQB + waves; }

// One workgroup: two blocks of 16 query rows of one head, block j from the start
// and block j from the end, so that under the causal mask every workgroup has the
// same number of 16-key blocks before it (one query block alone would have
// between 1 and q_len / 16 of them, and a launch of one round would last as long
// as the longest).  The W wavefronts are dealt to the two query blocks in
// proportion to their key blocks; those of a query block split its key blocks
// into equal contiguous shares, each with its own running (max, sum, output), and
// the partial results meet in LDS at the end.  W = 8 and pairs while the launch
// is at most one workgroup per compute unit.  A longer launch balances itself
// better with many workgroups of unequal length, the longest first: then a
// workgroup takes one query block (part 0 empty), W = 4, two workgroups per
// compute unit, so that one's staging and merge overlap the other's key loop.
// All products run on the f32 matrix cores (16x16x4):
//   S^T[key, query] = K . Q^T   (contraction over d; in step 4J + e a lane
//                                supplies d = 16 J + 4 (lane/16) + e, for K and
//                                Q alike)
//   O^T[d, query]  += V^T . P^T (contraction over the key; the S^T accumulator
//                                registers ARE the P^T operand of step r: a
//                                lane holds keys 4*(lane/16) + r of query lane%16)
// so the scores never leave the registers between the two products.
template <int kAttnWaves>
__global__ void __launch_bounds__(kAttnWaves *kWave) __attribute__((amdgpu_waves_per_eu(2, 2)))
attn_prefill_kernel(const float *p_k, const float *p_v, const float *p_mask, int64_t p_kv_stride,
                    int p_group, int p_nqb, int p_q_len, int p_k_len, int p_q_offset,
                    PrefillArgs rest) {
  static_assert(kAttnWaves == 4 || kAttnWaves == 8, "wavefronts per workgroup");
  // what comes before the first fetch arrives in SGPRs (this file is built with
  // -amdgpu-kernarg-preload-count); p_group carries the group size, whether the
  // launch is paired and the multiplier that divides a head index by the group
  PrefillArgs a = rest;
  a.k = p_k;
  a.v = p_v;
  a.mask = p_mask;
  a.kv_stride = p_kv_stride;
  a.group = p_group & 0xfff;
  a.paired = (p_group >> 12) & 1;
  a.nqb = p_nqb;
  a.q_len = p_q_len;
  a.k_len = p_k_len;
  a.q_offset = p_q_offset;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  f32x4 *q_s = reinterpret_cast<f32x4 *>(lds);          // [2][8][64]: part, J, lane
  float *slot_s = lds + kQFloats;                  // [kAttnWaves][kSlotFloats]
  float *m_s = slot_s + kAttnWaves * kSlotFloats;  // [kAttnWaves][kQB]
  float *l_s = m_s + kAttnWaves * kQB;
  int *part_s = reinterpret_cast<int *>(l_s + kAttnWaves * kQB); // [kAttnWaves]: part, or -1

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = blockIdx.x, kvh = (int)(((unsigned)h * (unsigned)(p_group >> 13)) >> 16); // h / group
  const int qi = lane & 15, lg = lane >> 4; // query of this lane; lane group
  // part 0: query block blockIdx.y, part 1: its mirror image (the same block in
  // the middle of an odd number of blocks: then part 0 is empty)
  // (unpaired launches: one query block per workgroup, part 0 stays empty; ids
  // start in order, so the blocks that see the most keys come first and the
  // short ones fill the gaps at the end)
  const int qb1 = a.nqb - 1 - (int)blockIdx.y;
  const bool single = !a.paired || qb1 == (int)blockIdx.y;
  int q0[2], nq[2], nb[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    q0[p] = (p ? qb1 : (int)blockIdx.y) * kQB;
    nq[p] = min(kQB, a.q_len - q0[p]);
    // last key any query of the block may see
    const int k_last = a.mask ? a.k_len - 1 : min(a.k_len - 1, a.q_offset + q0[p] + nq[p] - 1);
    nb[p] = k_last / kKB + 1;
  }
  if (single)
    nb[0] = 0;
  const int total = nb[0] + nb[1];
  // wavefronts [0, wa) work on part 0, the others on part 1
  const int wa = nb[0] ? max(1, min(kAttnWaves - 1, (kAttnWaves * nb[0] + total / 2) / total)) : 0;
  // key blocks [b0, b1) of its part (fewer than 2^16 blocks, at most 8 shares)
  const int part = wave < wa ? 0 : 1;
  const unsigned sn = part ? kAttnWaves - wa : wa, si = part ? wave - wa : wave;
  const int b0 = (int)((unsigned)nb[part] * si / sn), b1 = (int)((unsigned)nb[part] * (si + 1) / sn);
  const int pq0 = q0[part], pnq = nq[part];

  const float *kbase = a.k + (int64_t)kvh * a.kv_stride * kD;
  const float *vbase = a.v + (int64_t)kvh * a.kv_stride * kD;
  float *ks = slot_s + wave * kSlotFloats;

  // K and V of a key block: 16 loads, issued by hand one block ahead of the
  // block being multiplied (the compiler sinks ordinary loads down to their
  // first use, which leaves the matrix cores waiting out every L2 round trip).
  // A fetch is always exactly 16 loads, so that vmcnt(16) means "everything but
  // the newest fetch has arrived".  The registers of a fetch are only read after
  // such a wait names them; the build refuses scratch use in this file.
  struct Frag {
    f32x4 k[8], v[8];
  };
  auto issue = [](f32x4 &dst, const float *p) {
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
  };
  auto arrived = [](Frag &f, auto n_in_flight) { // at most N loads still in flight
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(decltype(n_in_flight)::value) : "memory");
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      asm volatile("" : "+v"(f.k[j])::"memory");
      asm volatile("" : "+v"(f.v[j])::"memory");
    }
  };
  auto fetch = [&](int b, Frag &f) {
    const int p0 = b * kKB;
    // K rows as they lie: load i is keys p0 + 2 i and p0 + 2 i + 1, a lane's four
    // values d = 4 (lane % 32) + 0..3 (half a wavefront reads one whole row)
#pragma unroll
    for (int i = 0; i < 8; ++i)
      issue(f.k[i], kbase + (int64_t)min(p0 + 2 * i + (lane >> 5), a.k_len - 1) * kD +
                        (lane & 31) * 4);
    // V^T fragments: key p0 + 4*lg + r, d = 64*half + 4*(lane%16) + 0..3
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float *vs = vbase + (int64_t)min(p0 + 4 * lg + r, a.k_len - 1) * kD + 4 * qi;
      issue(f.v[2 * r], vs);
      issue(f.v[2 * r + 1], vs + 64);
    }
  };
  Frag fa, fb;
  if (b0 < b1)
    fetch(b0, fa); // on its way while the queries are staged

  { // Q^T fragments into LDS: the 16 (part, J) pieces are dealt to the wavefronts
    constexpr int kPieces = 16 / kAttnWaves;
#pragma unroll
    for (int t = 0; t < kPieces; ++t) {
      const int piece = wave * kPieces + t, p = piece >> 3, J = piece & 7;
      const int qrow = q0[p] + min(qi, nq[p] - 1); // rows past the end repeat the last
      const float *src = a.q + (int64_t)qrow * a.q_stride + (int64_t)h * a.q_hstride + lg * 4;
      q_s[(p * 8 + J) * kWave + lane] = *reinterpret_cast<const f32x4 *>(src + 16 * J);
    }
  }
  __syncthreads();

  float qf[32]; // Q^T fragment: qf[4J + e] is d = 16 J + 4 lg + e of this lane's query
#pragma unroll
  for (int J = 0; J < 8; ++J) {
    const f32x4 v = q_s[(part * 8 + J) * kWave + lane];
    qf[4 * J] = v[0];
    qf[4 * J + 1] = v[1];
    qf[4 * J + 2] = v[2];
    qf[4 * J + 3] = v[3];
  }
  float m_run = kSeedM, l_run = 0.f; // l_run: this lane's share of the row sum
  f32x4 acc[8]; // O^T: acc[2*e + half][r] is d = 64*half + 4*(4*lg + r) + e
#pragma unroll
  for (int i = 0; i < 8; ++i)
    acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto block = [&](const Frag &f, int b) {
    // The K rows turn into fragments through this wavefront's part of LDS: lane
    // (qi, lg) reads d = 16 J + 4 lg + 0..3 of key p0 + qi.  (Fetched in that
    // layout straight from memory, a load touches 16 rows with every 16 lanes.)
#pragma unroll
    for (int i = 0; i < 8; ++i)
      *reinterpret_cast<f32x4 *>(ks + (2 * i + (lane >> 5)) * kKPitch + (lane & 31) * 4) = f.k[i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // ---- S^T block: keys x queries ------------------------------------------
    // four independent partial sums: a matrix instruction that adds to the
    // result of the one before it cannot issue until that one has finished
    f32x4 sp[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      sp[e] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const f32x4 kf = *reinterpret_cast<const f32x4 *>(ks + qi * kKPitch + 16 * j + 4 * lg);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        sp[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[e], qf[4 * j + e], sp[e], 0, 0, 0);
    }
    // (the next block's rows are written after these reads: one wavefront's LDS
    // operations complete in order)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const f32x4 st = (sp[0] + sp[1]) + (sp[2] + sp[3]);
    // lane holds keys p0 + 4*lg + r of query pq0 + qi
    const int p0 = b * kKB;
    float sc[4];
    float m_blk = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int kp = p0 + 4 * lg + r;
      float x = st[r] * a.scale;
      bool ok = qi < pnq && kp < a.k_len;
      if (ok) {
        if (a.mask)
          x += a.mask[(int64_t)(pq0 + qi) * a.k_len + kp];
        else
          ok = kp <= a.q_offset + pq0 + qi;
      }
      sc[r] = ok ? x : -INFINITY;
      m_blk = fmaxf(m_blk, sc[r]);
    }
    m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 16, 64));
    m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32, 64));
    const float m_new = fmaxf(m_run, m_blk); // m_run is finite, so m_new is
    const float alpha = expf(m_run - m_new);
    float pr[4];
    float l_blk = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      pr[r] = expf(sc[r] - m_new);
      l_blk += pr[r];
    }
    l_run = l_run * alpha + l_blk;
    m_run = m_new;
    // ---- O^T += V^T . P^T -----------------------------------------------------
#pragma unroll
    for (int i = 0; i < 8; ++i)
      acc[i] *= alpha;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const f32x4 vv = f.v[2 * r + half];
        acc[0 + half] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv[0], pr[r], acc[0 + half], 0, 0, 0);
        acc[2 + half] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv[1], pr[r], acc[2 + half], 0, 0, 0);
        acc[4 + half] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv[2], pr[r], acc[4 + half], 0, 0, 0);
        acc[6 + half] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv[3], pr[r], acc[6 + half], 0, 0, 0);
      }
    }
  };
  if (b0 < b1) {
    // fa holds (in flight) block b; nothing is fetched past the end of the share
    int b = b0;
    for (; b + 2 < b1; b += 2) {
      fetch(b + 1, fb);
      arrived(fa, std::integral_constant<int, 16>{});
      block(fa, b);
      fetch(b + 2, fa);
      arrived(fb, std::integral_constant<int, 16>{});
      block(fb, b + 1);
    }
    if (b + 1 < b1) {
      fetch(b + 1, fb);
      arrived(fa, std::integral_constant<int, 16>{});
      block(fa, b);
      arrived(fb, std::integral_constant<int, 0>{});
      block(fb, b + 1);
    } else {
      arrived(fa, std::integral_constant<int, 0>{});
      block(fa, b);
    }
    // this wavefront's row sums: the four lane groups hold different keys
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    // (rows of kWave + 1 floats: the merge reads them by column)
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        ks[(i * 4 + r) * kOutPitch + lane] = acc[i][r];
    if (lg == 0) {
      m_s[wave * kQB + qi] = m_run;
      l_s[wave * kQB + qi] = l_run;
    }
  }
  if (lane == 0)
    part_s[wave] = b0 < b1 ? part : -1;
  __syncthreads();

  // ---- merge the partial results (the reference's combine rule, in wave order).
  // A thread finishes four consecutive d of one query per part, so that a
  // wavefront writes two whole rows of the output at a time: value d = 64 half + 16 lg +
  // 4 r + e of query q is accumulator 2 e + half, register r of lane 16 lg + q.
  const int c = lane & 31;
  const int m_half = c >> 4, m_lg = (c >> 2) & 3, m_r = c & 3;
#pragma unroll
  for (int it = 0; it < 2 * (8 / kAttnWaves); ++it) {
    const int p = it & 1;
    const int mq = (2 * wave + (lane >> 5)) * (8 / kAttnWaves) + (it >> 1);
    if ((single && p == 0) || mq >= nq[p])
      continue;
    float wgt[kAttnWaves], m_w[kAttnWaves], m_all = kSeedM, l_all = 0.f;
    bool has[kAttnWaves];
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) {
      // (what a wavefront of the other part, or one without a share, left in its
      // slot is not a number to be multiplied by zero: it is not looked at)
      has[w] = part_s[w] == p;
      m_w[w] = has[w] ? m_s[w * kQB + mq] : kSeedM;
      m_all = fmaxf(m_all, m_w[w]);
    }
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) {
      wgt[w] = has[w] ? expf(m_w[w] - m_all) : 0.f;
      const float l = has[w] ? l_s[w * kQB + mq] : 0.f;
      l_all = fmaf(l, wgt[w], l_all);
    }
    const float inv = 1.0f / l_all;
    f32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < kAttnWaves; ++w) {
        const float x = slot_s[w * kSlotFloats + ((2 * e + m_half) * 4 + m_r) * kOutPitch +
                               16 * m_lg + mq];
        sum = fmaf(has[w] ? x : 0.f, wgt[w], sum);
      }
      o[e] = sum * inv;
    }
    *reinterpret_cast<f32x4 *>(a.out + (int64_t)(q0[p] + mq) * a.o_stride +
                               (int64_t)h * a.o_hstride + 4 * c) = o;
  }
}

// One workgroup per token: rotate q in place, rotate k into the cache, copy v.
__global__ void __launch_bounds__(256)
rope_kv_write_kernel(float *qkv, int64_t row_stride, const float *inv_freq,
                     float *kcache, float *vcache, int heads, int kv_heads,
                     int max_len, int start_pos) {
  __shared__ float cs[kD / 2], sn[kD / 2];
  const int t = blockIdx.x, pos = start_pos + t;
  if (threadIdx.x < kD / 2) {
    float s, c;
    sincosf(inv_freq[threadIdx.x] * (float)pos, &s, &c);
    cs[threadIdx.x] = c;
    sn[threadIdx.x] = s;
  }
  __syncthreads();
  float *row = qkv + (int64_t)t * row_stride;
  const int half = kD / 2;
  for (int i = threadIdx.x; i < (heads + kv_heads) * half; i += 256) {
    const int hh = i / half, j = i % half;
    float *v = row + (int64_t)hh * kD; // q heads first, then k heads
    const float lo = v[j], hi = v[j + half];
    const float nlo = lo * cs[j] + (-hi) * sn[j];
    const float nhi = hi * cs[j] + lo * sn[j];
    if (hh < heads) {
      v[j] = nlo;
      v[j + half] = nhi;
    } else {
      float *dst = kcache + ((int64_t)(hh - heads) * max_len + pos) * kD;
      dst[j] = nlo;
      dst[j + half] = nhi;
    }
  }
  const float *vsrc = row + (int64_t)(heads + kv_heads) * kD;
  for (int i = threadIdx.x; i < kv_heads * kD; i += 256)
    vcache[((int64_t)(i / kD) * max_len + pos) * kD + i % kD] = vsrc[i];
}

} // namespace

BH_VARIANT_FAMILY(AttnPrefillFamily, "attn_prefill_kernel");

int launch_attn_prefill(const AttnPrefillArgs &in, hipStream_t stream) {
  BH_REQUIRE(in.q && in.k && in.v && in.out, "attn_prefill: null pointer");
  BH_REQUIRE(in.head_dim == kD, "attn_prefill: head_dim %d (only %d is built)",
             in.head_dim, kD);
  BH_REQUIRE(in.kv_heads > 0 && in.heads % in.kv_heads == 0,
             "attn_prefill: heads=%d kv_heads=%d", in.heads, in.kv_heads);
  BH_REQUIRE(in.q_len > 0 && in.k_len > 0 && in.kv_stride >= in.k_len,
             "attn_prefill: q_len=%d k_len=%d kv_stride=%lld", in.q_len, in.k_len,
             (long long)in.kv_stride);
  BH_REQUIRE(in.q_stride >= kD && in.o_stride >= kD && in.q_hstride >= kD &&
                 in.o_hstride >= kD && in.q_stride % 4 == 0 && in.o_stride % 4 == 0 &&
                 in.q_hstride % 4 == 0 && in.o_hstride % 4 == 0,
             "attn_prefill: bad strides");
  BH_REQUIRE(((reinterpret_cast<uintptr_t>(in.q) | reinterpret_cast<uintptr_t>(in.k) |
               reinterpret_cast<uintptr_t>(in.v) | reinterpret_cast<uintptr_t>(in.out)) & 15) == 0,
             "attn_prefill: q, k, v and out must be 16-byte aligned");
  PrefillArgs a;
  a.q = in.q;
  a.k = in.k;
  a.v = in.v;
  a.mask = in.mask;
  a.out = in.out;
  a.q_stride = in.q_stride;
  a.q_hstride = in.q_hstride;
  a.o_stride = in.o_stride;
  a.o_hstride = in.o_hstride;
  a.kv_stride = in.kv_stride;
  a.heads = in.heads;
  a.group = in.heads / in.kv_heads;
  a.q_len = in.q_len;
  a.k_len = in.k_len;
  a.q_offset = in.k_len - in.q_len; // the last query sees every key
  a.scale = in.scale;
  a.nqb = (int)ceil_div(in.q_len, kQB);
  const int pairs = (a.nqb + 1) / 2;
  BH_REQUIRE(pairs <= 65535, "attn_prefill: q_len %d too long", in.q_len);
  constexpr int kComputeUnits = 256; // MI355X
  a.paired = (int64_t)in.heads * pairs <= kComputeUnits;
  // group | paired << 12 | (65536 / group + 1) << 13: (h * multiplier) >> 16 == h / group
  // while heads * group < 65536
  BH_REQUIRE(a.group >= 1 && a.group < 4096 && (int64_t)in.heads * a.group < 65536,
             "attn_prefill: heads=%d group=%d", in.heads, a.group);
  const int gp = a.group | a.paired << 12 | (65536 / a.group + 1) << 13;
  if (a.paired) {
    static DynLdsOnce dyn_lds;
    BH_CHECK_HIP(ensure_dyn_lds(dyn_lds, reinterpret_cast<const void *>(attn_prefill_kernel<8>),
                                (int)(lds_floats(8) * sizeof(float))));
    BH_NOTE_VARIANT(AttnPrefillFamily, 8);
    hipLaunchKernelGGL(attn_prefill_kernel<8>, dim3(in.heads, (unsigned)pairs), dim3(8 * kWave),
                       lds_floats(8) * sizeof(float), stream, a.k, a.v, a.mask, a.kv_stride, gp, a.nqb,
                       a.q_len, a.k_len, a.q_offset, a);
  } else {
    BH_REQUIRE(a.nqb <= 65535, "attn_prefill: q_len %d too long", in.q_len);
    static DynLdsOnce dyn_lds;
    BH_CHECK_HIP(ensure_dyn_lds(dyn_lds, reinterpret_cast<const void *>(attn_prefill_kernel<4>),
                                (int)(lds_floats(4) * sizeof(float))));
    BH_NOTE_VARIANT(AttnPrefillFamily, 4);
    hipLaunchKernelGGL(attn_prefill_kernel<4>, dim3(in.heads, (unsigned)a.nqb), dim3(4 * kWave),
                       lds_floats(4) * sizeof(float), stream, a.k, a.v, a.mask, a.kv_stride, gp, a.nqb,
                       a.q_len, a.k_len, a.q_offset, a);
  }
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_rope_kv_write(float *qkv, int64_t row_stride, const float *inv_freq,
                         float *kcache, float *vcache, int heads, int kv_heads,
                         int head_dim, int max_len, int start_pos, int n_tokens,
                         hipStream_t stream) {
  BH_REQUIRE(qkv && inv_freq && kcache && vcache, "rope_kv_write: null pointer");
  BH_REQUIRE(head_dim == kD, "rope_kv_write: head_dim %d", head_dim);
  BH_REQUIRE(n_tokens > 0 && start_pos >= 0 && start_pos + n_tokens <= max_len,
             "rope_kv_write: tokens %d..%d outside the cache (max_len %d)",
             start_pos, start_pos + n_tokens - 1, max_len);
  hipLaunchKernelGGL(rope_kv_write_kernel, dim3(n_tokens), dim3(256), 0, stream,
                     qkv, row_stride, inv_freq, kcache, vcache, heads, kv_heads,
                     max_len, start_pos);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace bh

extern "C" {

int buddy_hip_prefill_attention(const float *q, const float *k, const float *v,
                                const float *mask, float *out, int heads,
                                int kv_heads, int head_dim, int q_len, int k_len,
                                float scale, buddy_hip_stream stream) try {
  // the reference operator's layout: [heads, len, head_dim] for q/out,
  // [kv_heads, len, head_dim] for k/v
  bh::AttnPrefillArgs a;
  a.q = q;
  a.k = k;
  a.v = v;
  a.mask = mask;
  a.out = out;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.head_dim = head_dim;
  a.q_len = q_len;
  a.k_len = k_len;
  a.scale = scale;
  a.kv_stride = k_len;
  a.q_stride = head_dim;
  a.q_hstride = (int64_t)q_len * head_dim;
  a.o_stride = head_dim;
  a.o_hstride = (int64_t)q_len * head_dim;
  return bh::launch_attn_prefill(a, bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_prefill_attention")
}
