// attn_decode.hip -- GQA decode attention over a device-resident f32 KV cache,
// with RoPE and the KV-cache write fused in.
//
// Replaces, for one decode step of one layer:
//   * RoPE on q and k   (examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir
//                        :51-59 angles, :88-107 rotate-half)
//   * cache[0, h, pos, :] = k' / v                       (same file :108-142)
//   * gqa_attention_fused_op  (frontend/Python/ops/tosa.py:14130-14600):
//     softmax(scale * q.K^T + mask) V with mask = 0 for k <= pos, -inf beyond,
//     computed as flash-decoding partials over k ranges plus a combine.
//
// Differences from the reference kernel that follow from the hardware:
//   * the cache is scanned up to pos only (masked positions contribute exactly
//     zero in the reference, so skipping them changes nothing);
//   * one workgroup serves one query head (the step is latency bound: many
//     small workgroups beat few large ones), and the workgroups of the other
//     query heads of the same KV head run on the same XCD, so K and V rows
//     leave HBM once per group, not once per query head;
//   * the k range is cut into chunks of 64 positions (more, smaller partials
//     than the reference's 4): a decode step has only ~2 MB of KV per layer and
//     is latency bound, so the chunks are what spreads it over the CUs.
// Partials meet in a small workspace.  The decode step folds them while the
// o_proj kernel stages its input; stand-alone callers get a second kernel that
// folds them in chunk order with the reference's own combine rule.
#include "attn.h"

#include <type_traits>

#include <atomic>

namespace bh {
namespace {


constexpr int kPW = 16;           // cache positions per wavefront
constexpr int kMaxGroup = 8;     // query heads per KV head
constexpr int kD = kAttnHeadDim; // head_dim this kernel is written for
constexpr float kSeedM = -1.0e30f; // tosa.py:13971

struct AttnArgs {
  const float *qkv;      // [heads*D | kv_heads*D | kv_heads*D]
  const float *inv_freq; // [D/2]
  const float *rope_table; // [cos | sin] of the position, or null
  const int *pos_ptr;    // device scalar: index of the current token
  float *kcache, *vcache; // [kv_heads, max_len, D]
  float *part_acc;       // [heads, nchunks, D]
  float *part_ml;        // [heads, nchunks, 2]
  float *out;            // [heads*D]
  float *lse;            // [heads] or null: m + log l of the whole softmax
  int heads, kv_heads, group, max_len, nchunks, chunk;
  int used; // chunks this launch covers (the first ones of nchunks)
  int head_split; // grouped launches: workgroups per (chunk, KV head), each a share of its heads
  float scale;
  int pairs_padded; // (chunk, kv head) pairs rounded up to the XCD count
};

// One workgroup: 16 kWaves cache positions (64 by default) x one query head.  The workgroups that
// share a chunk (the query heads of one KV head: same K/V rows) get linear ids
// that are equal modulo 8, so they run on the same XCD and the rows come out of
// that XCD's L2 after the first of them has fetched them.
//
// The step is latency bound, so the kernel is built to have almost nothing
// behind the arrival of its K/V rows: the small operands (q, the token's own
// k and v, the RoPE table) are requested first, the K/V rows right behind
// them, and every lane rotates its own four dims of q in registers.  Each of the
// wavefronts then handles 16 positions entirely on its own (scores, its own
// max / exp / sum, its share of P.V) in registers and cross-lane operations, and
// they meet once in LDS.
//
// What a wavefront needs before its first load -- five pointers and four
// integers, 14 argument words -- are separate leading parameters: this file is
// built with -amdgpu-kernarg-preload-count=14, so they arrive in SGPRs and the
// loads do not wait for a scalar load of the argument block.
__host__ __device__ constexpr int pack_heads(int heads, int kv_heads, int group) {
  return heads | kv_heads << 12 | group << 24; // heads, kv_heads < 4096, group <= 8
}
template <int kWaves>
__global__ void __launch_bounds__(kWaves * 64)
    attn_decode_partial(const float *p_qkv, float *p_kcache, float *p_vcache,
                        const float *p_rope_table, const int *p_pos, int p_used, int p_max_len,
                        int p_heads, int p_unused, AttnArgs rest) {
  AttnArgs a = rest;
  a.qkv = p_qkv;
  a.kcache = p_kcache;
  a.vcache = p_vcache;
  a.rope_table = p_rope_table;
  a.pos_ptr = p_pos;
  a.used = p_used;
  a.max_len = p_max_len;
  a.heads = p_heads & 0xfff;
  a.kv_heads = (p_heads >> 12) & 0xfff;
  a.group = p_heads >> 24;
  constexpr int kChunk = kWaves * kPW; // cache positions per workgroup: 64, 128 or 256
  constexpr int kR = kPW / 2;          // rows per lane: 8
  __shared__ __attribute__((aligned(16))) float accw_s[kWaves][kD];
  __shared__ float mw_s[kWaves], lw_s[kWaves];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  // grid (pairs_padded, group): the workgroups of a (chunk, KV head) pair have
  // linear ids equal modulo 8.  No division ahead of the first load: a pair's KV
  // head is found by counting (there are few)
  const int hb = blockIdx.y;
  int chunk = blockIdx.x, kvh = 0;
  if (chunk >= a.used * a.kv_heads)
    return; // padding id
  while (chunk >= a.used) {
    chunk -= a.used;
    ++kvh;
  }
  const int p0 = chunk * kChunk;
  const int h = kvh * a.group + hb; // this workgroup's query head

  // ---- small operands first ----------------------------------------------
  // Every lane asks for what its own four dims (c4) need: q, the new k and v,
  // their rotation partners 64 dims away and the angles of (dim mod 64).  The
  // rotation then happens in registers: no wavefront waits for another before
  // the scores.
  const int j = tid & (kD - 1);
  const int c4 = lane & 31, par = lane >> 5;
  const int d0 = c4 * 4, dp = d0 ^ (kD / 2), ja = d0 & (kD / 2 - 1);
  const float *qh = a.qkv + (size_t)h * kD;
  const float *kh = a.qkv + (size_t)a.heads * kD + (size_t)kvh * kD;
  const float4 q_raw = *reinterpret_cast<const float4 *>(qh + d0);
  float4 q_pair = *reinterpret_cast<const float4 *>(qh + dp);
  const float4 k_raw = *reinterpret_cast<const float4 *>(kh + d0);
  float4 k_pair = *reinterpret_cast<const float4 *>(kh + dp);
  const float4 v_new = *reinterpret_cast<const float4 *>(kh + (size_t)a.kv_heads * kD + d0);
  float4 cs4, sn4; // without the table: cs4 holds the inverse frequencies for now
  if (a.rope_table) {
    cs4 = *reinterpret_cast<const float4 *>(a.rope_table + ja);
    sn4 = *reinterpret_cast<const float4 *>(a.rope_table + kD / 2 + ja);
  } else {
    cs4 = *reinterpret_cast<const float4 *>(a.inv_freq + ja);
    sn4 = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  // ---- then this wavefront's 16 K rows and 16 V rows -----------------------
  // One lane mapping for both: lane = (float4 column c4 of the 128 dims, row
  // parity par), rows par, par + 2, ..., so that every load instruction reads
  // two whole 512-byte rows (eight cache lines, nothing else).  The rows exist
  // whatever the position is (rows beyond it hold zeros or stale data and are
  // masked by select, never multiplied in), so nothing here waits for the
  // position to arrive.
  const int pw0 = p0 + wave * kPW; // first position of this wavefront
  float4 kreg[kR], vreg[kR];
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const int row = min(pw0 + par + 2 * i, a.max_len - 1);
    kreg[i] = *reinterpret_cast<const float4 *>(
        a.kcache + ((size_t)kvh * a.max_len + row) * kD + c4 * 4);
  }
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const int row = min(pw0 + par + 2 * i, a.max_len - 1);
    vreg[i] = *reinterpret_cast<const float4 *>(
        a.vcache + ((size_t)kvh * a.max_len + row) * kD + c4 * 4);
  }
  // a position outside the cache (a caller's mistake the host cannot see: the
  // position lives on the device) is clamped for the scan and writes nothing
  const int pos_raw = *a.pos_ptr;
  const bool pos_ok = pos_raw >= 0 && pos_raw < a.max_len;
  const int pos = min(max(pos_raw, 0), a.max_len - 1);

  if (p0 > pos) { // nothing visible in this chunk: an empty partial
    if (tid < kD)
      a.part_acc[((size_t)h * a.nchunks + chunk) * kD + j] = 0.f;
    if (tid == 0) {
      a.part_ml[((size_t)h * a.nchunks + chunk) * 2 + 0] = kSeedM;
      a.part_ml[((size_t)h * a.nchunks + chunk) * 2 + 1] = 0.f;
    }
    return;
  }
  const bool has_new = pos < p0 + kChunk; // the token's own row lies in this chunk

  // ---- RoPE: q' = q*cos + cat(-q[64:], q[:64])*sin, same for the new k ------
  if (!a.rope_table) {
    const float4 f = cs4;
    sincosf(f.x * (float)pos, &sn4.x, &cs4.x);
    sincosf(f.y * (float)pos, &sn4.y, &cs4.y);
    sincosf(f.z * (float)pos, &sn4.z, &cs4.z);
    sincosf(f.w * (float)pos, &sn4.w, &cs4.w);
  }
  if (d0 < kD / 2) {
    q_pair = make_float4(-q_pair.x, -q_pair.y, -q_pair.z, -q_pair.w);
    k_pair = make_float4(-k_pair.x, -k_pair.y, -k_pair.z, -k_pair.w);
  }
  const float4 q4 = make_float4(q_raw.x * cs4.x + q_pair.x * sn4.x, q_raw.y * cs4.y + q_pair.y * sn4.y,
                                q_raw.z * cs4.z + q_pair.z * sn4.z, q_raw.w * cs4.w + q_pair.w * sn4.w);
  const float4 k_new = make_float4(k_raw.x * cs4.x + k_pair.x * sn4.x, k_raw.y * cs4.y + k_pair.y * sn4.y,
                                   k_raw.z * cs4.z + k_pair.z * sn4.z, k_raw.w * cs4.w + k_pair.w * sn4.w);
  if (has_new && hb == 0 && pos_ok && tid < 32) { // one writer per cache row
    *reinterpret_cast<float4 *>(a.kcache + ((size_t)kvh * a.max_len + pos) * kD + d0) = k_new;
    *reinterpret_cast<float4 *>(a.vcache + ((size_t)kvh * a.max_len + pos) * kD + d0) = v_new;
  }

  // ---- scores of this wavefront's 16 positions ------------------------------
  // every lane of a half ends up with the 8 scores of its half's rows
  float sc[kR];
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const int p = pw0 + par + 2 * i;
    float4 k4 = kreg[i];
    if (p == pos) // the token's own key is not in the cache yet
      k4 = k_new;
    float d = fmaf(q4.x, k4.x, fmaf(q4.y, k4.y, fmaf(q4.z, k4.z, q4.w * k4.w)));
    d = row16_sum(d);               // the 16 lanes of a row
    d += __shfl_xor(d, 16, 64);     // the two rows of a half: all 128 dims
    sc[i] = p <= pos ? d * a.scale : -INFINITY;
  }
  // ---- this wavefront's own max, exp and sum --------------------------------
  float m_w = kSeedM; // stays there when no position is visible
#pragma unroll
  for (int i = 0; i < kR; ++i)
    m_w = fmaxf(m_w, sc[i]);
  m_w = fmaxf(m_w, __shfl_xor(m_w, 32, 64));
  float l_w = 0.f;
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    sc[i] = fast_exp(sc[i] - m_w); // -inf -> 0 beyond the position
    l_w += sc[i];
  }
  l_w += __shfl_xor(l_w, 32, 64);

  // ---- acc[d] = sum_p e[p] * V[p][d]: this lane's 8 rows x 4 dims -----------
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const int p = pw0 + par + 2 * i;
    float4 v = vreg[i];
    if (p == pos) // the token's own value row
      v = v_new;
    if (p <= pos) { // rows beyond the position may hold anything
      acc.x = fmaf(v.x, sc[i], acc.x);
      acc.y = fmaf(v.y, sc[i], acc.y);
      acc.z = fmaf(v.z, sc[i], acc.z);
      acc.w = fmaf(v.w, sc[i], acc.w);
    }
  }
  acc.x += __shfl_xor(acc.x, 32, 64);
  acc.y += __shfl_xor(acc.y, 32, 64);
  acc.z += __shfl_xor(acc.z, 32, 64);
  acc.w += __shfl_xor(acc.w, 32, 64);
  if (lane < 32)
    *reinterpret_cast<float4 *>(&accw_s[wave][c4 * 4]) = acc;
  if (lane == 0) {
    mw_s[wave] = m_w;
    lw_s[wave] = l_w;
  }
  __syncthreads();

  // ---- the wavefronts meet: one partial per (head, chunk) -------------------
  if (tid < kD) {
    float m = mw_s[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w)
      m = fmaxf(m, mw_s[w]);
    float o = 0.f, l = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float f = fast_exp(mw_s[w] - m);
      o = fmaf(accw_s[w][tid], f, o);
      l = fmaf(lw_s[w], f, l);
    }
    a.part_acc[((size_t)h * a.nchunks + chunk) * kD + tid] = o;
    if (tid == 0) {
      a.part_ml[((size_t)h * a.nchunks + chunk) * 2 + 0] = m;
      a.part_ml[((size_t)h * a.nchunks + chunk) * 2 + 1] = l;
    }
  }
}

// The same for a step far into a long cache, where the rows of a chunk coming
// out of L2 once per query head (six times for this model) is what the launch
// waits for: one workgroup takes all the query heads of a KV head, so that a K/V
// row is loaded once and multiplied with every head's query.
template <int kWaves>
__global__ void __launch_bounds__(kWaves * 64)
    attn_decode_partial_group(const float *p_qkv, float *p_kcache, float *p_vcache,
                              const float *p_rope_table, const int *p_pos, int p_used,
                              int p_max_len, int p_heads, int p_head_split, AttnArgs rest) {
  AttnArgs a = rest; // the leading parameters arrive in SGPRs (see attn_decode_partial)
  a.qkv = p_qkv;
  a.kcache = p_kcache;
  a.vcache = p_vcache;
  a.rope_table = p_rope_table;
  a.pos_ptr = p_pos;
  a.used = p_used;
  a.max_len = p_max_len;
  a.heads = p_heads & 0xfff;
  a.kv_heads = (p_heads >> 12) & 0xfff;
  a.group = p_heads >> 24;
  a.head_split = p_head_split;
  constexpr int kChunk = kWaves * kPW;
  constexpr int kR = kPW / 2;
  __shared__ __attribute__((aligned(16))) float q_s[kMaxGroup][kD], knew_s[kD], vnew_s[kD];
  // what the wavefronts leave for the merge, every head of the group at once
  extern __shared__ __attribute__((aligned(16))) float accw_s[]; // [group][kWaves][kD]
  __shared__ float mw_s[kMaxGroup][kWaves], lw_s[kMaxGroup][kWaves];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  // grid (pairs_padded, head_split): the workgroups that share a (chunk, KV head)
  // pair have linear ids equal modulo 8 -- one XCD, one L2 for the pair's rows
  const int hs = blockIdx.y;
  int chunk = blockIdx.x, kvh = 0;
  if (chunk >= a.used * a.kv_heads)
    return; // padding id
  while (chunk >= a.used) { // no division ahead of the first load
    chunk -= a.used;
    ++kvh;
  }
  // this workgroup's share of the group's query heads (head_split is 1 or 2)
  const int per = (a.group + a.head_split - 1) >> (a.head_split - 1);
  const int h_lo = hs * per, h_hi = min(a.group, h_lo + per);
  const int p0 = chunk * kChunk;
  const int c4 = lane & 31, par = lane >> 5;
  const int pw0 = p0 + wave * kPW;
  // ---- small operands first: the queries of the group and the token's key, an
  // element and its rotation partner per thread and pass, with their angles ----
  constexpr int kPasses = ((kMaxGroup + 1) * kD + kWaves * 64 - 1) / (kWaves * 64);
  float raw[kPasses], pair[kPasses], cs[kPasses], sn[kPasses], vraw[kPasses];
#pragma unroll
  for (int u = 0; u < kPasses; ++u) {
    const int i = min(tid + u * kWaves * 64, (a.group + 1) * kD - 1); // past the end: repeats
    const int hh = i / kD, j = i % kD, jj = j & (kD / 2 - 1);
    // the queries of the group, then (hh == group) the token's own key
    const float *src = hh < a.group ? a.qkv + (size_t)(kvh * a.group + hh) * kD
                                    : a.qkv + (size_t)a.heads * kD + (size_t)kvh * kD;
    raw[u] = src[j];
    pair[u] = j < kD / 2 ? -src[j + kD / 2] : src[j - kD / 2];
    vraw[u] = hh < a.group ? 0.f : src[(size_t)a.kv_heads * kD + j];
    if (a.rope_table) {
      cs[u] = a.rope_table[jj];
      sn[u] = a.rope_table[kD / 2 + jj];
    } else {
      cs[u] = a.inv_freq[jj]; // the angle needs the position
      sn[u] = 0.f;
    }
  }
  float4 kreg[kR], vreg[kR];
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const int row = min(pw0 + par + 2 * i, a.max_len - 1);
    kreg[i] = *reinterpret_cast<const float4 *>(
        a.kcache + ((size_t)kvh * a.max_len + row) * kD + c4 * 4);
  }
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const int row = min(pw0 + par + 2 * i, a.max_len - 1);
    vreg[i] = *reinterpret_cast<const float4 *>(
        a.vcache + ((size_t)kvh * a.max_len + row) * kD + c4 * 4);
  }
  const int pos_raw = *a.pos_ptr;
  const bool pos_ok = pos_raw >= 0 && pos_raw < a.max_len;
  const int pos = min(max(pos_raw, 0), a.max_len - 1);
  if (p0 > pos) { // nothing visible in this chunk: empty partials
    for (int i = tid; i < (h_hi - h_lo) * kD; i += kWaves * 64) {
      const int h = kvh * a.group + h_lo + i / kD;
      a.part_acc[((size_t)h * a.nchunks + chunk) * kD + i % kD] = 0.f;
    }
    if (tid < h_hi - h_lo) {
      const int h = kvh * a.group + h_lo + tid;
      a.part_ml[((size_t)h * a.nchunks + chunk) * 2 + 0] = kSeedM;
      a.part_ml[((size_t)h * a.nchunks + chunk) * 2 + 1] = 0.f;
    }
    return;
  }
  const bool has_new = pos < p0 + kChunk;
  // ---- RoPE of every query of the group and of the token's key --------------
#pragma unroll
  for (int u = 0; u < kPasses; ++u) {
    const int i = tid + u * kWaves * 64;
    if (i < (a.group + 1) * kD) {
      const int hh = i / kD, j = i % kD;
      if (!a.rope_table)
        sincosf(cs[u] * (float)pos, &sn[u], &cs[u]);
      const float rot = raw[u] * cs[u] + pair[u] * sn[u];
      if (hh < a.group) {
        q_s[hh][j] = rot;
      } else if (has_new) {
        knew_s[j] = rot;
        vnew_s[j] = vraw[u];
        if (pos_ok && hs == 0) { // one writer per cache row
          a.kcache[((size_t)kvh * a.max_len + pos) * kD + j] = rot;
          a.vcache[((size_t)kvh * a.max_len + pos) * kD + j] = vraw[u];
        }
      }
    }
  }
  __syncthreads();
  // the token's own rows replace what the cache holds at its position
#pragma unroll
  for (int i = 0; i < kR; ++i)
    if (pw0 + par + 2 * i == pos) {
      kreg[i] = *reinterpret_cast<const float4 *>(knew_s + c4 * 4);
      vreg[i] = *reinterpret_cast<const float4 *>(vnew_s + c4 * 4);
    }
  // The launch is bound by its vector instructions at long contexts, and every
  // chunk but the one the position lies in is visible whole: those run without the
  // comparisons and selects of the mask.
  auto heads_pass = [&](auto whole_chunk) {
    constexpr bool kWhole = decltype(whole_chunk)::value;
    for (int hh = h_lo; hh < h_hi; ++hh) {
      const float4 q4 = *reinterpret_cast<const float4 *>(q_s[hh] + c4 * 4);
      float sc[kR];
#pragma unroll
      for (int i = 0; i < kR; ++i) {
        const int p = pw0 + par + 2 * i;
        const float4 k4 = kreg[i];
        float d = fmaf(q4.x, k4.x, fmaf(q4.y, k4.y, fmaf(q4.z, k4.z, q4.w * k4.w)));
        d = row16_sum(d);
        d += __shfl_xor(d, 16, 64);
        sc[i] = kWhole || p <= pos ? d * a.scale : -INFINITY;
      }
      float m_w = kSeedM;
#pragma unroll
      for (int i = 0; i < kR; ++i)
        m_w = fmaxf(m_w, sc[i]);
      m_w = fmaxf(m_w, __shfl_xor(m_w, 32, 64));
      float l_w = 0.f;
#pragma unroll
      for (int i = 0; i < kR; ++i) {
        sc[i] = fast_exp(sc[i] - m_w);
        l_w += sc[i];
      }
      l_w += __shfl_xor(l_w, 32, 64);
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int i = 0; i < kR; ++i) {
        const int p = pw0 + par + 2 * i;
        float4 v = vreg[i];
        if (!kWhole && p > pos) // rows beyond the position may hold anything
          v = make_float4(0.f, 0.f, 0.f, 0.f);
        acc.x = fmaf(v.x, sc[i], acc.x);
        acc.y = fmaf(v.y, sc[i], acc.y);
        acc.z = fmaf(v.z, sc[i], acc.z);
        acc.w = fmaf(v.w, sc[i], acc.w);
      }
      acc.x += __shfl_xor(acc.x, 32, 64);
      acc.y += __shfl_xor(acc.y, 32, 64);
      acc.z += __shfl_xor(acc.z, 32, 64);
      acc.w += __shfl_xor(acc.w, 32, 64);
      if (lane < 32)
        *reinterpret_cast<float4 *>(&accw_s[((size_t)hh * kWaves + wave) * kD + c4 * 4]) = acc;
      if (lane == 0) {
        mw_s[hh][wave] = m_w;
        lw_s[hh][wave] = l_w;
      }
    }
  };
  if (p0 + kChunk - 1 <= pos)
    heads_pass(std::true_type{});
  else
    heads_pass(std::false_type{});
  __syncthreads();
  // ---- the wavefronts meet, once for all heads: one partial per (head, chunk) --
  for (int i = tid; i < (h_hi - h_lo) * kD; i += kWaves * 64) {
    const int hh = h_lo + i / kD, d = i % kD, h = kvh * a.group + hh;
    float m = mw_s[hh][0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w)
      m = fmaxf(m, mw_s[hh][w]);
    float o = 0.f, l = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float f = fast_exp(mw_s[hh][w] - m);
      o = fmaf(accw_s[((size_t)hh * kWaves + w) * kD + d], f, o);
      l = fmaf(lw_s[hh][w], f, l);
    }
    a.part_acc[((size_t)h * a.nchunks + chunk) * kD + d] = o;
    if (d == 0) {
      a.part_ml[((size_t)h * a.nchunks + chunk) * 2 + 0] = m;
      a.part_ml[((size_t)h * a.nchunks + chunk) * 2 + 1] = l;
    }
  }
}

// Folds the partials of one head in chunk order with the reference's combine
// (tosa.py:14485-14568): m_new = max(m_run, m_s); a = exp(m_run - m_new);
// b = exp(m_s - m_new); l = l*a + l_s*b; acc = acc_s*b + acc*a; out = acc / l.
__global__ void __launch_bounds__(kD) attn_decode_combine(AttnArgs a) {
  const int h = blockIdx.x, d = threadIdx.x;
  const int pos = min(max(*a.pos_ptr, 0), a.max_len - 1);
  const int used = min(a.nchunks, pos / a.chunk + 1);
  float m_run = kSeedM, l_run = 0.f, acc = 0.f;
  for (int s = 0; s < used; ++s) {
    const float m_c = a.part_ml[((size_t)h * a.nchunks + s) * 2 + 0];
    const float l_c = a.part_ml[((size_t)h * a.nchunks + s) * 2 + 1];
    const float m_new = m_c > m_run ? m_c : m_run;
    const float al = expf(m_run - m_new);
    const float be = expf(m_c - m_new);
    l_run = l_run * al + l_c * be;
    const float rescaled = acc * al;
    acc = fmaf(a.part_acc[((size_t)h * a.nchunks + s) * kD + d], be, rescaled);
    m_run = m_new;
  }
  a.out[(size_t)h * kD + d] = acc / l_run;
  if (a.lse && d == 0) // tosa.py:14576-14580
    a.lse[h] = m_run + logf(l_run);
}

// The same fold for a step far into a long cache, where one partial after the
// other would take a trip to memory each: a workgroup of 32 x 32 threads per head,
// thread (q, g) gathers d = 4 q .. 4 q + 3 of the chunks s = g, g + 32, ... with
// every load in flight at once, every wavefront works out the common maximum and
// the weights exp(m_s - max m) for itself, and the 32 groups meet in LDS.  The
// sums are those of the chunk-by-chunk rule in another order.
constexpr int kWideChunks = kAttnWideChunks; // partials per head it takes

__global__ void __launch_bounds__(1024)
    attn_decode_combine_wide(const float *p_acc, const float *p_ml, float *p_out, int p_nchunks,
                             int p_used) { // (arguments preloaded into SGPRs)
  constexpr int kPer = kWideChunks / 32; // chunks per thread at most
  constexpr int kFast = 4;               // passes of 64 chunks whose (max, sum) pairs stay in registers
  __shared__ float w_s[kWideChunks];
  __shared__ __attribute__((aligned(16))) float4 red_s[32][32];
  const int h = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
  const int q = tid & 31, g = tid >> 5;
  const int used = p_used;
  const float2 *ml = reinterpret_cast<const float2 *>(p_ml) + (size_t)h * p_nchunks;
  const float *acc = p_acc + (size_t)h * p_nchunks * kD + q * 4;
  // the partial sums of this thread's first four chunks and the (max, sum) pairs
  // are requested together, before anything is known of the weights: one trip
  // (chunks past the last repeat it and are not added)
  float4 v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    v[i] = *reinterpret_cast<const float4 *>(acc + (size_t)min(g + 32 * i, used - 1) * kD);
  float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
  // the weights: every wavefront computes all of them (64 chunks per pass) and
  // wavefront 0 leaves them in LDS
  float m_all = kSeedM, l_all = 0.f;
  if (used <= 64 * kFast) {
    float2 mine[kFast];
#pragma unroll
    for (int p = 0; p < kFast; ++p)
      mine[p] = ml[min(64 * p + lane, used - 1)];
#pragma unroll
    for (int p = 0; p < kFast; ++p)
      m_all = fmaxf(m_all, wave_max(64 * p + lane < used ? mine[p].x : kSeedM));
#pragma unroll
    for (int p = 0; p < kFast; ++p) {
      const bool in = 64 * p + lane < used;
      const float w = in ? fast_exp(mine[p].x - m_all) : 0.f;
      l_all += wave_sum(mine[p].y * w);
      if (tid < 64 && in)
        w_s[64 * p + lane] = w;
    }
  } else {
    for (int s0 = 0; s0 < used; s0 += 64)
      m_all = fmaxf(m_all, wave_max(s0 + lane < used ? ml[s0 + lane].x : kSeedM));
    for (int s0 = 0; s0 < used; s0 += 64) {
      const bool in = s0 + lane < used;
      const float2 mine = ml[min(s0 + lane, used - 1)];
      const float w = in ? fast_exp(mine.x - m_all) : 0.f;
      l_all += wave_sum(mine.y * w);
      if (tid < 64 && in)
        w_s[s0 + lane] = w;
    }
  }
  __syncthreads();
  for (int i0 = 0; i0 < kPer; i0 += 4) {
    if (g + 32 * i0 >= used)
      break;
    if (i0 > 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        v[i] = *reinterpret_cast<const float4 *>(acc + (size_t)min(g + 32 * (i0 + i), used - 1) * kD);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = g + 32 * (i0 + i);
      if (c < used) {
        const float w = w_s[c];
        sum.x = fmaf(v[i].x, w, sum.x);
        sum.y = fmaf(v[i].y, w, sum.y);
        sum.z = fmaf(v[i].z, w, sum.z);
        sum.w = fmaf(v[i].w, w, sum.w);
      }
    }
  }
  red_s[g][q] = sum;
  __syncthreads();
  if (tid < 32) {
    float4 o = red_s[0][tid];
#pragma unroll 8
    for (int gg = 1; gg < 32; ++gg) {
      const float4 r = red_s[gg][tid];
      o.x += r.x; o.y += r.y; o.z += r.z; o.w += r.w;
    }
    const float inv = 1.0f / l_all;
    *reinterpret_cast<float4 *>(p_out + (size_t)h * kD + tid * 4) =
        make_float4(o.x * inv, o.y * inv, o.z * inv, o.w * inv);
  }
}

// ---- scratch of the entry point that allocates nothing --------------------
// Flash-decoding partials for up to kStaticPartials (head, chunk) pairs, e.g.
// 32 heads x 16384 cache positions: 8192 x (128 + 2) floats = 4.06 MiB of
// device memory that every GPU the library runs on holds until the process
// ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress: the address a kernel may use is looked up once per
// device and kept in g_scratch_ptr.
constexpr int kStaticPartials = 8192;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) float g_attn_scratch[(size_t)kStaticPartials * (kD + 2)];
std::atomic<float *> g_scratch_ptr[kMaxDevices] = {};

// Device address of the current device's copy of g_attn_scratch.  The first
// call on a device asks the runtime (hipGetSymbolAddress, which may load the
// code object); that must not happen inside a stream capture, so a capturing
// caller that has not made an eager call or buddy_hip_static_scratch_init() on
// this device first is refused.  Later calls are one atomic load.
int static_scratch(float **out, hipStream_t stream) {
  int dev = -1;
  BH_CHECK_HIP(hipGetDevice(&dev));
  BH_REQUIRE(dev >= 0 && dev < kMaxDevices, "attn_decode: device index %d", dev);
  float *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (stream) {
      hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
      BH_CHECK_HIP(hipStreamIsCapturing(stream, &st));
      BH_REQUIRE(st == hipStreamCaptureStatusNone,
                 "attn_decode_static: call buddy_hip_static_scratch_init() on this device "
                 "before capturing");
    }
    void *q = nullptr;
    BH_CHECK_HIP(hipGetSymbolAddress(&q, HIP_SYMBOL(g_attn_scratch)));
    BH_REQUIRE(q, "attn_decode: no device address for the static scratch");
    p = static_cast<float *>(q);
    // two threads may both ask: they get the same address
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return BUDDY_HIP_OK;
}

} // namespace

size_t attn_decode_workspace_bytes(int heads, int max_len) {
  const int nchunks = (int)ceil_div(max_len, kAttnChunk); // the smallest chunk: the most partials
  return sizeof(float) * (size_t)heads * nchunks * (kD + 2);
}

AttnPartials attn_partials(void *workspace, int heads, int head_dim, int max_len, int chunk) {
  AttnPartials p;
  p.nchunks = (int)ceil_div(max_len, chunk);
  p.acc = static_cast<float *>(workspace);
  p.ml = p.acc + (size_t)heads * p.nchunks * head_dim;
  return p;
}

int launch_attn_decode(const AttnDecodeArgs &in, hipStream_t stream) {
  BH_REQUIRE(in.qkv && in.inv_freq && in.pos_ptr && in.kcache && in.vcache &&
                 (in.out || !in.combine) && in.workspace,
             "attn_decode: null pointer");
  auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  BH_REQUIRE(aligned16(in.qkv) && aligned16(in.inv_freq) && aligned16(in.rope_table) &&
                 aligned16(in.kcache) && aligned16(in.vcache),
             "attn_decode: qkv, inv_freq, the RoPE table and the caches must be 16-byte aligned");
  BH_REQUIRE(in.head_dim == kD, "attn_decode: head_dim %d (only %d is built)",
             in.head_dim, kD);
  BH_REQUIRE(in.kv_heads > 0 && in.heads % in.kv_heads == 0 &&
                 in.heads / in.kv_heads <= kMaxGroup,
             "attn_decode: heads=%d kv_heads=%d unsupported", in.heads,
             in.kv_heads);
  BH_REQUIRE(in.max_len > 0, "attn_decode: max_len=%d", in.max_len);
  BH_REQUIRE(!in.lse || in.combine, "attn_decode: lse needs the combine pass");
  BH_REQUIRE(in.workspace_bytes >=
                 attn_decode_workspace_bytes(in.heads, in.max_len),
             "attn_decode: workspace of %zu bytes needed, %zu given",
             attn_decode_workspace_bytes(in.heads, in.max_len),
             in.workspace_bytes);
  AttnArgs a;
  a.qkv = in.qkv;
  a.inv_freq = in.inv_freq;
  a.rope_table = in.rope_table;
  a.pos_ptr = in.pos_ptr;
  a.kcache = in.kcache;
  a.vcache = in.vcache;
  a.heads = in.heads;
  a.kv_heads = in.kv_heads;
  a.group = in.heads / in.kv_heads;
  a.max_len = in.max_len;
  BH_REQUIRE(in.chunk == 64 || in.chunk == 128 || in.chunk == 256, "attn_decode: chunk %d",
             in.chunk);
  a.chunk = in.chunk;
  a.nchunks = (int)ceil_div(in.max_len, in.chunk);
  a.scale = in.scale;
  const AttnPartials parts = attn_partials(in.workspace, in.heads, kD, in.max_len, in.chunk);
  a.part_acc = parts.acc;
  a.part_ml = parts.ml;
  a.out = in.out;
  a.lse = in.lse;
  a.used = in.chunks_used > 0 ? std::min(in.chunks_used, a.nchunks) : a.nchunks;
  a.head_split = 1;
  BH_REQUIRE(!in.combine || in.wide_combine || a.used == a.nchunks,
             "attn_decode: the combine pass needs a partial for every chunk");
  BH_REQUIRE(!in.wide_combine || (in.combine && !in.lse && a.used <= kWideChunks),
             "attn_decode: the wide combine takes up to %d partials per head and returns no lse",
             kWideChunks);
  a.pairs_padded = (int)round_up((int64_t)a.used * in.kv_heads, 8);
  if (in.wide_combine) {
    // far into a long cache: one workgroup per (chunk, KV head) for all its heads
    BH_REQUIRE(in.head_split == 1 || in.head_split == 2, "attn_decode: head_split %d",
               in.head_split);
    a.head_split = std::min(in.head_split, a.group); // a group of one head has nothing to share out
    const dim3 grid(a.pairs_padded, a.head_split);
    BH_REQUIRE(in.heads < 4096, "attn_decode: %d heads", in.heads);
    const int hp = pack_heads(a.heads, a.kv_heads, a.group);
    const size_t lds = sizeof(float) * (size_t)a.group * (in.chunk / kPW) * kD; // <= 64 KiB
    if (in.chunk == 64) {
      hipLaunchKernelGGL(attn_decode_partial_group<4>, grid, dim3(4 * 64), lds, stream, a.qkv,
                         a.kcache, a.vcache, a.rope_table, a.pos_ptr, a.used, a.max_len, hp,
                         a.head_split, a);
    } else if (in.chunk == 128) {
      hipLaunchKernelGGL(attn_decode_partial_group<8>, grid, dim3(8 * 64), lds, stream, a.qkv,
                         a.kcache, a.vcache, a.rope_table, a.pos_ptr, a.used, a.max_len, hp,
                         a.head_split, a);
    } else {
      // with 8 heads per KV head the 64 KiB of dynamic LDS come on top of 6 KiB
      static DynLdsOnce dyn_lds;
      BH_CHECK_HIP(ensure_dyn_lds(dyn_lds,
                                  reinterpret_cast<const void *>(attn_decode_partial_group<16>),
                                  (int)(sizeof(float) * kMaxGroup * 16 * kD)));
      hipLaunchKernelGGL(attn_decode_partial_group<16>, grid, dim3(16 * 64), lds, stream, a.qkv,
                         a.kcache, a.vcache, a.rope_table, a.pos_ptr, a.used, a.max_len, hp,
                         a.head_split, a);
    }
    hipLaunchKernelGGL(attn_decode_combine_wide, dim3(in.heads), dim3(1024), 0, stream, a.part_acc,
                       a.part_ml, a.out, a.nchunks, a.used);
    BH_CHECK_HIP(hipGetLastError());
    return BUDDY_HIP_OK;
  }
  const dim3 grid(a.pairs_padded, a.group);
  BH_REQUIRE(in.heads < 4096, "attn_decode: %d heads", in.heads);
  const int hp = pack_heads(a.heads, a.kv_heads, a.group);
  if (in.chunk == 64)
    hipLaunchKernelGGL(attn_decode_partial<4>, grid, dim3(4 * 64), 0, stream, a.qkv, a.kcache,
                       a.vcache, a.rope_table, a.pos_ptr, a.used, a.max_len, hp, 0, a);
  else if (in.chunk == 128)
    hipLaunchKernelGGL(attn_decode_partial<8>, grid, dim3(8 * 64), 0, stream, a.qkv, a.kcache,
                       a.vcache, a.rope_table, a.pos_ptr, a.used, a.max_len, hp, 0, a);
  else
    hipLaunchKernelGGL(attn_decode_partial<16>, grid, dim3(16 * 64), 0, stream, a.qkv, a.kcache,
                       a.vcache, a.rope_table, a.pos_ptr, a.used, a.max_len, hp, 0, a);
  if (in.combine && in.wide_combine)
    hipLaunchKernelGGL(attn_decode_combine_wide, dim3(in.heads), dim3(1024), 0, stream, a.part_acc,
                       a.part_ml, a.out, a.nchunks, a.used);
  else if (in.combine)
    hipLaunchKernelGGL(attn_decode_combine, dim3(in.heads), dim3(kD), 0, stream, a);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace bh

extern "C" {

size_t buddy_hip_attn_decode_workspace_bytes(int heads, int max_len) {
  return bh::attn_decode_workspace_bytes(heads, max_len);
}

int buddy_hip_attn_step_plan(int pos, int max_len, int kv_heads, int *chunk, int *partials,
                             int *own_fold) try {
  BH_REQUIRE(chunk && partials && own_fold, "attn_step_plan: null argument");
  BH_REQUIRE(max_len > 0 && pos >= 0 && pos < max_len && kv_heads > 0,
             "attn_step_plan: pos=%d max_len=%d kv_heads=%d", pos, max_len, kv_heads);
  const bh::AttnStepPlan p = bh::attn_step_plan(pos, max_len, kv_heads);
  *chunk = p.chunk;
  *partials = p.used;
  *own_fold = p.own_fold ? 1 : 0;
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_attn_step_plan")

int buddy_hip_gqa_decode_attention(const float *qkv, const float *inv_freq,
                                   const int *pos, float *kcache, float *vcache,
                                   float *out, float *lse, int heads,
                                   int kv_heads, int head_dim, int max_len,
                                   float scale, void *workspace,
                                   size_t workspace_bytes,
                                   buddy_hip_stream stream) try {
  bh::AttnDecodeArgs a;
  a.qkv = qkv;
  a.inv_freq = inv_freq;
  a.pos_ptr = pos;
  a.kcache = kcache;
  a.vcache = vcache;
  a.out = out;
  a.lse = lse;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.head_dim = head_dim;
  a.max_len = max_len;
  a.scale = scale;
  a.workspace = workspace;
  a.workspace_bytes = workspace_bytes;
  return bh::launch_attn_decode(a, bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_gqa_decode_attention")

int buddy_hip_gqa_decode_attention_static(const float *qkv, const float *inv_freq,
                                          const int *pos, float *kcache,
                                          float *vcache, float *out, float *lse,
                                          int heads, int kv_heads, int head_dim,
                                          int max_len, float scale,
                                          buddy_hip_stream stream) try {
  BH_REQUIRE(heads > 0 && max_len > 0, "attn_decode_static: heads=%d max_len=%d", heads,
             max_len);
  const int64_t pairs = (int64_t)heads * bh::ceil_div(max_len, bh::kAttnChunk);
  BH_REQUIRE(pairs <= bh::kStaticPartials,
             "attn_decode_static: heads x ceil(max_len / %d) = %lld exceeds the built-in "
             "scratch of %d partials; use buddy_hip_gqa_decode_attention with a workspace",
             bh::kAttnChunk, (long long)pairs, bh::kStaticPartials);
  float *scratch = nullptr;
  int rc = bh::static_scratch(&scratch, bh::as_stream(stream));
  if (rc)
    return rc;
  bh::AttnDecodeArgs a;
  a.qkv = qkv;
  a.inv_freq = inv_freq;
  a.pos_ptr = pos;
  a.kcache = kcache;
  a.vcache = vcache;
  a.out = out;
  a.lse = lse;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.head_dim = head_dim;
  a.max_len = max_len;
  a.scale = scale;
  a.workspace = scratch;
  a.workspace_bytes = sizeof(float) * (size_t)bh::kStaticPartials * (bh::kAttnHeadDim + 2);
  return bh::launch_attn_decode(a, bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_gqa_decode_attention_static")

int buddy_hip_static_scratch_init(void) try {
  float *scratch = nullptr;
  return bh::static_scratch(&scratch, nullptr);
} BH_CATCH_INT("buddy_hip_static_scratch_init")
}
