// attn.h -- launch descriptions of the attention kernels.
#pragma once

#include "common.h"

namespace bh {

constexpr int kAttnChunk = 64; // cache positions per flash-decoding partial (the default)
// How a decode step at position `pos` cuts its attention.  Up to position 5120
// the o_proj launch folds the partials, up to 36 per head in one trip to memory
// (18 at its best): chunks of 64 positions up to position 1152, 128 up to 2304,
// 256 beyond (8 or 16 wavefronts of 16 positions per workgroup).  From 5120 on
// (where those launches would outgrow one workgroup per compute unit) the
// partials are folded by a launch of their own and one workgroup takes all the
// query heads of a KV head, or half of them (a K/V row then leaves L2 once or
// twice, not once per head).  Attention and fold cover only the chunks up to the
// position (rounded up to a multiple of four; 18 with chunks of 64), whatever the
// cache's capacity.
struct AttnStepPlan {
  int chunk;     // cache positions per partial: 64, 128 or 256
  int used;      // partials per head the step produces and folds
  bool own_fold; // a launch of its own folds them; workgroups take whole head groups
  int head_split; // ... or (2) half a head group each
};
inline AttnStepPlan attn_step_plan(int pos, int max_len, int kv_heads) {
  AttnStepPlan p;
  p.head_split = 1;
  p.own_fold = pos >= 20 * 256;
  if (!p.own_fold) {
    p.chunk = pos < 18 * 64 ? 64 : pos < 18 * 128 ? 128 : 256;
  } else {
    // Measured on a 12-head, 2-KV-head model from 5 k to 32 k positions (ms per step
    // for chunk x split): workgroups of 16 wavefronts (chunks of 256) must not
    // outnumber the 256 compute units, and want at least ~150 of them busy.
    const int n256 = (pos / 256 + 1) * kv_heads; // workgroups of whole head groups on chunks of 256
    if (2 * n256 <= 256) {
      p.chunk = n256 >= 100 ? 256 : 128; // 16 k: 1.005 (256 x 2) vs 1.027; 12 k: 0.986 (128 x 2) vs 0.995
      p.head_split = 2;
    } else {
      p.chunk = 256; // 20 k: 1.138 (256 x 1) vs 1.159 (128 x 1); 17.5 k: 1.147 with 128 x 1
    }
  }
  const int all = (max_len + p.chunk - 1) / p.chunk, need = pos / p.chunk + 1;
  // 18 for chunks of 64 (one captured step serves a cache of 1152 positions, and
  // the fold's first trip takes 18 anyway); with larger chunks the next multiple
  // of four: every chunk past the position costs workgroups that find nothing to do
  int want = (need + 3) / 4 * 4;
  if (need <= 18)
    want = p.chunk == 64 || want > 18 ? 18 : want;
  p.used = want < all ? want : all;
  return p;
}
// partials per head the fold of its own takes: 2^20 positions at 256 per chunk
constexpr int kAttnWideChunks = 4096;
constexpr int kAttnHeadDim = 128; // the head size the decode kernel is written for

struct AttnDecodeArgs {
  const float *qkv = nullptr;      // [heads*D | kv_heads*D | kv_heads*D], pre-RoPE
  const float *inv_freq = nullptr; // [D/2]
  // optional: [cos | sin] of the current position, D/2 values each, computed
  // once per step; without it every workgroup evaluates them from inv_freq
  const float *rope_table = nullptr;
  const int *pos_ptr = nullptr;    // device scalar: index of the current token
  float *kcache = nullptr;         // [kv_heads, max_len, D]
  float *vcache = nullptr;
  float *out = nullptr;            // [heads*D]
  float *lse = nullptr;            // optional [heads]: log-sum-exp of the scores
  int heads = 0, kv_heads = 0, head_dim = 0, max_len = 0;
  float scale = 0.f;
  void *workspace = nullptr; // flash-decoding partials
  size_t workspace_bytes = 0;
  bool combine = true; // false: leave the partials for the consumer to fold
  // with combine: the form for a step far into a long cache -- one workgroup
  // per (chunk, KV head) for all its query heads, then a fold with all partials
  // in flight instead of chunk by chunk (covers chunks_used partials, no lse)
  bool wide_combine = false;
  int head_split = 1; // with wide_combine: 2 = two workgroups per (chunk, KV head), half its heads each
  int chunk = kAttnChunk; // cache positions per partial: 64, 128 or 256
  // partials to produce (the first ones; the caller knows the position lies in
  // them); 0: one for every chunk of the cache
  int chunks_used = 0;
};

// Where the partials live inside the workspace.
struct AttnPartials {
  float *acc; // [heads, nchunks, head_dim]
  float *ml;  // [heads, nchunks, 2] = (max, sum)
  int nchunks;
};
AttnPartials attn_partials(void *workspace, int heads, int head_dim, int max_len,
                           int chunk = kAttnChunk);

struct AttnPrefillArgs {
  const float *q = nullptr;   // token t, head h at q + t*q_stride + h*q_hstride
  const float *k = nullptr;   // [kv_heads, kv_stride rows, head_dim]
  const float *v = nullptr;
  const float *mask = nullptr; // additive [q_len, k_len]; null = causal
  float *out = nullptr;        // token t, head h at out + t*o_stride + h*o_hstride
  int64_t q_stride = 0, q_hstride = 0, o_stride = 0, o_hstride = 0, kv_stride = 0;
  int heads = 0, kv_heads = 0, head_dim = 0, q_len = 0, k_len = 0;
  float scale = 0.f;
};
int launch_attn_prefill(const AttnPrefillArgs &a, hipStream_t stream);
// Rotates q in place for n_tokens rows of [q | k | v], writes rotated k and v
// into cache rows start_pos .. start_pos + n_tokens - 1.
int launch_rope_kv_write(float *qkv, int64_t row_stride, const float *inv_freq,
                         float *kcache, float *vcache, int heads, int kv_heads,
                         int head_dim, int max_len, int start_pos, int n_tokens,
                         hipStream_t stream);

size_t attn_decode_workspace_bytes(int heads, int max_len);
int launch_attn_decode(const AttnDecodeArgs &a, hipStream_t stream);

} // namespace bh
