// attn.h -- launch descriptions of the attention kernels.
#pragma once

#include "common.h"

namespace bh {

constexpr int kAttnChunk = 64; // cache positions per flash-decoding partial
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
};

// Where the partials live inside the workspace.
struct AttnPartials {
  float *acc; // [heads, nchunks, head_dim]
  float *ml;  // [heads, nchunks, 2] = (max, sum)
  int nchunks;
};
AttnPartials attn_partials(void *workspace, int heads, int head_dim, int max_len);

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
