/* TEST INFRASTRUCTURE: one decode step of a Qwen2-shaped decoder, composed
 * from the restated kernels in the op order of
 * examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:46-260,4986-5004.
 * Not part of the shipped library. */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

static void linear(const float *x, const int8_t *W, const float *s,
                   const float *bias, float *y, int64_t K, int64_t N) {
  /* every MatmulOp output buffer is a zero tensor in model context
   * (frontend/Python/ops/linalg.py:1320-1334); bias is a separate tosa.add
   * computed as bias + matmul (subgraph0_decode_simplify.mlir:74-76). */
  memset(y, 0, sizeof(float) * (size_t)N);
  oracle_dequant_gemv_w8a32(x, W, s, y, K, N);
  if (bias)
    for (int64_t n = 0; n < N; ++n)
      y[n] = bias[n] + y[n];
}

/* q/k/v of the shipped w8a32 build: f32 weights through the plain decode GEMV
 * (MatMulVectorizationDecode.cpp:142-175) into a zero tensor, then bias + y
 * (subgraph0_decode_simplify.mlir:73-85). */
static void linear_f32(const float *x, const float *W, const float *bias, float *y,
                       int64_t K, int64_t N) {
  memset(y, 0, sizeof(float) * (size_t)N);
  oracle_gemv_f32(x, W, y, K, N, 32, 0);
  if (bias)
    for (int64_t n = 0; n < N; ++n)
      y[n] = bias[n] + y[n];
}

int64_t oracle_decode_step(const oracle_model *m, int64_t token, int64_t pos,
                           float **kv, float *logits) {
  const oracle_shape *S = &m->shape;
  const int64_t H = S->hidden, D = S->head_dim, I = S->inter;
  const int64_t QN = S->heads * D, KVN = S->kv_heads * D;
  const float inv_h = 1.0f / (float)H; /* 6.51041686e-4 for 1536 (:8) */
  float *x = (float *)malloc(sizeof(float) * H);
  float *xn = (float *)malloc(sizeof(float) * H);
  float *q = (float *)malloc(sizeof(float) * QN);
  float *k = (float *)malloc(sizeof(float) * KVN);
  float *v = (float *)malloc(sizeof(float) * KVN);
  float *att = (float *)malloc(sizeof(float) * QN);
  float *o = (float *)malloc(sizeof(float) * H);
  float *g = (float *)malloc(sizeof(float) * I);
  float *u = (float *)malloc(sizeof(float) * I);
  float *hh = (float *)malloc(sizeof(float) * I);
  float *mask = (float *)malloc(sizeof(float) * S->max_len);
  float cosv[1024], sinv[1024];

  /* embedding gather (:46-48) */
  memcpy(x, m->embed + token * H, sizeof(float) * H);
  /* mask[k] = pos >= k ? 0 : -inf (:50,:143-150) */
  for (int64_t j = 0; j < S->max_len; ++j)
    mask[j] = pos >= j ? 0.0f : -INFINITY;
  oracle_rope_cos_sin(m->inv_freq, D / 2, pos, cosv, sinv);
  const float scale = (float)(1.0 / sqrt((double)D)); /* 0.0883883461 (:17) */

  for (int64_t L = 0; L < S->layers; ++L) {
    const oracle_layer *W = &m->layer[L];
    float *Kc = kv[2 * L], *Vc = kv[2 * L + 1];
    oracle_rmsnorm(x, W->ln1, xn, H, inv_h, S->eps);
    if (W->wq) {
      linear(xn, W->wq, W->sq, W->bq, q, H, QN);
      linear(xn, W->wk, W->sk, W->bk, k, H, KVN);
      linear(xn, W->wv, W->sv, W->bv, v, H, KVN);
    } else {
      linear_f32(xn, W->fq, W->bq, q, H, QN);
      linear_f32(xn, W->fk, W->bk, k, H, KVN);
      linear_f32(xn, W->fv, W->bv, v, H, KVN);
    }
    oracle_rope_apply(q, S->heads, D, cosv, sinv);
    oracle_rope_apply(k, S->kv_heads, D, cosv, sinv);
    /* KV write: cache[0, h, pos, :] = k' / v (:108-142) */
    for (int64_t h = 0; h < S->kv_heads; ++h) {
      memcpy(Kc + (h * S->max_len + pos) * D, k + h * D, sizeof(float) * D);
      memcpy(Vc + (h * S->max_len + pos) * D, v + h * D, sizeof(float) * D);
    }
    oracle_gqa_decode_attention(q, Kc, Vc, mask, att, NULL, S->heads,
                                S->kv_heads, S->max_len, D, scale,
                                S->attn_splits);
    linear(att, W->wo, W->so, NULL, o, QN, H);
    for (int64_t i = 0; i < H; ++i)
      x[i] = x[i] + o[i]; /* (:207-209) */
    oracle_rmsnorm(x, W->ln2, xn, H, inv_h, S->eps);
    linear(xn, W->wg, W->sg, NULL, g, H, I);
    linear(xn, W->wu, W->su, NULL, u, H, I);
    oracle_silu_mul(g, u, hh, I);
    linear(hh, W->wd, W->sd, NULL, o, I, H);
    for (int64_t i = 0; i < H; ++i)
      x[i] = x[i] + o[i];
  }
  oracle_rmsnorm(x, m->ln_f, xn, H, inv_h, S->eps); /* (:4986-4998) */
  linear(xn, m->w_lm, m->s_lm, NULL, logits, H, S->vocab); /* (:4999-5003) */
  int64_t tok = oracle_argmax_first(logits, S->vocab);
  free(x); free(xn); free(q); free(k); free(v); free(att); free(o);
  free(g); free(u); free(hh); free(mask);
  return tok;
}
