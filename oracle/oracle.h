/*
 * oracle.h -- CPU restatement of buddy-mlir's int8 weight-only (w8a32) LLM
 * decode / prefill arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This is the parity checker and the timed CPU
 * baseline.  Nothing in the shipped library links, loads or calls it; only the
 * test-suite, the smoke check and the benchmark's cpu_baseline leg do.
 *
 * Every function restates the loop nest that one of the reference's MLIR
 * rewrite patterns (or Python lowering) emits, with the same operation order
 * and the same fused / unfused multiply-adds, and cites the reference file:line
 * it follows.  Build with -ffp-contract=off so that only explicit fmaf() calls
 * are fused, exactly where the reference emits vector.fma / math.fma.
 *
 * Pin status (what each function has been checked against, see tests/):
 *   quantize_w8 ............ closed forms + torch.round/f32 division (library)
 *   pack_panels ............ reference lit vector (K=128,N=64,V=32) + closed form
 *   gemv_packed_f32 ........ closed form vs float64, zero-init semantics
 *   dequant_gemv_w8a32 ..... reference known-answer vector [[8,8,0,...]] + float64
 *   blis_gemm .............. reference vectors (all 14; rows [8,8,8,8]) + float64
 *   gqa_decode_attention ... float64 two-pass softmax at the reference's stated
 *                            valid lengths/splits, -inf mask, lse identity
 *   prefill_flash_attention  float64 two-pass causal softmax + torch SDPA fixture
 *   rmsnorm/rope/silu_mul .. closed forms with the IR's constants, invariants
 *   argmax_first ........... first-index tie rule
 *   w8a8_matmul ............ exact int64 brute force
 *   decode_step ............ composition; cross-checked against an independent
 *                            numpy float64 model in the tests, and against the
 *                            logits of the pip `transformers` Qwen2 model for a
 *                            seeded tiny decoder (tests/golden fixture)
 *   kv_discard, kv_adjust_rope  the reference's own KVCacheManager.h built as
 *                            _ref/libref_llm.so (bit for bit); numpy slice
 *                            assignment; rotation by -d against the pinned RoPE
 *   f32_to_f16, pack_int4, w4a16_gemv  numpy.float16; closed form over all byte
 *                            values; the reference example's inputs
 *   sampler (sampler.cpp) .. the reference's own Sampler.h built as
 *                            _ref/libref_llm.so (token for token); numpy
 *                            re-derivation of the whole pipeline and of the
 *                            draw (MT19937 output sequence, libstdc++'s
 *                            canonical double and discrete_distribution);
 *                            closed-form frequencies
 * Parity unpinned: the order of parameters inside the reference's weight blobs
 * (no blob written by the reference's importer exists to check it against).
 */
#ifndef BUDDY_ORACLE_H
#define BUDDY_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- a1: per-output-channel symmetric quantizer ------------------------- */
/* tools/buddy-codegen/import_model.py:827-848,874-880 */
void oracle_quantize_w8(const float *W, int64_t K, int64_t N, int8_t *q,
                        float *scale);
/* W4 flavour of the same recipe (amax/7, clamp -8..7), one value per byte. */
void oracle_quantize_w4(const float *W, int64_t K, int64_t N, int8_t *q,
                        float *scale);

/* ---- a3: reference panel packing ---------------------------------------- */
/* frontend/Python/graph/transform/pack_decode_weights.py:94-108 */
int oracle_pack_panels(const void *B, int64_t K, int64_t N, int64_t V,
                       size_t elem, void *out);
int oracle_unpack_panels(const void *P, int64_t K, int64_t N, int64_t V,
                         size_t elem, void *out);

/* ---- a4 / a6: f32 decode GEMV, packed and plain ------------------------- */
/* MatMulVectorizationDecodePacked.cpp:207-248 */
void oracle_gemv_packed_f32(const float *A, const float *flatB, float *C,
                            int64_t K, int64_t N, int64_t V, int zero_init);
/* MatMulVectorizationDecode.cpp:142-175 */
void oracle_gemv_f32(const float *A, const float *B, float *C, int64_t K,
                     int64_t N, int64_t V, int zero_init);

/* ---- a5: int8 dequant decode GEMV (C += (A . W) * scale) ---------------- */
/* DequantMatMulVectorizationDecode.cpp:250-321 */
void oracle_dequant_gemv_w8a32(const float *A, const int8_t *W,
                               const float *scale, float *C, int64_t K,
                               int64_t N);
/* The same loop nest reading an int8 matrix stored in the reference's panel
 * order (the f32 packing idea applied to int8; not in the reference). */
void oracle_dequant_gemv_w8a32_panels(const float *A, const int8_t *Wp,
                                      const float *scale, float *C, int64_t K,
                                      int64_t N);

/* ---- a7: BLIS 5-loop GEMM, optional dequant fused into B packing -------- */
/* MatMulBlisVectorization.cpp:351-360,398-986 */
void oracle_blis_gemm_f32(const float *A, const float *B, float *C, int64_t M,
                          int64_t N, int64_t K);
void oracle_blis_gemm_w8a32(const float *A, const int8_t *W,
                            const float *scale, float *C, int64_t M, int64_t N,
                            int64_t K);

/* ---- a8: GQA decode attention ------------------------------------------- */
/* frontend/Python/ops/tosa.py:13966-13975,14087-14090,14130-14600 */
void oracle_gqa_decode_attention(const float *q, const float *kcache,
                                 const float *vcache, const float *mask,
                                 float *out, float *lse, int64_t n_heads,
                                 int64_t n_kv_heads, int64_t cache_len,
                                 int64_t head_dim, float scale,
                                 int64_t num_splits);

/* ---- a9: prefill flash attention ---------------------------------------- */
/* frontend/Python/ops/tosa.py:4376-4384,4415-4416,4431-4799 */
void oracle_prefill_flash_attention(const float *q, const float *k,
                                    const float *v, const float *mask,
                                    float *out, int64_t n_heads, int64_t q_len,
                                    int64_t k_len, int64_t head_dim,
                                    float scale);

/* ---- a10: element-wise chain -------------------------------------------- */
/* examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:60-72 */
void oracle_rmsnorm(const float *x, const float *w, float *y, int64_t n,
                    float inv_n, float eps);
/* :51-59 (angles) and :88-107 (rotate-half) */
void oracle_rope_cos_sin(const float *inv_freq, int64_t half, int64_t pos,
                         float *cosv, float *sinv);
void oracle_rope_apply(float *x, int64_t n_heads, int64_t head_dim,
                       const float *cosv, const float *sinv);
/* :225-232 */
void oracle_silu_mul(const float *g, const float *u, float *h, int64_t n);

/* ---- a11: greedy sampling ----------------------------------------------- */
/* runtime/include/buddy/runtime/llm/Sampler.h:101-104 */
int64_t oracle_argmax_first(const float *x, int64_t n);

/* ---- a14: w8a8 matmul with int32 partial sums --------------------------- */
/* frontend/Python/ops/linalg.py:12737-12845 */
void oracle_w8a8_quantize_activation(const float *x, int64_t n, int8_t *xq,
                                     float *scale);
void oracle_w8a8_matmul(const float *A, const int8_t *W, const float *wscale,
                        float *C, int32_t *acc_out, int64_t M, int64_t N,
                        int64_t K);

/* ---- a10 + a12: one decode step of a Qwen2-shaped decoder --------------- */
typedef struct {
  int64_t layers, hidden, heads, kv_heads, head_dim, inter, vocab, max_len;
  float eps;
  int64_t attn_splits; /* 4 in the reference when max_len % 64 == 0 */
} oracle_shape;

typedef struct {
  const float *ln1, *ln2;               /* [hidden] */
  const int8_t *wq, *wk, *wv, *wo;      /* [K,N] row-major */
  const float *sq, *sk, *sv, *so;       /* [N] */
  const float *bq, *bk, *bv;            /* [N] or NULL */
  const int8_t *wg, *wu, *wd;
  const float *sg, *su, *sd;
  /* q/k/v kept in f32 [K,N] (the reference's shipped w8a32 build): used when
   * wq is NULL, with the f32 decode GEMV and the bias add */
  const float *fq, *fk, *fv;
} oracle_layer;

typedef struct {
  oracle_shape shape;
  const float *embed;      /* [vocab, hidden] f32 */
  const float *inv_freq;   /* [head_dim/2] */
  const oracle_layer *layer;
  const float *ln_f;       /* [hidden] */
  const int8_t *w_lm;      /* [hidden, vocab] */
  const float *s_lm;       /* [vocab] */
} oracle_model;

/* kv: 2*layers caches, even = K, odd = V, each [kv_heads, max_len, head_dim].
 * Writes logits[vocab]; returns the greedy token. */
int64_t oracle_decode_step(const oracle_model *m, int64_t token, int64_t pos,
                           float **kv, float *logits);

int oracle_num_threads(void);

/* ---- KV-cache overflow handling (kv_cache.c) -------------------------------
 * runtime/include/buddy/runtime/llm/KVCacheManager.h:150-194, :200-268.
 * Pinned by: numpy slicing of the same move, rotation by -d composed with the
 * RoPE of position p equals the RoPE of position p - d, rotation by -d then +d
 * is the identity within rounding. */
int oracle_kv_discard(float *cache, int64_t heads, int64_t max_len, int64_t dim,
                      int64_t keep, int64_t discard, int64_t count);
void oracle_kv_adjust_rope(float *kcache, int64_t heads, int64_t max_len, int64_t dim,
                           int64_t keep, int64_t discard, int64_t count,
                           const float *inv_freq);

/* ---- int4 weight-only decode path, W4A16 (w4a16.c) -------------------------
 * tools/buddy-codegen/import_model.py:810-815 (nibble packing),
 * Int4DequantMatMulVectorizationDecode.cpp:385-468 (kernel, f16 throughout).
 * f16 values travel as their bit patterns (uint16_t).
 * Pinned by: numpy.float16 for the conversions; a numpy.float16 emulation of the
 * sequential f16 accumulation; the reference example's inputs
 * (examples/BuddyMatmul/int4-dequant-matmul-vectorization-decode.mlir:177-190:
 * A = 1, bytes = 2, scale = 1 -> [8, 0, 8, 0]); pack/unpack round trip over all
 * 256 byte values. */
void oracle_f32_to_f16(const float *x, int64_t n, uint16_t *y);
void oracle_f16_to_f32(const uint16_t *x, int64_t n, float *y);
int oracle_pack_int4(const int8_t *q, int64_t n, int8_t *packed);
void oracle_unpack_int4(const int8_t *packed, int64_t n, int8_t *q);
void oracle_w4a16_gemv(const uint16_t *a, const int8_t *packed, const uint16_t *scale,
                       uint16_t *c, int64_t K, int64_t N);

#ifdef __cplusplus
}
#endif
#endif
