/*
 * buddy_hip.h -- C ABI of libbuddy_hip.so: buddy-mlir's int8 weight-only
 * (w8a32) LLM decode / prefill arithmetic as hand-written HIP kernels for
 * gfx950 (MI355X).
 *
 * Two layers are exported.
 *
 *  (1) `_mlir_ciface_*` entry points that take pointers to memref descriptors,
 *      the convention of buddy-mlir's external kernels
 *      (runtime/include/buddy/runtime/Matmul.h:35-36,
 *      runtime/external_kernels/matmul/MatmulTorq.cpp:116-166) and of the
 *      compiled model library (tools/buddy-codegen/gen_session.py:974-1007).
 *      Data pointers may be host or device memory.
 *
 *  (2) `buddy_hip_*` entry points that take plain device pointers and sizes
 *      and launch on a caller-supplied HIP stream.  They are what layer (1)
 *      is built from and what a resident-weights caller uses directly.
 *
 * Every function returns 0 on success and a non-zero code on failure unless it
 * is `void` by the reference's convention; failures also print one
 * `[buddy_hip] ...` line to stderr and are queryable with
 * buddy_hip_last_error().  Nothing unwinds through this boundary.
 * Calls on one stream are ordered.
 */
#ifndef BUDDY_HIP_H
#define BUDDY_HIP_H

#include "buddy_hip/memref.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef void *buddy_hip_stream; /* a hipStream_t; NULL = the default stream */

enum {
  BUDDY_HIP_OK = 0,
  BUDDY_HIP_ERR_ARG = 1,     /* shape / pointer / size check failed */
  BUDDY_HIP_ERR_HIP = 2,     /* a HIP runtime call failed */
  BUDDY_HIP_ERR_NO_DEVICE = 3,
  BUDDY_HIP_ERR_HOST = 4     /* host side: out of memory or a C++ exception,
                                caught at this boundary */
};

/* ---- library ---------------------------------------------------------- */
const char *buddy_hip_version(void);
const char *buddy_hip_last_error(void);
int buddy_hip_device_count(void);

/* Which compiled variants of the hand-scheduled kernels (the ones that issue
 * their global loads by hand) this process has launched.  Writes one line per
 * variant, "name<template arguments>\tlaunch count\n", into `text` (at most
 * capacity - 1 characters and a terminating 0) and returns the size the whole
 * report needs.  A variant is listed from the moment the library is loaded,
 * launched or not, so a test can tell which ones its cases did not reach.
 * buddy_hip_variant_reset sets every count back to 0.  Host only; no
 * counterpart in the reference. */
int64_t buddy_hip_variant_report(char *text, int64_t capacity);
void buddy_hip_variant_reset(void);

/* ---- packed int8 weight layout ("wave tiles") --------------------------
 * Replaces frontend/Python/graph/transform/pack_decode_weights.py:102-108
 * (panels [N/V][K][V], refused for int8 by tools/buddy-codegen/gen_config.py:
 * 366-370) with a layout cut for 64-lane wavefronts issuing 128-bit loads:
 * the matrix W[K,N] is padded to Kp = ceil64(K), Np = ceil16(N) and stored as
 * tiles of 16 output channels x 64 k (1 KiB).  Tile (g = n/16, c = k/64) is at
 * byte ((g * Kp/64) + c) * 1024; inside it lane L (0..63) owns 16 consecutive
 * bytes holding k = c*64 + (L/16)*16 + 0..15 of channel n = g*16 + L%16.
 * A wavefront's one load instruction therefore reads one contiguous KiB and a
 * channel group's whole K extent is one contiguous run.  Padding is zero. */
size_t buddy_hip_w8_packed_bytes(int64_t K, int64_t N);
/* W: device int8 [K,N] row-major (the reference layout).  packed: device. */
int buddy_hip_pack_w8(const int8_t *W, int64_t K, int64_t N, int8_t *packed,
                      buddy_hip_stream stream);
int buddy_hip_unpack_w8(const int8_t *packed, int64_t K, int64_t N, int8_t *W,
                        buddy_hip_stream stream);
/* Narrower tiles for narrow matrices at M = 1 (down / o_proj: 1536 outputs are
 * only 96 groups of 16, fewer than the 256 CUs): a tile is tile_n channels x
 * (1024 / tile_n) k, tile_n = 16 (as above), 8 or 4; lane L owns channel
 * g*tile_n + L % tile_n and k = c*(1024/tile_n) + (L / tile_n)*16 + 0..15.
 * Only buddy_hip_linear_w8a32 with M = 1 and one matrix reads these. */
size_t buddy_hip_w8_packed_bytes_tiles(int64_t K, int64_t N, int tile_n);
int buddy_hip_pack_w8_tiles(const int8_t *W, int64_t K, int64_t N, int tile_n,
                            int8_t *packed, buddy_hip_stream stream);
int buddy_hip_unpack_w8_tiles(const int8_t *packed, int64_t K, int64_t N,
                              int tile_n, int8_t *W, buddy_hip_stream stream);

/* ---- per-output-channel symmetric quantizer ----------------------------
 * tools/buddy-codegen/import_model.py:837-848,874-880 on device: W f32 [K,N],
 * q int8 [K,N], scale f32 [N].  Bit-exact with the reference recipe. */
int buddy_hip_quantize_w8(const float *W, int64_t K, int64_t N, int8_t *q,
                          float *scale, buddy_hip_stream stream);

/* ---- int4 weight-only decode path (W4A16) -------------------------------
 * The same recipe with amax/7 and a clamp to [-8, 7]
 * (tools/buddy-codegen/import_model.py:800-802,838-842), the nibble packing of
 * import_model.py:810-815 (element 2i in the low nibble, 2i+1 in the high one;
 * for a row-major [K,N] matrix: even channel low, odd channel high), and the
 * decode GEMV of Int4DequantMatMulVectorizationDecode.cpp:385-468:
 *   C[n] = C[n] + (sum_k A[k] * w[k][n]) * scale[n]
 * with f16 A [K], scale [N] and C [N] (bit patterns) and packed [K, N/2]
 * bytes.  The sum runs in the reference's order, rounded to f16 after every
 * step, so the result is the reference's bit for bit. */
int buddy_hip_quantize_w4(const float *W, int64_t K, int64_t N, int8_t *q,
                          float *scale, buddy_hip_stream stream);
int buddy_hip_pack_int4(const int8_t *q, int64_t count, int8_t *packed,
                        buddy_hip_stream stream);
int buddy_hip_gemv_w4a16(const uint16_t *A, const int8_t *packed, const uint16_t *scale,
                         uint16_t *C, int64_t K, int64_t N, buddy_hip_stream stream);
/* The same operands with another summation, opt-in:
 *   C[n] = f16(f32(C[n]) + (sum_k A[k] * w[k][n]) * f32(scale[n]))
 * with exact products and a sum that is exact up to one rounding of every
 * activation to 2^-31 of the largest of its run of 128..1024 values, rounded to
 * f16 once at the end.  The reference's f16 chain
 * (Int4DequantMatMulVectorizationDecode.cpp:438-446) rounds after every one of
 * its K steps, so this result is at least as close to the real-number sum as
 * the reference's own but is not the reference's bit for bit; in exchange the
 * launch is bound by the half byte per weight it reads (the bit-exact kernel
 * above by its chain of K dependent roundings).  A NaN or an infinity among
 * the activations of a run turns C into NaN.  The weights come as "int4 wave
 * tiles" (16 channels x 128 k per KiB, in the order the int8 matrix cores take
 * them), made once from the reference's [K, N/2] bytes by
 * buddy_hip_pack_w4_tiles into buddy_hip_w4_tiles_bytes(K, N) bytes (16-byte
 * aligned; K and N are zero padded inside).  A: 8-byte aligned.  No counterpart
 * in the reference. */
size_t buddy_hip_w4_tiles_bytes(int64_t K, int64_t N);
int buddy_hip_pack_w4_tiles(const int8_t *packed, int64_t K, int64_t N, int8_t *tiles,
                            buddy_hip_stream stream);
int buddy_hip_gemv_w4a16_fast(const uint16_t *A, const int8_t *tiles, const uint16_t *scale,
                              uint16_t *C, int64_t K, int64_t N, buddy_hip_stream stream);

/* ---- int8 dequant decode GEMV / small-batch matmul ---------------------
 * Replaces the kernel that
 * midend/lib/Conversion/MatMulOptimization/DequantMatMulVectorizationDecode.cpp
 * :250-321 generates:  C[m,n] (+)= (sum_k A[m,k] * W[k,n]) * scale[n].
 * M is 1..16 (the reference pattern is m == 1 only; M > 1 streams the weights
 * once for all rows).  A: f32 [M,K] row-major (lda = K), C: f32 [M,N].
 * Up to 4 rows, with at most 16 tiles of 64 k per wavefront (every matrix of a
 * decoder layer) and 16-byte aligned rows, run on the int8 matrix cores: a
 * wavefront rounds the 64..1024 activations of a row it multiplies to 2^-31 of
 * the largest of them (one within 2^7 of it keeps all 24 bits), the products
 * and sums are exact, and a NaN or an infinity turns the
 * row of C into NaN; the environment variable BUDDY_HIP_GEMV_ROW=f32, read once
 * per process, keeps the f32 multiply-add kernel instead.  Longer runs and
 * unaligned rows: every product is
 * an f32 multiply-add.  From 5 rows (with K a
 * multiple of 4 and A 16-byte aligned) the int8 matrix cores are used: the
 * activations of a row are rounded, 64 at a time, to 2^-23 of the largest of
 * the 64, the sums are exact; a NaN or an infinity in a row turns that row of C
 * into NaN.  buddy_hip_set_gemv_batch_kernel(BUDDY_HIP_GEMV_BATCH_BF16) makes
 * those batches keep every bit of the activations instead, on the bf16 matrix
 * cores, at about two thirds of the speed; the environment variable
 * BUDDY_HIP_GEMV_BATCH=bf16, read once per process, sets that as the default.
 * The choice is process-wide.  (No counterpart in the reference, whose decode
 * pattern is m == 1 only.) */
enum { BUDDY_HIP_GEMV_BATCH_INT8 = 0, BUDDY_HIP_GEMV_BATCH_BF16 = 1 };
int buddy_hip_set_gemv_batch_kernel(int kernel);
enum {
  BUDDY_HIP_GEMV_ACCUMULATE = 1 /* C += ...  (linalg.matmul semantics);
                                   without it C = ... and C need not be
                                   initialised */
};
/* How a launch of buddy_hip_gemv_w8a32 / buddy_hip_linear_w8a32 would be cut:
 * host arithmetic only, nothing is launched and no device is touched.  For
 * tests of the launch shapes, and for callers that want to know which kernel a
 * shape gets.  (No counterpart in the reference, whose loop nest is fixed at
 * compile time.) */
enum {
  BUDDY_HIP_PLAN_TWO_MATRICES = 1,   /* the SiLU(gate) * up form */
  BUDDY_HIP_PLAN_FOLD_INPUT = 2,     /* input folded from attention partials */
  BUDDY_HIP_PLAN_UNALIGNED_ROWS = 4  /* A or lda not a multiple of 16 bytes */
};
enum {
  BUDDY_HIP_PLAN_DIGITS = 0,     /* digit planes on the int8 matrix cores, 1..4 rows */
  BUDDY_HIP_PLAN_F32 = 1,        /* f32 multiply-add kernel */
  BUDDY_HIP_PLAN_BATCH_INT8 = 2, /* 5..16 rows, int8 matrix cores */
  BUDDY_HIP_PLAN_BATCH_BF16 = 3  /* 5..16 rows, bf16 matrix cores */
};
typedef struct {
  int32_t kernel;               /* BUDDY_HIP_PLAN_* */
  int32_t rows_compiled;        /* rows the kernel variant is compiled for */
  int32_t channel_groups;       /* ceil(N / 16) */
  int32_t tiles;                /* ceil(K / 64): 1 KiB tiles per channel group */
  int32_t groups_per_workgroup; /* channel groups a workgroup covers */
  int32_t k_slices;             /* wavefronts that share one channel group */
  int32_t wavefronts;           /* per workgroup */
  int32_t workgroups;
  int32_t split;                /* 1: two workgroups per channel group */
  int32_t tiles_per_wavefront;
  int32_t slots;                /* tile slots of the digit-plane variant, else 0 */
  int32_t reserved;
  int64_t lds_bytes;            /* dynamic LDS of one workgroup */
} buddy_hip_gemv_plan;
int buddy_hip_gemv_w8a32_plan(int64_t M, int64_t K, int64_t N, unsigned flags,
                              buddy_hip_gemv_plan *out);

int buddy_hip_gemv_w8a32(const float *A, const int8_t *packed,
                         const float *scale, float *C, int64_t M, int64_t K,
                         int64_t N, unsigned flags, buddy_hip_stream stream);

/* One MLP block of a decoder layer at a decode batch of M = 1..16 rows:
 *   y (+)= (SiLU(x' . gate) * (x' . up)) . down,   x' = RMSNorm(x) * norm_w or x
 * (subgraph0_decode_simplify.mlir:210-260 over M rows): the two launches of
 * buddy_hip_linear_w8a32 that make it (gate and up fused with SiLU * mul, then
 * down) behind one call, with the same kernels and roundings.  All three
 * matrices are wave-tile packed ([hidden, inter] twice, [inter, hidden]).  The
 * intermediate rows [M, inter] f32 live in `workspace`
 * (buddy_hip_mlp_block_workspace_bytes(M, inter) bytes, 16-byte aligned).  No
 * counterpart in the reference, whose decode kernels are m == 1 only. */
typedef struct buddy_hip_mlp_block_desc {
  const float *x;          /* [M, hidden], row stride ldx */
  int64_t ldx;
  const float *norm_w;     /* [hidden] or NULL; 16-byte aligned */
  float norm_eps;
  const int8_t *gate;      /* packed [hidden, inter] */
  const float *gate_scale; /* [inter] */
  const int8_t *up;
  const float *up_scale;
  const int8_t *down;      /* packed [inter, hidden] */
  const float *down_scale; /* [hidden] */
  float *y;                /* [M, hidden], row stride ldy */
  int64_t ldy;
  int64_t M, hidden, inter;
  unsigned flags;          /* BUDDY_HIP_GEMV_ACCUMULATE: y += ... (the residual) */
  void *workspace;
  size_t workspace_bytes;
} buddy_hip_mlp_block_desc;
size_t buddy_hip_mlp_block_workspace_bytes(int64_t M, int64_t inter);
int buddy_hip_mlp_block_w8a32(const buddy_hip_mlp_block_desc *d, buddy_hip_stream stream);

/* Full form of the kernel above with the fusions a decoder layer uses.
 * Every pointer is device memory. */
typedef struct buddy_hip_linear_desc {
  const float *A;       /* [M, K], row stride lda (>= K) */
  int64_t lda;
  const int8_t *W0;     /* wave-tile packed [K, N] */
  const float *scale0;  /* [N] */
  const int8_t *W1;     /* second matrix (epilogue SILU_MUL) or NULL */
  const float *scale1;
  const float *bias;    /* [N] or NULL: C = bias + acc*scale (epilogue STORE) */
  const float *norm_w;  /* [K] or NULL: RMSNorm applied to A first
                           (subgraph0_decode_simplify.mlir:60-72); 16-byte
                           aligned, other addresses are refused */
  float norm_eps;
  float *C;             /* [M, N], row stride ldc (>= N) */
  int64_t ldc;
  int64_t M, K, N;      /* M in 1..16 */
  int epilogue;         /* BUDDY_HIP_EPI_* */
  int tile_n;           /* channels per packed tile: 0 or 16 (default), 8, 4 */
} buddy_hip_linear_desc;
enum {
  BUDDY_HIP_EPI_STORE = 0,   /* C = acc*scale (+ bias) */
  BUDDY_HIP_EPI_ACCUM = 1,   /* C = C + acc*scale (residual add) */
  BUDDY_HIP_EPI_SILU_MUL = 2 /* C = silu(acc0*scale0) * (acc1*scale1)
                                (subgraph0_decode_simplify.mlir:225-232) */
};
int buddy_hip_linear_w8a32(const buddy_hip_linear_desc *desc,
                           buddy_hip_stream stream);

/* ---- int8 dequant prefill matmul on the matrix cores ----------------------
 * Replaces the BLIS-style kernel with dequantisation fused into B packing
 * (midend/lib/Conversion/MatMulOptimization/MatMulBlisVectorization.cpp:351-360,
 * 398-986): C[M,N] (+)= A[M,K] . (W[K,N] * scale[N]), any M.  `packed` is the
 * same wave-tile copy the decode kernel reads.  Activations are cast to bf16
 * (round to nearest even) and multiplied on MFMA with f32 accumulation; with
 * BUDDY_HIP_GEMM_A_F32_EXACT each activation is carried as three bf16 terms,
 * i.e. with all 24 significand bits.  With BUDDY_HIP_GEMM_A_I8_DIGITS the
 * activations become fixed point instead -- per row a power-of-two step s with
 * |a| / s < 2^22, rint(a / s) written as three balanced base-256 digits -- and
 * the int8 weights are multiplied as they are on the int8 matrix cores, with
 * exact int32 sums: the only rounding is that of a, at most 2^-23 of the row's
 * largest magnitude (a NaN or an infinity in a row turns that row of C into
 * NaN; K <= 2^17).  BUDDY_HIP_GEMM_TWO_DIGITS (with BUDDY_HIP_GEMM_A_I8_DIGITS)
 * keeps two digits, |a| / s < 2^14: the rounding is 2^-15 of the row's largest
 * magnitude -- the fixed-point counterpart of casting the activations to bf16
 * (2^-9 of each value), for two thirds of the matrix instructions.
 * BUDDY_HIP_GEMV_ACCUMULATE as above.
 * BUDDY_HIP_GEMM_SILU_PAIR (with BUDDY_HIP_GEMM_A_I8_DIGITS; N % 16 == 0; no
 * accumulation): `packed` holds two [K,N] matrices one behind the other, each
 * packed on its own, `scale` 2 N values, and C[M,N] = SiLU(A . W0) * (A . W1),
 * the prefill form of BUDDY_HIP_EPI_SILU_MUL
 * (subgraph0_decode_simplify.mlir:225-232 over M rows). */
enum {
  BUDDY_HIP_GEMM_A_F32_EXACT = 2,
  BUDDY_HIP_GEMM_A_I8_DIGITS = 4,
  BUDDY_HIP_GEMM_SILU_PAIR = 8,
  BUDDY_HIP_GEMM_TWO_DIGITS = 16
};
int buddy_hip_gemm_w8a32(const float *A, const int8_t *packed, const float *scale,
                         float *C, int64_t M, int64_t K, int64_t N,
                         unsigned flags, buddy_hip_stream stream);

/* ---- element-wise pieces of a decoder layer ------------------------------
 * Stand-alone forms of what the decode step runs fused; constants and op order
 * from examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:51-72,88-107,
 * 225-232.  `pos` is a device scalar. */
int buddy_hip_rmsnorm(const float *x, const float *w, float *y, int rows, int n,
                      float eps, buddy_hip_stream stream);
int buddy_hip_rope(float *x, const float *inv_freq, const int *pos, int n_heads,
                   int head_dim, buddy_hip_stream stream);
int buddy_hip_silu_mul(const float *g, const float *u, float *h, int64_t n,
                       buddy_hip_stream stream);
/* Greedy sampling: the FIRST index of the maximum, like std::max_element
 * (runtime/include/buddy/runtime/llm/Sampler.h:101-104). */
size_t buddy_hip_argmax_workspace_bytes(void);
int buddy_hip_argmax(const float *x, int n, void *workspace, int *out_index,
                     buddy_hip_stream stream);

/* ---- GQA decode attention -------------------------------------------------
 * Replaces gqa_attention_fused_op (frontend/Python/ops/tosa.py:14130-14600)
 * together with the RoPE and KV-cache write in front of it
 * (subgraph0_decode_simplify.mlir:88-142).  qkv = [q | k | v] as the
 * projections leave them (before RoPE); the kernel rotates q and k, writes k'
 * and v into row *pos of the caches ([kv_heads, max_len, head_dim] f32 each)
 * and attends over rows 0..*pos.  out: [heads*head_dim].  lse: [heads] or NULL,
 * the op's second result, max + log(sum) of each head's scaled scores
 * (tosa.py:14576-14594).  head_dim must be 128.  *pos must lie in
 * 0..max_len-1; a position outside writes no cache row.  qkv, inv_freq and the
 * caches must be 16-byte aligned (the kernels read them four floats at a time);
 * other addresses are refused. */
size_t buddy_hip_attn_decode_workspace_bytes(int heads, int max_len);
/* How the session cuts the attention of a decode step at position `pos` (host
 * arithmetic, no device needed): cache positions per partial (64, 128 or 256),
 * partials per head the step produces and folds (they cover the position), and
 * whether a launch of its own folds them (1) or the o_proj launch does (0).
 * No counterpart in the reference (its cache length is a compile-time tier,
 * tools/buddy-codegen/gen_session.py:358-379). */
int buddy_hip_attn_step_plan(int pos, int max_len, int kv_heads, int *chunk, int *partials,
                             int *own_fold);
int buddy_hip_gqa_decode_attention(const float *qkv, const float *inv_freq,
                                   const int *pos, float *kcache, float *vcache,
                                   float *out, float *lse, int heads,
                                   int kv_heads, int head_dim, int max_len,
                                   float scale, void *workspace,
                                   size_t workspace_bytes,
                                   buddy_hip_stream stream);

/* The same call for callers that cannot allocate device memory or pass a
 * workspace around (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The flash-decoding partials go to a buffer built into the library (4.06 MiB
 * of device memory per GPU, held until the process ends) instead of a
 * caller's workspace, and the call allocates nothing.  Limit: heads x
 * ceil(max_len / 64) <= 8192 (e.g. 32 heads x 16384 positions); larger shapes
 * are refused with BUDDY_HIP_ERR_ARG.  Results are bit-identical to
 * buddy_hip_gqa_decode_attention.  Every call on a GPU shares that GPU's
 * buffer: calls that overlap on one GPU (two streams, two threads) race; calls
 * on one stream are ordered.  The device that is current at the call must be
 * the stream's device.  The first call on a device looks the buffer's address
 * up in the runtime; a caller that records the call into a HIP graph makes one
 * eager call, or buddy_hip_static_scratch_init() with that device current,
 * before the capture starts (a first call under capture is refused). */
int buddy_hip_gqa_decode_attention_static(const float *qkv, const float *inv_freq,
                                          const int *pos, float *kcache,
                                          float *vcache, float *out, float *lse,
                                          int heads, int kv_heads, int head_dim,
                                          int max_len, float scale,
                                          buddy_hip_stream stream);
/* Resolves the built-in buffer of the current device (no allocation, no
 * launch); idempotent.  No counterpart in the reference. */
int buddy_hip_static_scratch_init(void);

/* ---- prefill attention ----------------------------------------------------
 * Replaces flash_attention_for_cpu_prefill_op
 * (frontend/Python/ops/tosa.py:4326-4810).  q, out: [heads, q_len, head_dim];
 * k, v: [kv_heads, k_len, head_dim] (the reference passes K/V repeated to
 * kv_heads == heads; fewer KV heads are read in place).  mask: additive f32
 * [q_len, k_len], or NULL for the causal mask in which query i sees keys
 * 0 .. k_len - q_len + i.  head_dim must be 128. */
int buddy_hip_prefill_attention(const float *q, const float *k, const float *v,
                                const float *mask, float *out, int heads,
                                int kv_heads, int head_dim, int q_len, int k_len,
                                float scale, buddy_hip_stream stream);

/* ---- plain f32 matmul ---------------------------------------------------
 * C (+)= A[M,K] * B[K,N], all dense row-major device pointers.  The f32
 * sibling of the kernel above (MatMulVectorizationDecode.cpp:142-175); the
 * reference's shipped w8a32 build keeps q/k/v projections in f32. */
int buddy_hip_matmul_f32(const float *A, const float *B, float *C, int64_t M,
                         int64_t N, int64_t K, unsigned flags,
                         buddy_hip_stream stream);

/* ---- resident decoder session ---------------------------------------------
 * A Qwen2-shaped int8 (w8a32) decoder kept on one GPU: weights repacked into
 * wave tiles, f32 KV cache, activations, and one hipGraph per decode step.
 * Stands where the generated ModelSession and the compiled forward_decode
 * stand in the reference (tools/buddy-codegen/gen_session.py:1381-1452;
 * op order of examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:46-260,
 * 4986-5004) and runs the greedy part of runtime/llm/TextGeneration.cpp:215-266
 * on the device.  Field names follow the HF config, not the reference's
 * (its `head_num` is kv_heads and its `hidden_size` is head_dim:
 * tools/buddy-codegen/gen_config.py:288-299).  Not re-entrant per session.
 * max_len is the capacity of the cache only: what a decode step costs follows
 * its position (the attention is cut by it: larger chunks far into a long
 * cache, only the chunks up to the position; one captured graph per cut). */
typedef struct buddy_hip_model_shape {
  int layers, hidden, heads, kv_heads, head_dim, inter, vocab;
  int max_len;    /* KV cache capacity in positions */
  float rms_eps;
} buddy_hip_model_shape;

/* One decoder layer as the importer leaves it: int8 W[K,N] row-major with
 * K = in, N = out (frontend/Python/graph/transform/eliminate_weight_transpose
 * .py:28-41) and f32 scale[N]; biases may be NULL (all three or none).
 * Pointers are device memory and are read only during the call. */
typedef struct buddy_hip_layer_weights {
  const float *ln1, *ln2;
  const int8_t *wq, *wk, *wv, *wo, *wg, *wu, *wd;
  const float *sq, *sk, *sv, *so, *sg, *su, *sd;
  const float *bq, *bk, *bv;
  /* q/k/v kept in f32 [K,N], as in the reference's shipped w8a32 build where
   * they import as AddMMOp and are not quantized (docs/DecodeWeightPacking.md:
   * 128-131): set all three plus the biases and leave wq/wk/wv/sq/sk/sv NULL. */
  const float *fq, *fk, *fv;
} buddy_hip_layer_weights;

typedef struct buddy_hip_session buddy_hip_session;

/* stream NULL: the session creates its own.  Returns NULL on failure. */
buddy_hip_session *buddy_hip_session_create(const buddy_hip_model_shape *shape,
                                            buddy_hip_stream stream);
void buddy_hip_session_destroy(buddy_hip_session *s);
/* embed: f32 [vocab, hidden], borrowed (must outlive the session); the other
 * arguments are copied / repacked: inv_freq f32 [head_dim/2], ln_f f32
 * [hidden], lm_head int8 [hidden, vocab] + scale [vocab]. */
int buddy_hip_session_set_globals(buddy_hip_session *s, const float *embed,
                                  const float *inv_freq, const float *ln_f,
                                  const int8_t *w_lm, const float *s_lm);
int buddy_hip_session_set_layer(buddy_hip_session *s, int index,
                                const buddy_hip_layer_weights *w);
/* KV tensors in the reference's numbering: even index = K, odd = V of layer
 * index/2 (runtime/include/buddy/runtime/llm/KVCacheManager.h:200-201), each
 * f32 [kv_heads, max_len, head_dim]; src/dst may be host or device memory. */
int buddy_hip_session_set_kv(buddy_hip_session *s, int kv_index, const float *src);
int buddy_hip_session_get_kv(buddy_hip_session *s, int kv_index, float *dst);
/* Rows row0 .. row0 + rows - 1 of all 2 * layers caches at once, packed as
 * dst[kv_index][kv_head][row][head_dim] (host or device): the rows a decode
 * step or a prefill just wrote, for a caller that mirrors the caches on the
 * host the way the generated ModelSession does (gen_session.py:1421-1430). */
int buddy_hip_session_get_kv_rows(buddy_hip_session *s, int row0, int rows, float *dst);
/* 1 (default): a decode step is replayed from a captured hipGraph; 0: launched
 * kernel by kernel. */
int buddy_hip_session_use_graph(buddy_hip_session *s, int enable);
/* One decode step for `token` at cache row `pos` (ModelSession::decode).
 * logits_out (host or device, vocab floats) and next_token may be NULL.
 * next_token is the greedy choice (first maximum).  Synchronous. */
int buddy_hip_session_decode(buddy_hip_session *s, int token, int pos,
                             float *logits_out, int *next_token);
/* The same, and the cache rows the step wrote are handed back as well:
 * kv_rows_out (host or device, may be NULL) receives row `pos` of all
 * 2 * layers caches as [kv_index][kv_head][head_dim]. */
int buddy_hip_session_decode_mirror(buddy_hip_session *s, int token, int pos,
                                    float *logits_out, float *kv_rows_out,
                                    int *next_token);
/* `steps` greedy steps starting from first_token at start_pos; each step's
 * argmax feeds the next step on the device.  tokens_out[i] = token chosen by
 * step i.  Synchronous. */
int buddy_hip_session_decode_greedy(buddy_hip_session *s, int first_token,
                                    int start_pos, int steps, int *tokens_out);
/* Prompt processing (ModelSession::prefill, gen_session.py:1345-1369): runs
 * n_tokens tokens (host or device int array) through the decoder as one block,
 * filling cache rows start_pos .. start_pos + n_tokens - 1, on the MFMA matmul
 * and the causal attention kernel.  logits_out (vocab floats) and next_token
 * are for the LAST prompt token, the only row the decode loop reads
 * (runtime/llm/TextGeneration.cpp:191-194).  Synchronous. */
int buddy_hip_session_prefill(buddy_hip_session *s, const int *tokens,
                              int n_tokens, int start_pos, float *logits_out,
                              int *next_token);
/* The same with the logits of every row, [n_tokens, vocab] (host or device):
 * what the compiled forward_prefill returns (PrefillABI, gen_session.py:908-911). */
int buddy_hip_session_prefill_all_logits(buddy_hip_session *s, const int *tokens,
                                         int n_tokens, int start_pos,
                                         float *logits_out);
/* Hands a device allocation to the session, which frees it when destroyed. */
void buddy_hip_session_adopt(buddy_hip_session *s, void *device_ptr);
/* How the prefill matmuls carry their f32 activations:
 * 1: all f32 bits (three bf16 terms); 0: cast to bf16, one MFMA pass instead of
 * three; 2 (default): three int8 digit planes on the int8 matrix cores, 23 bits
 * below each row's largest magnitude (BUDDY_HIP_GEMM_A_I8_DIGITS); 3: two digit
 * planes, 15 bits below it (BUDDY_HIP_GEMM_TWO_DIGITS), the int8 counterpart of
 * mode 0. */
int buddy_hip_session_set_prefill_precision(buddy_hip_session *s, int mode);
/* Asynchronous pieces of the call above, for timing: set the device-side
 * (token, position), then enqueue steps on the session stream. */
int buddy_hip_session_set_state(buddy_hip_session *s, int token, int pos);
int buddy_hip_session_enqueue_steps(buddy_hip_session *s, int steps);
const float *buddy_hip_session_logits(buddy_hip_session *s); /* device */
buddy_hip_stream buddy_hip_session_stream(buddy_hip_session *s);
int buddy_hip_session_vocab(buddy_hip_session *s);

/* ---- token sampler ----------------------------------------------------------
 * buddy::runtime::Sampler (runtime/include/buddy/runtime/llm/Sampler.h:38-46
 * the configuration, :62-206 sample()): repetition penalty over the last
 * repeat_last_n ids, temperature, top-K, min-P, top-P, and a draw from
 * std::discrete_distribution over std::mt19937 seeded with `seed` (0: from
 * std::random_device, :51-56).  temperature 0 is greedy: the first maximum after
 * the penalty (:101-104).  The logits stay on the device: penalty, temperature
 * and the top-K selection run there and top_k (value, id) pairs come back; the
 * rest runs on the host with the same standard-library generator, so a seeded
 * sampler picks the reference's tokens.  Logits of equal value rank by id.
 * top_k 0 (no limit), top_k above BUDDY_HIP_SAMPLER_MAX_TOP_K or a penalty
 * window above 1024 ids copy the logits back and run everything on the host.
 * A sampler owns its generator state and device buffers: one call at a time
 * per sampler. */
#define BUDDY_HIP_SAMPLER_MAX_TOP_K 128
typedef struct buddy_hip_sampler_config {
  float temperature;    /* Sampler.h:39; 0 = greedy */
  int top_k;            /* :40; 0 = no limit */
  float top_p;          /* :41; 1 = off */
  float min_p;          /* :42; 0 = off */
  float repeat_penalty; /* :43; 1 = off */
  int repeat_last_n;    /* :44; the reference's default is 64 */
  uint64_t seed;        /* :45; 0 = from std::random_device */
} buddy_hip_sampler_config;
typedef struct buddy_hip_sampler buddy_hip_sampler;
buddy_hip_sampler *buddy_hip_sampler_create(const buddy_hip_sampler_config *cfg);
void buddy_hip_sampler_destroy(buddy_hip_sampler *s);
/* logits: device (or host-visible) f32[vocab]; recent: host array of the ids
 * generated so far (Sampler.h:63 recentTokens), n_recent may be 0.  Synchronous
 * on `stream`. */
int buddy_hip_sampler_sample(buddy_hip_sampler *s, const float *logits, int vocab,
                             const int *recent, int n_recent, int *token_out,
                             buddy_hip_stream stream);
/* One decode step of the session at (token, pos) followed by a sampled choice
 * from its logits: the non-greedy branch of the generation loop
 * (runtime/llm/TextGeneration.cpp:215-266 with a Sampler). */
int buddy_hip_session_decode_sample(buddy_hip_session *sess, buddy_hip_sampler *s,
                                    int token, int pos, const int *recent,
                                    int n_recent, int *next_token);

/* ---- KV-cache overflow ------------------------------------------------------
 * kvcache::discardKVCache followed by kvcache::adjustKeyCacheRope
 * (runtime/include/buddy/runtime/llm/KVCacheManager.h:150-194, :240-268), on
 * caches that live on the device: keep the first `keep` tokens, drop the next
 * `discard`, move the tail forward, zero the rest, and rotate the moved keys
 * back by `discard` positions.  `count` is the token count before the call.
 * tensors: host array of device pointers to [heads, max_len, head_dim] f32
 * caches, even index = keys, odd = values (KVCacheManager.h:200-201,209).
 * inv_freq: host pointer to head_dim/2 inverse RoPE frequencies; NULL moves
 * without re-rotating.  Parameters the reference refuses (KVCacheManager.h
 * :154-167) are refused here too and leave the caches untouched.  The moved
 * bytes and the rotated keys equal the reference's bit for bit. */
int buddy_hip_kv_discard(float *const *tensors, int num_tensors, int heads, int max_len,
                         int head_dim, int keep, int discard, int count,
                         const float *inv_freq, buddy_hip_stream stream);
/* The same for a session's own caches; the caller continues decoding at
 * position count - discard. */
int buddy_hip_session_discard_kv(buddy_hip_session *s, int keep, int discard,
                                 int count);
/* The same with the caller's inverse frequencies (host, head_dim/2 floats): what
 * ModelSession::handleKVCacheOverflow(keepTokenNum, ropeTheta) does with
 * kvcache::buildInverseRopeFreqs(ropeTheta, head_dim)
 * (tools/buddy-codegen/gen_session.py:1471-1511).  NULL: the session's own. */
int buddy_hip_session_discard_kv_freqs(buddy_hip_session *s, int keep, int discard,
                                       int count, const float *inv_freq);

/* y[N] = bias[N] + x[K] . B[K,N] in f32 (bias may be NULL): the decode GEMV
 * of MatMulVectorizationDecode.cpp:142-175 followed by the q/k/v bias add. */
int buddy_hip_gemv_f32(const float *x, const float *B, const float *bias,
                       float *y, int64_t K, int64_t N, unsigned flags,
                       buddy_hip_stream stream);

/* The same product over a device-side tile layout, for f32 matrices that stay
 * resident (the model path's f32 q|k|v weights): 32-row x 8-column tiles of
 * 1 KiB, zero padded, T[((n/8)*ceil(K/32) + k/32)*256 + (k%32)*8 + n%8] =
 * B[k,n] with B dense row-major.  It plays the part that the panel packing of
 * MatMulVectorizationDecodePacked.cpp:207-248 plays on the CPU (each worker
 * streams one contiguous run), sized for wavefront loads.  With norm_w the
 * RMSNorm of examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:38-58 is
 * applied to x on the way: y = bias + (norm_w (.) x * rsqrt(mean(x^2) + eps)) . B.
 * tiles: buddy_hip_f32_tiles_bytes(K, N) bytes, 16-byte aligned. */
size_t buddy_hip_f32_tiles_bytes(int64_t K, int64_t N);
int buddy_hip_tile_f32(const float *B, int64_t K, int64_t N, float *tiles,
                       buddy_hip_stream stream);
int buddy_hip_gemv_f32_tiles(const float *x, const float *tiles, const float *bias,
                             const float *norm_w, float norm_eps, float *y, int64_t K,
                             int64_t N, unsigned flags, buddy_hip_stream stream);

/* ---- the reference's f32 panel packing -------------------------------------
 * pack_decode_matmul_weights (frontend/Python/graph/transform/
 * pack_decode_weights.py:94-108): flat[nt*K*V + k*V + v] = B[k, nt*V + v]; same
 * bytes, same shape; N % V != 0 is refused (:95-99).  The GEMV reads that
 * order directly (MatMulVectorizationDecodePacked.cpp:207-248, V = 32):
 * y (+)= x[K] . B[K,N]; without BUDDY_HIP_GEMV_ACCUMULATE y need not be
 * initialised (the zero-init case of :209-222). */
int buddy_hip_pack_panels_f32(const float *B, int64_t K, int64_t N, int V,
                              float *packed, buddy_hip_stream stream);
int buddy_hip_unpack_panels_f32(const float *packed, int64_t K, int64_t N, int V,
                                float *B, buddy_hip_stream stream);
int buddy_hip_gemv_f32_panels(const float *x, const float *packed, float *y,
                              int64_t K, int64_t N, unsigned flags,
                              buddy_hip_stream stream);

/* ---- w8a8: int8 activations x int8 weights, int32 partial sums -------------
 * quantized_matmul_op (frontend/Python/ops/linalg.py:12728-12847): per-tensor
 * dynamic activation scale s_a = max(absmax(A)/127, 1e-10), A_q = clamp(rint(
 * A/s_a)), acc = A_q . W in int32 (exact), C = f32(acc) * (s_a * wscale[n]).
 * `packed` is the wave-tile copy of W; acc_out (int32 [M,N], dense) may be
 * NULL.  Up to 16 rows run as a GEMV; more rows run on the int8 matrix cores
 * (the i8 x i8 -> i32 branch of the BLIS kernel,
 * midend/lib/Conversion/MatMulOptimization/MatMulBlisVectorization.cpp:668-724)
 * and need K <= 131072.  A and C are dense ([M,K], [M,N]).
 * workspace: buddy_hip_w8a8_workspace_bytes, 16-byte aligned. */
size_t buddy_hip_w8a8_workspace_bytes(int64_t M, int64_t K);
int buddy_hip_w8a8_matmul(const float *A, const int8_t *packed, const float *wscale,
                          float *C, int32_t *acc_out, int64_t M, int64_t K,
                          int64_t N, void *workspace, size_t workspace_bytes,
                          buddy_hip_stream stream);

/* ---- the reference's w8a32 weight package ---------------------------------
 * Builds a session from the two flat blobs the reference's importer writes for
 * the w8a32 variant (arg0-w8a32-f32.data, arg0-w8a32-i8.data;
 * tools/buddy-codegen/gen_config.py:55-58).  Parameter order inside the blobs
 * (argument list of examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:4,
 * split by dtype, scalers appended in weight order --
 * frontend/Python/graph/transform/quantization/quantize.py:561-590):
 *   f32: embed[V,H], inv_freq[D/2], per layer { ln1[H], q_bias, q_w[H,QN],
 *        k_bias, k_w[H,KVN], v_bias, v_w[H,KVN], ln2[H] }, ln_f[H],
 *        per layer { s_o[H], s_gate[I], s_up[I], s_down[H] }, s_lm[V]
 *   i8 : per layer { o_w[QN,H], gate[H,I], up[H,I], down[I,H] }, lm_head[H,V]
 * For the Qwen2-1.5B shape these counts equal the reference's F32ParamsSize =
 * 322338752 and I8ParamsSize = 1455489024
 * (examples/BuddyDeepSeekR1/buddy-deepseek-r1-w8a32-main.cpp:32-33).
 * Blobs may be host or device memory and are not referenced after the call. */
void buddy_hip_w8a32_blob_sizes(const buddy_hip_model_shape *shape, int64_t *n_f32,
                                int64_t *n_i8);
/* The same layout as a table, one entry per parameter in blob order: which
 * parameter, its layer (-1: none), which blob, its shape and its element
 * offset inside that blob (the running offsets of
 * frontend/Python/graph/graph.py:848-863,1001-1018).  The blob reader below
 * cuts the blobs by this table and nothing else.  Writes at most `capacity`
 * entries and returns how many the layout has (0: null shape).  Host only. */
enum { BUDDY_HIP_BLOB_F32 = 0, BUDDY_HIP_BLOB_I8 = 1 };
enum {
  BUDDY_HIP_PARAM_EMBED = 0, BUDDY_HIP_PARAM_INV_FREQ, BUDDY_HIP_PARAM_LN1,
  BUDDY_HIP_PARAM_Q_BIAS, BUDDY_HIP_PARAM_Q_W, BUDDY_HIP_PARAM_K_BIAS,
  BUDDY_HIP_PARAM_K_W, BUDDY_HIP_PARAM_V_BIAS, BUDDY_HIP_PARAM_V_W,
  BUDDY_HIP_PARAM_O_W, BUDDY_HIP_PARAM_LN2, BUDDY_HIP_PARAM_GATE_W,
  BUDDY_HIP_PARAM_UP_W, BUDDY_HIP_PARAM_DOWN_W, BUDDY_HIP_PARAM_LN_F,
  BUDDY_HIP_PARAM_LM_HEAD_W, BUDDY_HIP_PARAM_O_SCALE, BUDDY_HIP_PARAM_GATE_SCALE,
  BUDDY_HIP_PARAM_UP_SCALE, BUDDY_HIP_PARAM_DOWN_SCALE, BUDDY_HIP_PARAM_LM_HEAD_SCALE
};
typedef struct buddy_hip_blob_entry {
  int32_t param;    /* BUDDY_HIP_PARAM_* */
  int32_t layer;    /* 0.., or -1 */
  int32_t dtype;    /* BUDDY_HIP_BLOB_F32 / BUDDY_HIP_BLOB_I8 */
  int32_t reserved;
  int64_t rows, cols; /* [rows, cols]; vectors have rows = 1 */
  int64_t offset;   /* elements from the start of its blob */
  int64_t count;    /* rows * cols */
} buddy_hip_blob_entry;
int64_t buddy_hip_w8a32_blob_layout(const buddy_hip_model_shape *shape,
                                    buddy_hip_blob_entry *entries, int64_t capacity);
buddy_hip_session *buddy_hip_session_create_from_w8a32_blobs(
    const buddy_hip_model_shape *shape, const float *f32_params, int64_t n_f32,
    const int8_t *i8_params, int64_t n_i8);

/* ---- model-level memref entry points ---------------------------------------
 * The two symbols the generated ModelSession resolves with dlsym
 * (tools/buddy-codegen/gen_session.py:1127-1143) with the argument lists of
 * PrefillFn / DecodeFn (gen_session.py:974-1007) for the 28-layer
 * DeepSeek-R1-Distill-Qwen-1.5B w8a32 package: result block, f32 blob, int8
 * blob, then tokens [1,max_len] (prefill) or token [1,1], cache_position [1],
 * kv0, kv1 and 27 x (position copy, k, v) (decode).  `result` is the
 * PrefillABI / DecodeABI block (gen_session.py:908-932).  Decode results alias
 * the caller's KV and position buffers and hand over a malloc'd [1,1,vocab]
 * logits buffer; prefill hands over malloc'd KV tensors and [1,max_len,vocab]
 * logits.  The device session is built on the first call and reused while the
 * blob addresses stay the same.  The caller's KV tensors and the device cache
 * are kept equal: the cache is uploaded from the caller's tensors on the first
 * decode that no prefill preceded, and every decode writes the row it produced
 * through to the caller's tensors, as the compiled model does.  A caller may
 * therefore edit its tensors between calls the way the generated
 * ModelSession::handleKVCacheOverflow does (gen_session.py:1471-1511: shift,
 * re-rotate, lower the position): a decode whose cache_position is not the one
 * that follows the previous call reloads the device cache from the caller's
 * tensors.  buddy_hip_forward_invalidate_kv() forces that reload.
 * The hand-written program for the same model
 * (examples/BuddyDeepSeekR1/buddy-deepseek-r1-w8a32-main.cpp:163-249) reads its
 * decode results in another order -- position, kv0, kv1, the 27 position copies
 * together, kv2..kv55, logits -- and frees every member at exit; with
 * BUDDY_HIP_DECODE_RESULT_LAYOUT=grouped in the environment the block is written
 * that way and the position comes back in a buffer of its own.  Arguments may
 * be members of the result block itself (that program passes them so). */
void _mlir_ciface_forward_prefill(void *result, buddy_memref_f32_1d *f32_params,
                                  buddy_memref_i8_1d *i8_params,
                                  buddy_memref_i64_2d *tokens);
#define BUDDY_HIP_KV_(n) , buddy_memref_f32_4d *k##n, buddy_memref_f32_4d *v##n
#define BUDDY_HIP_DKV_(n) , buddy_memref_i64_1d *d##n BUDDY_HIP_KV_(n)
void _mlir_ciface_forward_decode(
    void *result, buddy_memref_f32_1d *f32_params, buddy_memref_i8_1d *i8_params,
    buddy_memref_i64_2d *token, buddy_memref_i64_1d *cache_position BUDDY_HIP_KV_(0)
    BUDDY_HIP_DKV_(1) BUDDY_HIP_DKV_(2) BUDDY_HIP_DKV_(3) BUDDY_HIP_DKV_(4)
    BUDDY_HIP_DKV_(5) BUDDY_HIP_DKV_(6) BUDDY_HIP_DKV_(7) BUDDY_HIP_DKV_(8)
    BUDDY_HIP_DKV_(9) BUDDY_HIP_DKV_(10) BUDDY_HIP_DKV_(11) BUDDY_HIP_DKV_(12)
    BUDDY_HIP_DKV_(13) BUDDY_HIP_DKV_(14) BUDDY_HIP_DKV_(15) BUDDY_HIP_DKV_(16)
    BUDDY_HIP_DKV_(17) BUDDY_HIP_DKV_(18) BUDDY_HIP_DKV_(19) BUDDY_HIP_DKV_(20)
    BUDDY_HIP_DKV_(21) BUDDY_HIP_DKV_(22) BUDDY_HIP_DKV_(23) BUDDY_HIP_DKV_(24)
    BUDDY_HIP_DKV_(25) BUDDY_HIP_DKV_(26) BUDDY_HIP_DKV_(27));
void buddy_hip_forward_reset(void);         /* drops the cached device session */
void buddy_hip_forward_invalidate_kv(void); /* next decode re-uploads the KV cache */
/* discardKVCache + adjustKeyCacheRope on the device-resident cache of the
 * session behind _mlir_ciface_forward_*: what a decode loop may call instead of
 * editing its host tensors (TextGeneration.cpp:231-237); it saves the reload.
 * From then on the device cache is the only complete copy: the caller's tensors
 * keep receiving the new rows but are not shifted, and are never reloaded,
 * whatever position later decode calls carry (a rewind, a repeated position),
 * until buddy_hip_forward_invalidate_kv(), buddy_hip_forward_reset() or a
 * prefill. */
int buddy_hip_forward_discard_kv(int keep, int discard, int count);

/* ---- operator-level memref entry points --------------------------------
 * result = A * B, f32.  Same symbol and contract as
 * runtime/external_kernels/matmul/MatmulTorq.cpp:116-166: `result` is an
 * uninitialised descriptor; the callee malloc()s M*N floats and fills it;
 * strided inputs are honoured. */
void _mlir_ciface_buddy_matmul_f32(buddy_memref_f32_2d *result,
                                   buddy_memref_f32_2d *A,
                                   buddy_memref_f32_2d *B);
/* result = A * (sitofp(W) (.) scale), W int8 [K,N], scale f32 [1,N] or [N,1]
 * viewed as N values.  New symbol in the same convention (the reference has no
 * int8 external kernel: runtime/external_kernels/CMakeLists.txt:5-9); it
 * stands for the sitofp -> mulf -> linalg.matmul chain that
 * DequantMatMulVectorizationDecode.cpp:93-189 matches.  The packed device copy
 * of W is cached by (W pointer, scale pointer, K, N) because weights are
 * immutable after loadWeights (tools/buddy-codegen/gen_session.py:1301-1331).
 * Every call compares a fingerprint of the operands as they are now (64
 * leading bytes of four rows of W, the first and last 16 scales, the shape)
 * with the one taken when the copy was made: a buffer that was freed and
 * reused at the same address with other contents is packed again.  The cache
 * holds at most a byte limit (16 GiB, or BUDDY_HIP_WEIGHT_CACHE_BYTES in the
 * environment); the least recently used copies are freed first.  The
 * reference's own external kernel caches nothing
 * (runtime/external_kernels/matmul/MatmulTorq.cpp:116-166). */
void _mlir_ciface_buddy_dequant_matmul_i8_f32(buddy_memref_f32_2d *result,
                                              buddy_memref_f32_2d *A,
                                              buddy_memref_i8_2d *W,
                                              buddy_memref_f32_2d *scale);
/* C += A * (sitofp(W) (.) scale) in place: linalg.matmul's accumulate-into-
 * outs semantics (DequantMatMulVectorizationDecode.cpp:313-320). */
void _mlir_ciface_buddy_dequant_matmul_i8_f32_acc(buddy_memref_f32_2d *C,
                                                  buddy_memref_f32_2d *A,
                                                  buddy_memref_i8_2d *W,
                                                  buddy_memref_f32_2d *scale);
/* Drops every cached device copy made by the entry points above. */
void buddy_hip_clear_weight_cache(void);
/* The byte limit of that cache (entries beyond it are freed at once, least
 * recently used first) and its counters.  No counterpart in the reference. */
typedef struct buddy_hip_weight_cache_info {
  int64_t entries;     /* packed copies held */
  int64_t bytes;       /* device bytes they take */
  int64_t limit_bytes; /* the limit in force */
  int64_t uploads;     /* copies made since the library was loaded */
  int64_t evictions;   /* copies freed to stay under the limit */
} buddy_hip_weight_cache_info;
void buddy_hip_set_weight_cache_limit(size_t bytes);
void buddy_hip_weight_cache_stats(buddy_hip_weight_cache_info *info);

#ifdef __cplusplus
}
#endif
#endif /* BUDDY_HIP_H */
