// gemv_w8a32.h -- launch description of the int8 dequant GEMV kernel family.
#pragma once

#include "common.h"

namespace bh {

// What happens to the raw sums before they are stored.
enum GemvEpilogue : int {
  kEpiStore = 0,  // C = acc*scale (+ bias)
  kEpiAccum = 1,  // C = C + acc*scale        (linalg.matmul accumulate / residual)
  kEpiSiluMul = 2 // C = silu(acc0*s0) * (acc1*s1), two weight matrices
};

struct GemvArgs {
  const float *A = nullptr;   // [M, K], row stride lda
  int64_t lda = 0;
  const int8_t *W0 = nullptr; // wave-tile packed [Kp, Np]
  const int8_t *W1 = nullptr; // second matrix for kEpiSiluMul
  const float *s0 = nullptr;  // [N]
  const float *s1 = nullptr;
  const float *bias = nullptr; // [N] or null; y = bias + acc*scale
  float *C = nullptr;          // [M, N], row stride ldc
  int64_t ldc = 0;
  // Optional RMSNorm applied to A while it is staged:
  //   x' = norm_w[k] * (x[k] * rsqrt(sum(x^2) * inv_k + eps))
  const float *norm_w = nullptr;
  float norm_eps = 0.f;
  float norm_inv_k = 0.f;
  // Alternative input: A = attention output folded on the fly from flash-
  // decoding partials (acc [heads, nchunks, head_dim], ml [heads, nchunks, 2]),
  // chunks 0 .. *pos_ptr / attn_chunk; A is ignored then.
  const float *attn_acc = nullptr, *attn_ml = nullptr;
  const int *pos_ptr = nullptr;
  int attn_nchunks = 0, attn_chunk = 0, head_dim = 0;
  int attn_used = 0; // chunks to fold (the first ones); 0: all attn_nchunks
  int tile_n = 16; // channels per packed tile: 16 (default), 8 or 4
  // One row with the STORE epilogue, optional: the first maximum of every
  // channel group's 16 results, (value, index) at [group] of these two arrays
  // (NaNs are not candidates; a group without one holds (-inf, INT_MAX)), so
  // that a greedy pick need not read the row again.  *argmax_groups receives
  // the number of groups written, or 0 when the launch's kernel does not emit
  // them (the caller then scans the row itself).
  float *argmax_v = nullptr;
  int *argmax_i = nullptr;
  int *argmax_groups = nullptr;
  int M = 1;
  int64_t K = 0, N = 0;
  int epilogue = kEpiStore;
};

int launch_gemv(const GemvArgs &a, hipStream_t stream);
// Matrix-core variants for 5..16 rows (chosen by launch_gemv): int8 matrix
// instructions over fixed-point activations (the default), or bf16 ones over
// three bf16 terms of every activation (every f32 bit; BUDDY_HIP_GEMV_BATCH=bf16).
int launch_gemv_i8(const GemvArgs &a, hipStream_t stream);
int launch_gemv_mfma(const GemvArgs &a, hipStream_t stream);

} // namespace bh
