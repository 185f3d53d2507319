// gemm.h -- launch description of the prefill matmul.
#pragma once

#include "common.h"

namespace bh {

struct GemmW8Args {
  const float *A = nullptr; // [M, K], row stride lda
  int64_t lda = 0;
  const int8_t *W = nullptr; // wave-tile packed [K, N]
  const float *scale = nullptr; // [N]
  const float *bias = nullptr;  // [N] or null (not with accumulate)
  float *C = nullptr;           // [M, N], row stride ldc
  int64_t ldc = 0;
  int64_t M = 0, K = 0, N = 0;
  bool accumulate = false;
  int terms = 1; // bf16 terms per activation: 1 = cast to bf16, 3 = all f32 bits
  // A (same pointer, shape, terms, contents) was the input of the previous
  // matmul on this stream: its bf16 copy is still staged, skip the conversion
  bool reuse_staged_a = false;
  // Caller-provided bf16 staging of A (written by one of the producers below for
  // exactly this M, K and terms): no conversion, A itself is not read.
  const unsigned short *staged = nullptr;
};

// Layout of a bf16 staging buffer: [terms][rows_padded][cols_padded] bf16, term t
// holding the bf16 rounding of what the terms before it left over; valid rows
// are zero beyond K.
struct GemmStagingLayout {
  int rows_padded = 0, cols_padded = 0;
  size_t bytes(int terms) const {
    return sizeof(unsigned short) * (size_t)terms * rows_padded * cols_padded;
  }
};
GemmStagingLayout gemm_staging_layout(int64_t M, int64_t K);
// Producers that write their result straight into a staging buffer:
//   RMSNorm rows: y = w * (x * rsqrt(mean(x^2) + eps))
//   SiLU(g) * u
int launch_rmsnorm_to_staging(const float *x, const float *w, int rows, int n, float eps,
                              int terms, unsigned short *staged, hipStream_t stream);
int launch_silu_mul_to_staging(const float *g, const float *u, int rows, int n, int terms,
                               unsigned short *staged, hipStream_t stream);

int launch_gemm_w8(const GemmW8Args &a, hipStream_t stream);

// The matmul keeps a bf16 copy of its activations in a grow-only device buffer
// per stream; a stream's owner drops it before destroying the stream.
void release_gemm_staging(hipStream_t stream);

} // namespace bh
