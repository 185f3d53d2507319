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
};

int launch_gemm_w8(const GemmW8Args &a, hipStream_t stream);

// The matmul keeps a bf16 copy of its activations in a grow-only device buffer
// per stream; a stream's owner drops it before destroying the stream.
void release_gemm_staging(hipStream_t stream);

} // namespace bh
