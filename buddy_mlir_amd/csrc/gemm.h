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
  // 2 or 3: carry the activations as that many int8 digit planes (fixed point
  // relative to each row's maximum) and multiply on the int8 matrix cores;
  // 0: bf16 terms as above
  int digits = 0;
  // digits only: W holds two matrices of N / 2 channels one behind the other
  // (scales likewise), and C [M, N / 2] = SiLU(A . first) * (A . second)
  bool silu_pair = false;
  // digits only: the finished rows of C also leave as RMSNorm(row) * then_norm_w
  // in digit planes (then_norm_staged: layout of gemm_staging_layout(M, N)), the
  // input of the matmul that follows -- written by the kernel that adds the K
  // slices where there is one, by a launch of its own otherwise
  const float *then_norm_w = nullptr;
  float then_norm_eps = 0.f;
  void *then_norm_staged = nullptr;
  // A (same pointer, shape, terms, contents) was the input of the previous
  // matmul on this stream: its bf16 copy is still staged, skip the conversion
  bool reuse_staged_a = false;
  // Caller-provided staging of A (written by one of the producers below for
  // exactly this M, K and terms / digits): no conversion, A itself is not read.
  const void *staged = nullptr;
};

// Layout of a bf16 staging buffer: [terms][rows_padded][cols_padded] bf16, term t
// holding the bf16 rounding of what the terms before it left over; valid rows
// are zero beyond K.
struct GemmStagingLayout {
  int rows_padded = 0, cols_padded = 0;
  size_t bytes(int terms) const {
    return sizeof(unsigned short) * (size_t)terms * rows_padded * cols_padded;
  }
  // digit planes: [digits][rows_padded][cols_padded] int8, then the row steps
  // (f32 [rows_padded])
  size_t bytes_digits(int digits) const {
    return (size_t)digits * rows_padded * cols_padded + sizeof(float) * (size_t)rows_padded;
  }
};
GemmStagingLayout gemm_staging_layout(int64_t M, int64_t K);
// Producers that write their result straight into a staging buffer:
//   RMSNorm rows: y = w * (x * rsqrt(mean(x^2) + eps))
//   SiLU(g) * u   (g and u rows `ld` floats apart)
int launch_rmsnorm_to_staging(const float *x, const float *w, int rows, int n, float eps,
                              int terms, unsigned short *staged, hipStream_t stream);
int launch_silu_mul_to_staging(const float *g, const float *u, int64_t ld, int rows, int n, int terms,
                               unsigned short *staged, hipStream_t stream);
// the same producers for digit planes, and the plain conversion of A
int launch_rmsnorm_to_digits(const float *x, int64_t ldx, const float *w, int rows, int n,
                             float eps, int digits, void *staged, hipStream_t stream);
int launch_silu_mul_to_digits(const float *g, const float *u, int64_t ld, int rows, int n, int digits,
                              void *staged, hipStream_t stream);
int launch_activations_to_digits(const float *A, int64_t lda, int64_t M, int64_t K,
                                 int digits, void *staged, hipStream_t stream);
// the matmul over digit planes (called by launch_gemm_w8 when digits != 0)
int launch_gemm_w8_digits(const GemmW8Args &a, const void *planes, hipStream_t stream);

int launch_gemm_w8(const GemmW8Args &a, hipStream_t stream);

// w8a8 for more than 16 rows: one int8 plane of activations (layout of
// gemm_staging_layout(M, K) with one digit, every row step = the activation
// scale) times the packed int8 weights; C = f32(sum) * (step * wscale[n]) and,
// when `sums` is not null, the int32 sums themselves (dense [M, N]).
int launch_gemm_w8a8_plane(const void *plane, const int8_t *W, const float *wscale, float *C,
                           int32_t *sums, int64_t M, int64_t K, int64_t N,
                           hipStream_t stream);

// split-K workspace of the int8 matmul (dropped together with the staging)
void release_gemm_i8_workspace(hipStream_t stream);

// The matmul keeps a bf16 copy of its activations in a grow-only device buffer
// per stream; a stream's owner drops it before destroying the stream.
void release_gemm_staging(hipStream_t stream);

} // namespace bh
