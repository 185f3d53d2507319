// elementwise.h -- launchers of the small kernels around the matmuls.
#pragma once

#include "common.h"

namespace bh {

constexpr int kArgmaxParts = 256;

int launch_embedding(const float *table, const int *token, int64_t hidden,
                     int64_t vocab, float *out, hipStream_t stream);
int launch_rmsnorm(const float *x, const float *w, float *y, int rows, int n,
                   float eps, hipStream_t stream);
int launch_rope(float *x, const float *inv_freq, const int *pos, int n_heads,
                int head_dim, hipStream_t stream);
int launch_silu_mul(const float *g, const float *u, float *h, int64_t n,
                    hipStream_t stream);
size_t argmax_workspace_bytes();
// out_token <- first index of the maximum; optionally token_log[*step_ptr] too.
int launch_argmax(const float *x, int n, void *workspace, int *out_token,
                  int *token_log, int *step_ptr, hipStream_t stream);

} // namespace bh
