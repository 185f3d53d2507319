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

// First half of the argmax; *nparts_out candidates are left in the workspace.
int launch_argmax_partial(const float *x, int n, void *workspace, int *nparts_out,
                          hipStream_t stream);
// Tail of a decode step (nparts > 0: pick + log the token; advance: pos/step += 1)
// and head of the next one (x = embedding row of state[0], rope = [cos | sin] of
// state[1]).  With nparts = 0 and advance = false it only prepares a step.
// The candidates are (value, index) pairs in two arrays: the workspace of
// launch_argmax_partial (values, then indices kArgmaxParts further on) or the
// per-group maxima a GEMV left behind.
int launch_finish_step(const float *cand_v, const int *cand_i, int nparts, int *state,
                       int *token_log, const float *table, int64_t hidden, int64_t vocab,
                       float *x, const float *inv_freq, int head_dim, float *rope,
                       bool advance, int token_log_cap, hipStream_t stream);

} // namespace bh
