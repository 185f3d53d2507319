// kv_cache.h -- KV-cache overflow handling (discard + key re-rotation).
#pragma once

#include "common.h"

namespace bh {

// tensors: host array of device pointers, each [heads, max_len, head_dim] f32,
// even index = keys, odd = values.  inv_freq_host: host pointer to head_dim/2
// inverse RoPE frequencies, or null to move without re-rotating the keys.
int launch_kv_discard(float *const *tensors, int num_tensors, int heads, int max_len,
                      int head_dim, int keep, int discard, int count,
                      const float *inv_freq_host, hipStream_t stream);

// Rows row0 .. row0 + rows - 1 of every cache, packed as
// dst[tensor][head][row][head_dim] (device memory): what a caller that mirrors
// the caches on the host needs after a decode step.
int launch_kv_gather_rows(const float *const *tensors, int num_tensors, int heads,
                          int max_len, int head_dim, int row0, int rows, float *dst,
                          hipStream_t stream);

} // namespace bh
