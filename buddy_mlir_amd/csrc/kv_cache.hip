// kv_cache.hip -- KV-cache overflow handling on the device.
//
// Replaces, for caches that live in HBM,
//   kvcache::discardKVCache      runtime/include/buddy/runtime/llm/KVCacheManager.h:150-194
//   kvcache::adjustKeyCacheRope  same file :240-268 (applyRotaryDeltaToSlice :200-228)
// which the reference's decode loop calls when the cache is full
// (runtime/include/buddy/runtime/llm/TextGeneration.cpp:231-237): keep a prefix,
// drop `discard` tokens after it, move the tail forward, zero what is left, and
// rotate the moved keys back by `discard` positions so that their RoPE matches
// their new place.
//
// One launch does both for up to kMaxTensors cache tensors.  Row t of the tail
// takes its data from row t + discard, so the rows with the same t mod discard
// form a chain that must be walked in order, and different chains never touch
// the same row: a thread owns one chain of one rotation pair (d, d + dim/2) of
// one head of one tensor, reads row t + discard, then writes row t.  The move
// is in place and race free without a scratch copy.  cos/sin of the rotation are
// computed on the host with the C library, like the reference, and travel as
// kernel arguments; the device multiplies and adds without contraction, so the
// moved values are the reference's bit for bit.
#include "kv_cache.h"

#include <algorithm>
#include <cmath>

namespace bh {
namespace {

constexpr int kMaxTensors = 64;
constexpr int kMaxHalf = 128; // head_dim <= 256

struct DiscardArgs {
  float *tensor[kMaxTensors];
  unsigned long long rotate_mask; // bit i: tensor i holds keys
  int tensors, heads, max_len, dim, keep, discard, tail;
  float cosv[kMaxHalf], sinv[kMaxHalf];
};

__global__ void __launch_bounds__(256) kv_discard_kernel(DiscardArgs a) {
// the reference multiplies and adds separately: no fused multiply-add here
#pragma clang fp contract(off)
  const int half = a.dim / 2;
  const int chains = min(a.discard, a.tail + (a.max_len - a.keep - a.tail));
  const int per_head = chains * half, per_tensor = a.heads * per_head;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)a.tensors * per_tensor)
    return;
  const int tn = (int)(i / per_tensor), rem = (int)(i % per_tensor);
  const int h = rem / per_head, r = (rem % per_head) / half, d = rem % half;
  const bool rotate = (a.rotate_mask >> tn) & 1ull;
  const float c = a.cosv[d], s = a.sinv[d];
  float *base = a.tensor[tn] + (size_t)h * a.max_len * a.dim + d;
  float *dst = base + (size_t)a.keep * a.dim;
  const float *src = dst + (size_t)a.discard * a.dim;
  // chain r: rows r, r + discard, r + 2 discard, ... of the tail, in order
  for (int t = r; t < a.tail; t += a.discard) {
    const float v1 = src[(size_t)t * a.dim], v2 = src[(size_t)t * a.dim + half];
    float o1 = v1, o2 = v2;
    if (rotate) { // (v1 cos - v2 sin, v1 sin + v2 cos), KVCacheManager.h:218-222
      const float p1 = v1 * c, p2 = v2 * s, p3 = v1 * s, p4 = v2 * c;
      o1 = p1 - p2;
      o2 = p3 + p4;
    }
    dst[(size_t)t * a.dim] = o1;
    dst[(size_t)t * a.dim + half] = o2;
  }
  // rows keep + tail .. max_len - 1 are cleared (KVCacheManager.h:184-190); a
  // row there is the source of at most one row of the same chain, read above
  for (int t = a.keep + a.tail + (((r - a.tail) % a.discard) + a.discard) % a.discard;
       t < a.max_len; t += a.discard) {
    base[(size_t)t * a.dim] = 0.f;
    base[(size_t)t * a.dim + half] = 0.f;
  }
}

struct GatherArgs {
  const float *tensor[kMaxTensors];
  int tensors, heads, max_len, dim, row0, rows;
};

// dst[((tensor * heads + head) * rows + r) * dim + d] = cache row row0 + r
__global__ void __launch_bounds__(256)
kv_gather_rows_kernel(GatherArgs a, float *__restrict__ dst) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t per_tensor = (int64_t)a.heads * a.rows * a.dim;
  if (i >= a.tensors * per_tensor)
    return;
  const int tn = (int)(i / per_tensor);
  const int64_t rem = i % per_tensor;
  const int h = (int)(rem / ((int64_t)a.rows * a.dim));
  const int r = (int)(rem / a.dim % a.rows), d = (int)(rem % a.dim);
  dst[i] = a.tensor[tn][((size_t)h * a.max_len + a.row0 + r) * a.dim + d];
}

} // namespace

int launch_kv_gather_rows(const float *const *tensors, int num_tensors, int heads,
                          int max_len, int head_dim, int row0, int rows, float *dst,
                          hipStream_t stream) {
  BH_REQUIRE(tensors && dst && num_tensors > 0 && heads > 0 && head_dim > 0,
             "kv_gather_rows: bad argument");
  BH_REQUIRE(row0 >= 0 && rows > 0 && (int64_t)row0 + rows <= max_len,
             "kv_gather_rows: rows %d..%d outside the cache (max_len %d)", row0,
             row0 + rows - 1, max_len);
  for (int t0 = 0; t0 < num_tensors; t0 += kMaxTensors) {
    GatherArgs a;
    a.tensors = num_tensors - t0 < kMaxTensors ? num_tensors - t0 : kMaxTensors;
    for (int i = 0; i < kMaxTensors; ++i) {
      a.tensor[i] = i < a.tensors ? tensors[t0 + i] : nullptr;
      BH_REQUIRE(i >= a.tensors || a.tensor[i], "kv_gather_rows: tensor %d is null", t0 + i);
    }
    a.heads = heads;
    a.max_len = max_len;
    a.dim = head_dim;
    a.row0 = row0;
    a.rows = rows;
    const int64_t per_tensor = (int64_t)heads * rows * head_dim;
    hipLaunchKernelGGL(kv_gather_rows_kernel,
                       dim3((unsigned)ceil_div(a.tensors * per_tensor, 256)), dim3(256), 0,
                       stream, a, dst + (size_t)t0 * per_tensor);
    BH_CHECK_HIP(hipGetLastError());
  }
  return BUDDY_HIP_OK;
}

int launch_kv_discard(float *const *tensors, int num_tensors, int heads, int max_len,
                      int head_dim, int keep, int discard, int count,
                      const float *inv_freq_host, hipStream_t stream) {
  BH_REQUIRE(tensors && num_tensors > 0 && heads > 0 && max_len > 0 && head_dim > 0 &&
                 head_dim % 2 == 0 && head_dim / 2 <= kMaxHalf,
             "kv_discard: bad shape (tensors=%d heads=%d max_len=%d head_dim=%d)",
             num_tensors, heads, max_len, head_dim);
  // the reference's own refusals (KVCacheManager.h:154-167): the cache is left
  // untouched
  if (count < 0)
    count = 0;
  if (count > max_len)
    count = max_len;
  BH_REQUIRE(discard > 0 && keep >= 0 && keep < count,
             "kv_discard: invalid parameters (keep=%d discard=%d count=%d)", keep,
             discard, count);
  BH_REQUIRE(keep + discard < count,
             "kv_discard: keep + discard = %d >= current token count %d", keep + discard,
             count);
  for (int t0 = 0; t0 < num_tensors; t0 += kMaxTensors) {
    DiscardArgs a;
    a.tensors = num_tensors - t0 < kMaxTensors ? num_tensors - t0 : kMaxTensors;
    a.rotate_mask = 0;
    for (int i = 0; i < a.tensors; ++i) {
      BH_REQUIRE(tensors[t0 + i], "kv_discard: tensor %d is null", t0 + i);
      a.tensor[i] = tensors[t0 + i];
      // even indices are key caches (KVCacheManager.h:209)
      if (inv_freq_host && ((t0 + i) & 1) == 0)
        a.rotate_mask |= 1ull << i;
    }
    for (int i = a.tensors; i < kMaxTensors; ++i)
      a.tensor[i] = nullptr;
    a.heads = heads;
    a.max_len = max_len;
    a.dim = head_dim;
    a.keep = keep;
    a.discard = discard;
    a.tail = count - keep - discard;
    const float delta = -static_cast<float>(discard);
    for (int i = 0; i < kMaxHalf; ++i) {
      float c = 1.f, s = 0.f;
      if (inv_freq_host && i < head_dim / 2) {
        const float angle = inv_freq_host[i] * delta; // KVCacheManager.h:255-259
        c = std::cos(angle);
        s = std::sin(angle);
      }
      a.cosv[i] = c;
      a.sinv[i] = s;
    }
    const int chains = std::min(discard, max_len - keep);
    const int64_t threads = (int64_t)a.tensors * heads * chains * (head_dim / 2);
    hipLaunchKernelGGL(kv_discard_kernel, dim3((unsigned)ceil_div(threads, 256)),
                       dim3(256), 0, stream, a);
    BH_CHECK_HIP(hipGetLastError());
  }
  return BUDDY_HIP_OK;
}

} // namespace bh

extern "C" {

int buddy_hip_kv_discard(float *const *tensors, int num_tensors, int heads, int max_len,
                         int head_dim, int keep, int discard, int count,
                         const float *inv_freq, buddy_hip_stream stream) try {
  return bh::launch_kv_discard(tensors, num_tensors, heads, max_len, head_dim, keep,
                               discard, count, inv_freq, bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_kv_discard")
}
