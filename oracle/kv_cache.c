/* kv_cache.c -- CPU restatement of the reference's KV-cache overflow handling.
 * TEST INFRASTRUCTURE: only tests, the smoke check and the CPU baseline of the
 * benchmark may use it.
 *
 * Follows runtime/include/buddy/runtime/llm/KVCacheManager.h:
 *   discardKVCache       :150-194  (keep a prefix, drop `discard` tokens after
 *                                    it, move the tail forward, zero the rest)
 *   adjustKeyCacheRope   :240-268  (rotate the moved keys back by `discard`
 *                                    positions; applyRotaryDeltaToSlice :200-228)
 * for one [heads, max_len, dim] f32 tensor (the reference loops over the 2 x
 * layers tensors; even indices are keys).
 */
#include "oracle.h"

#include <math.h>
#include <string.h>

/* KVCacheManager.h:150-194.  Returns 0, or -1 where the reference prints an
 * error and leaves the cache untouched. */
int oracle_kv_discard(float *cache, int64_t heads, int64_t max_len, int64_t dim,
                      int64_t keep, int64_t discard, int64_t count) {
  if (count < 0)
    count = 0;
  if (count > max_len)
    count = max_len;
  if (discard <= 0 || keep < 0 || keep >= count)
    return -1;
  const int64_t src = keep + discard;
  if (src >= count)
    return -1;
  const int64_t tail = count - src;
  for (int64_t h = 0; h < heads; ++h) {
    float *base = cache + h * max_len * dim;
    memmove(base + keep * dim, base + src * dim, (size_t)(tail * dim) * sizeof(float));
    const int64_t clear = max_len - (keep + tail);
    if (clear > 0)
      memset(base + (keep + tail) * dim, 0, (size_t)(clear * dim) * sizeof(float));
  }
  return 0;
}

/* KVCacheManager.h:240-268 with :200-228: angle_i = inv_freq[i] * (-discard);
 * (v1, v2) = (x[i], x[i + half]) -> (v1 cos - v2 sin, v1 sin + v2 cos) for the
 * `count - keep - discard` rows that start at `keep`.  `count` is the token
 * count BEFORE the discard, the data is the already moved one. */
void oracle_kv_adjust_rope(float *kcache, int64_t heads, int64_t max_len, int64_t dim,
                           int64_t keep, int64_t discard, int64_t count,
                           const float *inv_freq) {
  if (discard <= 0)
    return;
  const int64_t src = keep + discard;
  if (src >= count)
    return;
  const int64_t tokens = count - src, half = dim / 2;
  const float delta = -(float)discard;
  for (int64_t h = 0; h < heads; ++h)
    for (int64_t t = 0; t < tokens; ++t) {
      float *row = kcache + (h * max_len + keep + t) * dim;
      for (int64_t i = 0; i < half; ++i) {
        const float angle = inv_freq[i] * delta;
        const float c = cosf(angle), s = sinf(angle);
        const float v1 = row[i], v2 = row[i + half];
        const float a = v1 * c, b = v2 * s, d = v1 * s, e = v2 * c;
        row[i] = a - b;
        row[i + half] = d + e;
      }
    }
}
