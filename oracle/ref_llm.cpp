/*
 * ref_llm.cpp -- exposes two header-only pieces of the reference's own runtime
 * through a C interface, compiled from the headers where they lie in the
 * reference tree (nothing of them is copied here):
 *   runtime/include/buddy/runtime/llm/Sampler.h        buddy::Sampler
 *   runtime/include/buddy/runtime/llm/KVCacheManager.h buddy::kvcache::discardKVCache,
 *                                                      adjustKeyCacheRope,
 *                                                      buildInverseRopeFreqs
 * Both need the C++ standard library only.  The result, oracle/_ref/libref_llm.so,
 * is what the restated sampler and KV-cache functions of the oracle are checked
 * against.
 *
 * TEST INFRASTRUCTURE ONLY, like the rest of this directory.
 */
#include <cstdint>
#include <vector>

#include "buddy/runtime/llm/KVCacheManager.h"
#include "buddy/runtime/llm/Sampler.h"

extern "C" {

void *ref_sampler_create(float temperature, int top_k, float top_p, float min_p,
                         float repeat_penalty, int repeat_last_n, uint64_t seed) {
  buddy::SamplerConfig c;
  c.temperature = temperature;
  c.topK = top_k;
  c.topP = top_p;
  c.minP = min_p;
  c.repeatPenalty = repeat_penalty;
  c.repeatLastN = repeat_last_n;
  c.seed = seed;
  return new buddy::Sampler(c);
}

void ref_sampler_destroy(void *s) { delete static_cast<buddy::Sampler *>(s); }

int ref_sampler_sample(void *s, const float *logits, int64_t vocab, const int *recent,
                       int64_t n_recent) {
  const std::vector<int> rec(recent, recent + n_recent);
  return static_cast<buddy::Sampler *>(s)->sample(logits, (size_t)vocab, rec);
}

void ref_kv_discard(float **tensors, int num_tensors, int heads, int max_len, int head_dim,
                    int keep, int discard, int count) {
  buddy::kvcache::discardKVCache<float>(tensors, num_tensors, heads, max_len, head_dim, keep,
                                        discard, count);
}

void ref_kv_adjust_rope(float **tensors, int num_tensors, int heads, int max_len, int head_dim,
                        int keep, int discard, int count, const float *inv_freq) {
  const std::vector<float> f(inv_freq, inv_freq + head_dim / 2);
  buddy::kvcache::adjustKeyCacheRope<float>(tensors, num_tensors, heads, max_len, head_dim, keep,
                                            discard, count, f);
}

void ref_inverse_rope_freqs(float theta, int head_dim, float *out) {
  const std::vector<float> f = buddy::kvcache::buildInverseRopeFreqs(theta, head_dim);
  for (size_t i = 0; i < f.size(); ++i)
    out[i] = f[i];
}

int ref_inverse_rope_freqs_count(float theta, int head_dim) {
  return (int)buddy::kvcache::buildInverseRopeFreqs(theta, head_dim).size();
}
}
