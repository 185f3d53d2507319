/*
 * ref_llm.cpp -- exposes two header-only pieces of the reference's own runtime
 * through a C interface, compiled from the headers where they lie in the
 * reference tree (nothing of them is copied here):
 *   runtime/include/buddy/runtime/llm/Sampler.h        buddy::Sampler
 *   runtime/include/buddy/runtime/llm/KVCacheManager.h buddy::kvcache::discardKVCache,
 *                                                      adjustKeyCacheRope,
 *                                                      buildInverseRopeFreqs
 *   frontend/Interfaces/buddy/Core/Container.h         MemRef<T, N>, whose object
 *                                                      layout is the descriptor the
 *                                                      _mlir_ciface_* symbols receive
 * All need the C++ standard library only.  The result, oracle/_ref/libref_llm.so,
 * is what the restated sampler and KV-cache functions of the oracle are checked
 * against.
 *
 * TEST INFRASTRUCTURE ONLY, like the rest of this directory.
 */
#include <cstdint>
#include <vector>

#include <cstring>

#include "buddy/Core/Container.h"
#include "buddy/runtime/llm/KVCacheManager.h"
#include "buddy/runtime/llm/Sampler.h"

namespace {
// Builds a MemRef<T, N> over `data` and copies the object's own bytes out: what
// a callee that is handed `&memref` sees.  Returns sizeof(MemRef<T, N>).
template <typename T, size_t N>
int memref_bytes(const T *data, const int64_t *sizes, int64_t offset, void *out, int cap) {
  intptr_t sz[N];
  for (size_t i = 0; i < N; ++i)
    sz[i] = (intptr_t)sizes[i];
  MemRef<T, N> m(data, sz, (intptr_t)offset);
  if ((int)sizeof(m) <= cap)
    std::memcpy(out, static_cast<const void *>(&m), sizeof(m));
  return (int)sizeof(m);
}
} // namespace

extern "C" {

// kind: 0 = float, 1 = int8, 2 = int64; the object's bytes of a MemRef built over
// `data` with the given sizes and offset
int ref_memref_object(int kind, int rank, const void *data, const int64_t *sizes, int64_t offset,
                      void *out, int cap) {
  switch (kind * 10 + rank) {
  case 1: return memref_bytes<float, 1>((const float *)data, sizes, offset, out, cap);
  case 2: return memref_bytes<float, 2>((const float *)data, sizes, offset, out, cap);
  case 3: return memref_bytes<float, 3>((const float *)data, sizes, offset, out, cap);
  case 4: return memref_bytes<float, 4>((const float *)data, sizes, offset, out, cap);
  case 11: return memref_bytes<int8_t, 1>((const int8_t *)data, sizes, offset, out, cap);
  case 12: return memref_bytes<int8_t, 2>((const int8_t *)data, sizes, offset, out, cap);
  case 21: return memref_bytes<long long, 1>((const long long *)data, sizes, offset, out, cap);
  case 22: return memref_bytes<long long, 2>((const long long *)data, sizes, offset, out, cap);
  }
  return -1;
}

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
