/*
 * sampler.cpp -- CPU restatement of the reference's token sampler
 * (runtime/include/buddy/runtime/llm/Sampler.h:62-206): repetition penalty over
 * the last repeatLastN tokens (:112-129), temperature (:131-136), a full sort
 * of the vocabulary by logit, top-K, softmax over the kept candidates in f32,
 * min-P, top-P, renormalisation (:139-197) and a draw from
 * std::discrete_distribution driven by std::mt19937 (:199-202).
 *
 * TEST INFRASTRUCTURE ONLY (see oracle.h).  C++ because the draw is defined by
 * the standard library's own generator and distribution, as in the reference.
 */
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <random>
#include <utility>
#include <vector>

namespace {

struct OracleSampler {
  float temperature, top_p, min_p, repeat_penalty;
  int top_k, repeat_last_n;
  std::mt19937 rng;
};

int greedy(const float *logits, int64_t n) { // Sampler.h:101-104: first maximum
  return (int)std::distance(logits, std::max_element(logits, logits + n));
}

} // namespace

extern "C" {

void *oracle_sampler_create(float temperature, int top_k, float top_p, float min_p,
                            float repeat_penalty, int repeat_last_n, uint64_t seed) {
  OracleSampler *s = new OracleSampler{temperature, top_p, min_p, repeat_penalty, top_k,
                                       repeat_last_n, std::mt19937()};
  if (seed != 0) // Sampler.h:51-56 (seed 0 = random device there; the tests always seed)
    s->rng.seed(seed);
  return s;
}

void oracle_sampler_destroy(void *p) { delete static_cast<OracleSampler *>(p); }

/* Returns the chosen token; n_kept (may be NULL) receives the size of the final
 * candidate set (0 on the greedy paths). */
int oracle_sampler_sample(void *p, const float *logits, int64_t vocab, const int *recent,
                          int64_t n_recent, int64_t *n_kept) {
  OracleSampler &s = *static_cast<OracleSampler *>(p);
  if (n_kept)
    *n_kept = 0;
  const bool penalty = s.repeat_penalty != 1.0f && n_recent > 0;
  if (s.temperature == 0.0f && !penalty)
    return greedy(logits, vocab);
  std::vector<float> work(logits, logits + vocab);
  if (penalty) { // :112-129, once per occurrence, in window order
    int64_t start = n_recent - s.repeat_last_n;
    if (start < 0)
      start = 0;
    for (int64_t i = start; i < n_recent; ++i) {
      const int t = recent[i];
      if (t < 0 || t >= (int)vocab)
        continue;
      if (work[t] > 0.0f)
        work[t] /= s.repeat_penalty;
      else
        work[t] *= s.repeat_penalty;
    }
  }
  if (s.temperature == 0.0f)
    return greedy(work.data(), vocab);
  const float inv_temp = 1.0f / s.temperature; // :131-136
  for (float &v : work)
    v *= inv_temp;
  // :139-203
  std::vector<std::pair<int, float>> cand((size_t)vocab);
  for (int64_t i = 0; i < vocab; ++i)
    cand[(size_t)i] = {(int)i, work[(size_t)i]};
  std::sort(cand.begin(), cand.end(),
            [](const std::pair<int, float> &a, const std::pair<int, float> &b) {
              return a.second > b.second;
            });
  size_t limit = cand.size();
  if (s.top_k > 0 && (size_t)s.top_k < limit)
    limit = (size_t)s.top_k;
  const float max_logit = cand[0].second;
  std::vector<float> probs(limit);
  float sum_exp = 0.0f;
  for (size_t i = 0; i < limit; ++i) {
    probs[i] = std::exp(cand[i].second - max_logit);
    sum_exp += probs[i];
  }
  for (size_t i = 0; i < limit; ++i)
    probs[i] /= sum_exp;
  if (s.min_p > 0.0f) {
    const float threshold = s.min_p * probs[0];
    size_t nl = limit;
    for (size_t i = 0; i < limit; ++i)
      if (probs[i] < threshold) {
        nl = i;
        break;
      }
    if (nl > 0)
      limit = nl;
  }
  if (s.top_p < 1.0f) {
    float cum = 0.0f;
    size_t nl = limit;
    for (size_t i = 0; i < limit; ++i) {
      cum += probs[i];
      if (cum >= s.top_p) {
        nl = i + 1;
        break;
      }
    }
    limit = nl;
  }
  float final_sum = 0.0f;
  for (size_t i = 0; i < limit; ++i)
    final_sum += probs[i];
  for (size_t i = 0; i < limit; ++i)
    probs[i] /= final_sum;
  std::discrete_distribution<int> dist(probs.begin(), probs.begin() + (long)limit);
  const int chosen = dist(s.rng);
  if (n_kept)
    *n_kept = (int64_t)limit;
  return cand[(size_t)chosen].first;
}
}
