// sampler.hip -- the reference's token sampler with its vocabulary-sized part on
// the device.
//
// runtime/include/buddy/runtime/llm/Sampler.h:62-206 copies the logits, applies
// the repetition penalty (:112-129) and the temperature (:131-136), sorts the
// whole vocabulary (:147-149), keeps the top K, and then works on those K
// candidates only: softmax in f32, min-P, top-P, renormalisation and a draw from
// std::discrete_distribution over std::mt19937 (:151-203).  In a decode loop
// whose logits live on the device that would mean 608 KB over PCIe and a
// 152k-element sort on the host per token.  Here the penalty, the temperature
// and the top-K selection run on the device, K (value, index) pairs come back,
// and the host does what the reference does with them, with the same standard
// library generator and distribution, so the chosen token is the reference's.
//
// Selection: (1) every logit becomes a 32-bit key that orders like its value and
// is counted in a 4096-bin histogram of the key's leading bits; (2) the bin in
// which the K-th largest key falls is found from the histogram and every key in
// that bin or above (a few hundred for logits that are not all alike) is
// appended to a candidate list; (3) one workgroup sorts the candidates and
// writes the first K to pinned host memory.  Logits so alike that more than
// 4096 share the leading bins go through a full sort instead: bitonic sorts of
// 4096-logit blocks, then one sort of the block winners.
// Candidates of equal value are ordered by index (the reference's std::sort
// leaves their order unspecified).  Without a top-K limit (or with one beyond
// what the device selection holds) the logits are copied back and the whole of
// the reference's algorithm runs on the host.
#include "common.h"

#include <algorithm>
#include <cmath>
#include <new>
#include <random>
#include <utility>
#include <vector>

struct buddy_hip_sampler {
  buddy_hip_sampler_config cfg;
  std::mt19937 rng;
  int *h_recent = nullptr;                 // pinned staging of a window beyond 64 ids
  int *d_recent = nullptr;
  unsigned long long *h_out = nullptr;     // pinned: [0] candidate count, [1..K] keys
  unsigned *d_hist = nullptr;              // kBins + 1 (the candidate counter); kept zero
  unsigned *d_keys = nullptr;              // one per logit
  unsigned long long *d_cand = nullptr;    // kMaxCand
  unsigned long long *d_partial = nullptr; // full-sort path: block winners
  size_t keys_cap = 0, partial_cap = 0;
  std::vector<float> h_logits;
};

namespace bh {
namespace {

typedef unsigned long long u64;

constexpr int kBlockElems = 4096; // logits per workgroup of the first launch
constexpr int kMergeElems = 8192; // keys the second launch sorts
constexpr int kMaxWindow = 1024;  // repetition-penalty window held in LDS
constexpr int kArgWindow = 64;    // ... of which a kernel argument carries this many

// A window of up to 64 ids (the reference's default repeatLastN) travels with
// the launch; a longer one is read from device memory.
struct Window {
  int ids[kArgWindow];
};

constexpr int kSelectElems = 1024; // logits per workgroup of the threshold selection
constexpr int kBins = 4096;       // histogram over the leading 12 bits of a key
constexpr int kMaxCand = 4096;    // candidates the threshold selection holds

// a 32-bit integer that orders like the float
__device__ __forceinline__ unsigned value_key(float v) {
  const unsigned u = __float_as_uint(v);
  return u ^ ((u >> 31) ? 0xffffffffu : 0x80000000u);
}
// (value, index) as one integer: larger value first, then the smaller index
__device__ __forceinline__ u64 pair_key(unsigned vkey, int i) {
  return ((u64)vkey << 32) | (u64)(0xffffffffu - (unsigned)i);
}
__device__ __forceinline__ u64 make_key(float v, int i) { return pair_key(value_key(v), i); }

// Penalty once per occurrence in the window (like the reference), then
// temperature.  win holds the window padded with -1 to a multiple of four; the
// occurrences are counted first, without branches, so that the LDS reads of the
// whole window are in flight together.
__device__ __forceinline__ float adjust(float v, int i, const int *win, int n_recent,
                                        float penalty, float inv_temp) {
  int count = 0;
  const int4 *w4 = reinterpret_cast<const int4 *>(win);
  for (int r = 0; r < (n_recent + 3) / 4; ++r) {
    const int4 w = w4[r];
    count += (w.x == i) + (w.y == i) + (w.z == i) + (w.w == i);
  }
  for (int c = 0; c < count; ++c)
    v = v > 0.0f ? v / penalty : v * penalty;
  return v * inv_temp;
}

inline void split_key(u64 k, float *v, int *i) {
  unsigned u = (unsigned)(k >> 32);
  u ^= (u >> 31) ? 0x80000000u : 0xffffffffu;
  union {
    unsigned u;
    float f;
  } c;
  c.u = u;
  *v = c.f;
  *i = (int)(0xffffffffu - (unsigned)(k & 0xffffffffu));
}

// descending bitonic sort of N keys in LDS by T threads
template <int N, int T> __device__ __forceinline__ void sort_desc(u64 *keys) {
  for (int size = 2; size <= N; size <<= 1)
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      __syncthreads();
      for (int t = threadIdx.x; t < N / 2; t += T) {
        const int lo = 2 * t - (t & (stride - 1)), hi = lo + stride;
        const bool desc = (lo & size) == 0;
        const u64 a = keys[lo], b = keys[hi];
        if ((a < b) == desc) {
          keys[lo] = b;
          keys[hi] = a;
        }
      }
    }
  __syncthreads();
}

// descending bitonic sort of n (a power of two) keys in LDS by 256 threads
__device__ __forceinline__ void sort_desc_n(u64 *keys, int n) {
  for (int size = 2; size <= n; size <<= 1)
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      __syncthreads();
      for (int t = threadIdx.x; t < n / 2; t += 256) {
        const int lo = 2 * t - (t & (stride - 1)), hi = lo + stride;
        const bool desc = (lo & size) == 0;
        const u64 a = keys[lo], b = keys[hi];
        if ((a < b) == desc) {
          keys[lo] = b;
          keys[hi] = a;
        }
      }
    }
  __syncthreads();
}

// (1) Workgroup b: keys of logits [b*1024, +1024) to vkeys, their leading 12
// bits counted into hist.  Only logits whose id is in the window (a bitmap of
// this block's ids) walk the window.
__global__ void __launch_bounds__(256)
sampler_keys_kernel(const float *__restrict__ logits, int vocab, Window small,
                    const int *__restrict__ recent, int n_recent, float penalty, float inv_temp,
                    unsigned *__restrict__ vkeys, unsigned *__restrict__ hist) {
  __shared__ unsigned bins[kBins];
  __shared__ unsigned in_window[kSelectElems / 32];
  __shared__ __align__(16) int win[kMaxWindow];
  const int base = blockIdx.x * kSelectElems;
  for (int i = threadIdx.x; i < kBins; i += 256)
    bins[i] = 0;
  if (threadIdx.x < kSelectElems / 32)
    in_window[threadIdx.x] = 0;
  __syncthreads();
  for (int r = threadIdx.x; r < (n_recent + 3) / 4 * 4; r += 256) {
    const int t = r >= n_recent ? -1 : n_recent <= kArgWindow ? small.ids[r] : recent[r];
    win[r] = t;
    const unsigned e = (unsigned)(t - base);
    if (e < (unsigned)kSelectElems)
      atomicOr(&in_window[e >> 5], 1u << (e & 31));
  }
  __syncthreads();
  for (int e = threadIdx.x; e < kSelectElems; e += 256) {
    const int i = base + e;
    if (i >= vocab)
      break;
    float v = logits[i];
    if (in_window[e >> 5] >> (e & 31) & 1)
      v = adjust(v, i, win, n_recent, penalty, 1.0f);
    const unsigned k = value_key(v * inv_temp);
    vkeys[i] = k;
    atomicAdd(&bins[k >> 20], 1u);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < kBins; i += 256)
    if (bins[i])
      atomicAdd(&hist[i], bins[i]);
}

// (2) The bin holding the K-th largest key, from the histogram; keys of this
// block in that bin or above go to cand (counter = hist[kBins]).
__global__ void __launch_bounds__(256)
sampler_candidates_kernel(const unsigned *__restrict__ vkeys, int vocab, int K,
                          unsigned *__restrict__ hist, u64 *__restrict__ cand) {
  __shared__ unsigned above[256]; // keys in the bins above thread t's 16
  __shared__ int threshold;
  const int t = threadIdx.x;
  unsigned mine[16], sum = 0;
  for (int j = 0; j < 16; ++j) {
    mine[j] = hist[t * 16 + j];
    sum += mine[j];
  }
  above[t] = sum;
  __syncthreads();
  for (int d = 1; d < 256; d <<= 1) { // inclusive suffix sums
    const unsigned add = t + d < 256 ? above[t + d] : 0;
    __syncthreads();
    above[t] += add;
    __syncthreads();
  }
  // the one thread whose bins take the count from below K to K or more
  const unsigned higher = above[t] - sum;
  if (higher < (unsigned)K && above[t] >= (unsigned)K) {
    unsigned c = higher;
    int b = 15;
    for (; b > 0; --b) {
      c += mine[b];
      if (c >= (unsigned)K)
        break;
    }
    threshold = t * 16 + b;
  }
  __syncthreads();
  const unsigned lowest = (unsigned)threshold << 20;
  const int base = blockIdx.x * kSelectElems;
  for (int e = t; e < kSelectElems; e += 256) {
    const int i = base + e;
    if (i >= vocab)
      break;
    const unsigned k = vkeys[i];
    if (k >= lowest) {
      const unsigned slot = atomicAdd(&hist[kBins], 1u);
      if (slot < (unsigned)kMaxCand)
        cand[slot] = pair_key(k, i);
    }
  }
}

// (3) One workgroup: sorts the candidates, writes their count and the first K
// to out (pinned host memory), and clears the histogram and the counter for the
// next call.  More than kMaxCand candidates: only the count is written.
__global__ void __launch_bounds__(256)
sampler_pick_kernel(const u64 *__restrict__ cand, int K, unsigned *__restrict__ hist,
                    u64 *__restrict__ out) {
  __shared__ u64 keys[kMaxCand];
  const unsigned n = hist[kBins];
  __syncthreads();
  for (int i = threadIdx.x; i <= kBins; i += 256)
    hist[i] = 0;
  if (n <= (unsigned)kMaxCand) {
    int p = 64;
    while (p < (int)n)
      p <<= 1;
    for (int i = threadIdx.x; i < p; i += 256)
      keys[i] = i < (int)n ? cand[i] : 0;
    sort_desc_n(keys, p);
    for (int j = threadIdx.x; j < K; j += 256)
      out[1 + j] = keys[j];
  }
  if (threadIdx.x == 0)
    out[0] = n;
}

// Full-sort path, workgroup b: penalty and temperature on logits
// [b*4096, +4096), its K largest in order to partial[b*K ..].
__global__ void __launch_bounds__(256)
sampler_block_topk_kernel(const float *__restrict__ logits, int vocab, Window small,
                          const int *__restrict__ recent, int n_recent, float penalty,
                          float inv_temp, int K, u64 *__restrict__ partial) {
  __shared__ u64 keys[kBlockElems];
  __shared__ __align__(16) int win[kMaxWindow];
  for (int i = threadIdx.x; i < (n_recent + 3) / 4 * 4; i += 256)
    win[i] = i >= n_recent ? -1 : n_recent <= kArgWindow ? small.ids[i] : recent[i];
  __syncthreads();
  const int base = blockIdx.x * kBlockElems;
  for (int e = threadIdx.x; e < kBlockElems; e += 256) {
    const int i = base + e;
    u64 key = 0; // below every real key
    if (i < vocab) {
      key = make_key(adjust(logits[i], i, win, n_recent, penalty, inv_temp), i);
    }
    keys[e] = key;
  }
  sort_desc<kBlockElems, 256>(keys);
  for (int j = threadIdx.x; j < K; j += 256)
    partial[(size_t)blockIdx.x * K + j] = keys[j];
}

// Full-sort path, one workgroup: the K largest of the block winners, in order.
__global__ void __launch_bounds__(1024)
sampler_merge_kernel(const u64 *__restrict__ partial, int n, int K, u64 *__restrict__ out) {
  __shared__ u64 keys[kMergeElems];
  for (int i = threadIdx.x; i < kMergeElems; i += 1024)
    keys[i] = i < n ? partial[i] : 0;
  sort_desc<kMergeElems, 1024>(keys);
  for (int j = threadIdx.x; j < K; j += 1024)
    out[1 + j] = keys[j];
}

// Sampler.h:151-203 on candidates sorted by value (all of them the top-K limit
// lets through).  Returns the position of the chosen candidate.
int draw(buddy_hip_sampler *s, const std::vector<std::pair<int, float>> &cand) {
  size_t limit = cand.size();
  const float max_logit = cand[0].second;
  std::vector<float> probs(limit);
  float sum_exp = 0.0f;
  for (size_t i = 0; i < limit; ++i) {
    probs[i] = std::exp(cand[i].second - max_logit);
    sum_exp += probs[i];
  }
  for (size_t i = 0; i < limit; ++i)
    probs[i] /= sum_exp;
  if (s->cfg.min_p > 0.0f) {
    const float threshold = s->cfg.min_p * probs[0];
    size_t nl = limit;
    for (size_t i = 0; i < limit; ++i)
      if (probs[i] < threshold) {
        nl = i;
        break;
      }
    if (nl > 0)
      limit = nl;
  }
  if (s->cfg.top_p < 1.0f) {
    float cum = 0.0f;
    size_t nl = limit;
    for (size_t i = 0; i < limit; ++i) {
      cum += probs[i];
      if (cum >= s->cfg.top_p) {
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
  return dist(s->rng);
}

} // namespace
} // namespace bh

extern "C" {

buddy_hip_sampler *buddy_hip_sampler_create(const buddy_hip_sampler_config *cfg) try {
  if (!cfg || cfg->temperature < 0.0f || cfg->top_k < 0 || cfg->repeat_last_n < 0 ||
      !(cfg->repeat_penalty > 0.0f)) {
    bh::fail(BUDDY_HIP_ERR_ARG, "sampler_create: bad configuration");
    return nullptr;
  }
  buddy_hip_sampler *s = new (std::nothrow) buddy_hip_sampler;
  if (!s) {
    bh::fail(BUDDY_HIP_ERR_ARG, "sampler_create: out of host memory");
    return nullptr;
  }
  s->cfg = *cfg;
  if (cfg->seed != 0) { // Sampler.h:51-56
    s->rng.seed(cfg->seed);
  } else {
    std::random_device rd;
    s->rng.seed(rd());
  }
  const int K = BUDDY_HIP_SAMPLER_MAX_TOP_K;
  if (hipHostMalloc((void **)&s->h_recent, sizeof(int) * bh::kMaxWindow) != hipSuccess ||
      hipMalloc((void **)&s->d_recent, sizeof(int) * bh::kMaxWindow) != hipSuccess ||
      hipHostMalloc((void **)&s->h_out, sizeof(bh::u64) * (K + 1)) != hipSuccess ||
      hipMalloc((void **)&s->d_hist, sizeof(unsigned) * (bh::kBins + 1)) != hipSuccess ||
      hipMalloc((void **)&s->d_cand, sizeof(bh::u64) * bh::kMaxCand) != hipSuccess ||
      hipMemset(s->d_hist, 0, sizeof(unsigned) * (bh::kBins + 1)) != hipSuccess) {
    bh::fail(BUDDY_HIP_ERR_HIP, "sampler_create: allocation failed");
    buddy_hip_sampler_destroy(s);
    return nullptr;
  }
  return s;
} BH_CATCH_NULL("buddy_hip_sampler_create")

void buddy_hip_sampler_destroy(buddy_hip_sampler *s) try {
  if (!s)
    return;
  for (void *p : {(void *)s->d_hist, (void *)s->d_keys, (void *)s->d_cand, (void *)s->d_partial,
                  (void *)s->d_recent})
    if (p)
      (void)hipFree(p);
  for (void *p : {(void *)s->h_recent, (void *)s->h_out})
    if (p)
      (void)hipHostFree(p);
  delete s;
} BH_CATCH_VOID("buddy_hip_sampler_destroy")

int buddy_hip_sampler_sample(buddy_hip_sampler *s, const float *logits, int vocab,
                             const int *recent, int n_recent, int *token_out,
                             buddy_hip_stream hstream) try {
  BH_REQUIRE(s && logits && token_out && vocab > 0 && n_recent >= 0 && (recent || !n_recent),
             "sampler_sample: bad argument");
  hipStream_t stream = bh::as_stream(hstream);
  const buddy_hip_sampler_config &c = s->cfg;
  // the window the penalty looks at (Sampler.h:114-117)
  int w0 = n_recent - c.repeat_last_n;
  if (w0 < 0)
    w0 = 0;
  const bool penalty = c.repeat_penalty != 1.0f && n_recent > 0;
  const int window = penalty ? n_recent - w0 : 0;
  const bool greedy = c.temperature == 0.0f;
  const float inv_temp = greedy ? 1.0f : 1.0f / c.temperature;
  // greedy = the first maximum (Sampler.h:101-104): the top 1 with ties by index
  const int K = greedy ? 1 : c.top_k;
  const int blocks = (int)bh::ceil_div(vocab, bh::kBlockElems);
  const bool on_device = K >= 1 && K <= BUDDY_HIP_SAMPLER_MAX_TOP_K && K <= vocab &&
                         (int64_t)blocks * K <= bh::kMergeElems && window <= bh::kMaxWindow;
  std::vector<std::pair<int, float>> cand;
  if (on_device) {
    bh::Window small = {};
    if (window <= bh::kArgWindow) {
      for (int i = 0; i < window; ++i)
        small.ids[i] = recent[w0 + i];
    } else {
      for (int i = 0; i < window; ++i)
        s->h_recent[i] = recent[w0 + i];
      BH_CHECK_HIP(hipMemcpyAsync(s->d_recent, s->h_recent, sizeof(int) * window,
                                  hipMemcpyHostToDevice, stream));
    }
    bool selected = false;
    {
      const int sel_blocks = (int)bh::ceil_div(vocab, bh::kSelectElems);
      if (s->keys_cap < (size_t)vocab) {
        if (s->d_keys)
          BH_CHECK_HIP(hipFree(s->d_keys));
        s->d_keys = nullptr;
        s->keys_cap = 0;
        BH_CHECK_HIP(hipMalloc((void **)&s->d_keys, sizeof(unsigned) * (size_t)vocab));
        s->keys_cap = (size_t)vocab;
      }
      hipLaunchKernelGGL(bh::sampler_keys_kernel, dim3(sel_blocks), dim3(256), 0, stream, logits,
                         vocab, small, s->d_recent, window, c.repeat_penalty, inv_temp,
                         s->d_keys, s->d_hist);
      hipLaunchKernelGGL(bh::sampler_candidates_kernel, dim3(sel_blocks), dim3(256), 0, stream,
                         s->d_keys, vocab, K, s->d_hist, s->d_cand);
      hipLaunchKernelGGL(bh::sampler_pick_kernel, dim3(1), dim3(256), 0, stream, s->d_cand, K,
                         s->d_hist, s->h_out);
      BH_CHECK_HIP(hipGetLastError());
      BH_CHECK_HIP(hipStreamSynchronize(stream));
      selected = s->h_out[0] <= (bh::u64)bh::kMaxCand;
    }
    if (!selected) { // too many logits alike: sort everything
      if (s->partial_cap < (size_t)blocks * K) {
        if (s->d_partial)
          BH_CHECK_HIP(hipFree(s->d_partial));
        s->d_partial = nullptr;
        s->partial_cap = 0;
        BH_CHECK_HIP(hipMalloc((void **)&s->d_partial, sizeof(bh::u64) * (size_t)blocks * K));
        s->partial_cap = (size_t)blocks * K;
      }
      hipLaunchKernelGGL(bh::sampler_block_topk_kernel, dim3(blocks), dim3(256), 0, stream,
                         logits, vocab, small, s->d_recent, window, c.repeat_penalty, inv_temp,
                         K, s->d_partial);
      hipLaunchKernelGGL(bh::sampler_merge_kernel, dim3(1), dim3(1024), 0, stream, s->d_partial,
                         blocks * K, K, s->h_out);
      BH_CHECK_HIP(hipGetLastError());
      BH_CHECK_HIP(hipStreamSynchronize(stream));
    }
    cand.resize((size_t)K);
    for (int j = 0; j < K; ++j)
      bh::split_key(s->h_out[1 + j], &cand[(size_t)j].second, &cand[(size_t)j].first);
  } else {
    // the whole of the reference's algorithm on the host
    s->h_logits.resize((size_t)vocab);
    BH_CHECK_HIP(hipMemcpyAsync(s->h_logits.data(), logits, sizeof(float) * (size_t)vocab,
                                hipMemcpyDefault, stream));
    BH_CHECK_HIP(hipStreamSynchronize(stream));
    std::vector<float> &work = s->h_logits;
    for (int i = w0; penalty && i < n_recent; ++i) {
      const int t = recent[i];
      if (t < 0 || t >= vocab)
        continue;
      if (work[(size_t)t] > 0.0f)
        work[(size_t)t] /= c.repeat_penalty;
      else
        work[(size_t)t] *= c.repeat_penalty;
    }
    if (greedy) {
      *token_out = (int)std::distance(work.begin(), std::max_element(work.begin(), work.end()));
      return BUDDY_HIP_OK;
    }
    for (float &v : work)
      v *= inv_temp;
    cand.resize((size_t)vocab);
    for (int i = 0; i < vocab; ++i)
      cand[(size_t)i] = {i, work[(size_t)i]};
    std::sort(cand.begin(), cand.end(),
              [](const std::pair<int, float> &a, const std::pair<int, float> &b) {
                return a.second > b.second;
              });
    if (c.top_k > 0 && c.top_k < vocab)
      cand.resize((size_t)c.top_k);
  }
  if (greedy) {
    *token_out = cand[0].first;
    return BUDDY_HIP_OK;
  }
  *token_out = cand[(size_t)bh::draw(s, cand)].first;
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_sampler_sample")

int buddy_hip_session_decode_sample(buddy_hip_session *sess, buddy_hip_sampler *s, int token,
                                    int pos, const int *recent, int n_recent,
                                    int *next_token) try {
  BH_REQUIRE(sess && s && next_token, "session_decode_sample: null argument");
  int rc = buddy_hip_session_set_state(sess, token, pos);
  if (rc)
    return rc;
  if ((rc = buddy_hip_session_enqueue_steps(sess, 1)))
    return rc;
  return buddy_hip_sampler_sample(s, buddy_hip_session_logits(sess), buddy_hip_session_vocab(sess),
                                  recent, n_recent, next_token, buddy_hip_session_stream(sess));
} BH_CATCH_INT("buddy_hip_session_decode_sample")
}
