/* TEST INFRASTRUCTURE: CPU restatement of the element-wise chain of one
 * decoder layer, greedy sampling, and the w8a8 matmul.  Not part of the
 * shipped library. */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>

/* examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:60-72
 *   sq = fpowi(x, 2) ; s = reduce_sum(sq) ; mean = s * (1/n as f32)  (:8,:62-68)
 *   r = rsqrt(mean + eps)                                           (:69-70)
 *   y = w * (x * r)                                                 (:71-73)
 * tosa.reduce_sum lowers to a sequential linalg reduction. */
void oracle_rmsnorm(const float *x, const float *w, float *y, int64_t n,
                    float inv_n, float eps) {
  float s = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    float sq = x[i] * x[i];
    s = s + sq;
  }
  float mean = s * inv_n;
  float r = 1.0f / sqrtf(mean + eps);
  for (int64_t i = 0; i < n; ++i) {
    float t = x[i] * r;
    y[i] = w[i] * t;
  }
}

/* subgraph0_decode_simplify.mlir:51-59: ang[j] = inv_freq[j % half] * f32(pos);
 * cos/sin over the concatenated [2*half] vector. */
void oracle_rope_cos_sin(const float *inv_freq, int64_t half, int64_t pos,
                         float *cosv, float *sinv) {
  float p = (float)pos;
  for (int64_t j = 0; j < 2 * half; ++j) {
    float ang = inv_freq[j % half] * p;
    cosv[j] = cosf(ang);
    sinv[j] = sinf(ang);
  }
}

/* :88-107 rotate-half: y = x*cos + cat(-x[half:], x[:half])*sin, per head. */
void oracle_rope_apply(float *x, int64_t n_heads, int64_t head_dim,
                       const float *cosv, const float *sinv) {
  const int64_t half = head_dim / 2;
  float tmp[1024];
  for (int64_t h = 0; h < n_heads; ++h) {
    float *v = x + h * head_dim;
    for (int64_t j = 0; j < head_dim; ++j) {
      float rot = j < half ? -v[j + half] : v[j - half];
      float a = v[j] * cosv[j];
      float b = rot * sinv[j];
      tmp[j] = a + b;
    }
    for (int64_t j = 0; j < head_dim; ++j)
      v[j] = tmp[j];
  }
}

/* :225-232: h = (g * sigmoid(g)) * u ; tosa.sigmoid = 1/(1+exp(-g)). */
void oracle_silu_mul(const float *g, const float *u, float *h, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    float sig = 1.0f / (1.0f + expf(-g[i]));
    float silu = g[i] * sig;
    h[i] = silu * u[i];
  }
}

/* runtime/include/buddy/runtime/llm/Sampler.h:101-104: std::max_element
 * returns the FIRST maximum. */
int64_t oracle_argmax_first(const float *x, int64_t n) {
  int64_t best = 0;
  for (int64_t i = 1; i < n; ++i)
    if (x[best] < x[i])
      best = i;
  return best;
}

/* frontend/Python/ops/linalg.py:12737-12792: dynamic per-tensor activation
 * quantisation.  s = max(absmax * recip(127), 1e-10) ; inv = recip(s) ;
 * xq = clamp(f32(i32(x*inv)), -128, 127) with the TOSA f32->i32 cast rounding
 * to nearest even. */
void oracle_w8a8_quantize_activation(const float *x, int64_t n, int8_t *xq,
                                     float *scale) {
  float amax = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    float a = fabsf(x[i]);
    if (a > amax)
      amax = a;
  }
  float r127 = 1.0f / 127.0f;
  float s = amax * r127;
  if (s < 1e-10f)
    s = 1e-10f;
  float inv = 1.0f / s;
  for (int64_t i = 0; i < n; ++i) {
    float r = rintf(x[i] * inv);
    if (r < -128.0f)
      r = -128.0f;
    if (r > 127.0f)
      r = 127.0f;
    xq[i] = (int8_t)r;
  }
  *scale = s;
}

/* linalg.py:12814-12845: acc_i32 = xq . W ; y = f32(acc) * (s_a * s_w[n]).
 * The int32 partial sums are exact and returned for bit-exact comparison. */
void oracle_w8a8_matmul(const float *A, const int8_t *W, const float *wscale,
                        float *C, int32_t *acc_out, int64_t M, int64_t N,
                        int64_t K) {
  int8_t *xq = (int8_t *)malloc((size_t)(M * K));
  float sa;
  oracle_w8a8_quantize_activation(A, M * K, xq, &sa);
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t m = 0; m < M; ++m) {
      int32_t acc = 0;
      for (int64_t k = 0; k < K; ++k)
        acc += (int32_t)xq[m * K + k] * (int32_t)W[k * N + n];
      if (acc_out)
        acc_out[m * N + n] = acc;
      float comb = sa * wscale[n];
      C[m * N + n] = (float)acc * comb;
    }
  free(xq);
}
