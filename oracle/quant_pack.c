/* TEST INFRASTRUCTURE: CPU restatement of the reference quantizer and panel
 * packing.  Not part of the shipped library. */
#include "oracle.h"
#include <math.h>
#include <string.h>

/* tools/buddy-codegen/import_model.py:837-848 (weights) and :874-880 (scales):
 *   amax  = tensor.abs().amax(dim=all-but-quant-axis, keepdim=True)
 *   scale = (amax / quant_max).clamp(min=1e-10)
 *   q     = clamp(round(tensor / scale), lo, hi).to(int8)
 * with the quant axis = the output channel (last dim of [K,N]),
 * weight_only_channel_wise.py:443-454.  All arithmetic is f32; torch.round is
 * round-half-to-even, i.e. rintf() under the default rounding mode. */
static void quantize_generic(const float *W, int64_t K, int64_t N, int8_t *q,
                             float *scale, float qmax, float lo, float hi) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    float amax = 0.0f;
    for (int64_t k = 0; k < K; ++k) {
      float a = fabsf(W[k * N + n]);
      if (a > amax)
        amax = a;
    }
    float s = amax / qmax;
    if (s < 1e-10f)
      s = 1e-10f;
    scale[n] = s;
  }
#pragma omp parallel for schedule(static)
  for (int64_t k = 0; k < K; ++k) {
    for (int64_t n = 0; n < N; ++n) {
      float r = rintf(W[k * N + n] / scale[n]);
      if (r < lo)
        r = lo;
      if (r > hi)
        r = hi;
      q[k * N + n] = (int8_t)r;
    }
  }
}

void oracle_quantize_w8(const float *W, int64_t K, int64_t N, int8_t *q,
                        float *scale) {
  quantize_generic(W, K, N, q, scale, 127.0f, -128.0f, 127.0f);
}

void oracle_quantize_w4(const float *W, int64_t K, int64_t N, int8_t *q,
                        float *scale) {
  quantize_generic(W, K, N, q, scale, 7.0f, -8.0f, 7.0f);
}

/* frontend/Python/graph/transform/pack_decode_weights.py:102-108:
 *   weight.reshape(k, n/V, V).permute(1, 0, 2).contiguous().reshape(k, n)
 * so flat[nt*K*V + k*V + v] = B[k, nt*V + v]
 * (docs/DecodeWeightPacking.md:41-44).  N % V != 0 is refused (:95-99). */
int oracle_pack_panels(const void *B, int64_t K, int64_t N, int64_t V,
                       size_t elem, void *out) {
  if (V <= 0 || N % V != 0)
    return -1;
  const char *src = (const char *)B;
  char *dst = (char *)out;
  for (int64_t nt = 0; nt < N / V; ++nt)
    for (int64_t k = 0; k < K; ++k)
      memcpy(dst + (size_t)(nt * K * V + k * V) * elem,
             src + (size_t)(k * N + nt * V) * elem, (size_t)V * elem);
  return 0;
}

int oracle_unpack_panels(const void *P, int64_t K, int64_t N, int64_t V,
                         size_t elem, void *out) {
  if (V <= 0 || N % V != 0)
    return -1;
  const char *src = (const char *)P;
  char *dst = (char *)out;
  for (int64_t nt = 0; nt < N / V; ++nt)
    for (int64_t k = 0; k < K; ++k)
      memcpy(dst + (size_t)(k * N + nt * V) * elem,
             src + (size_t)(nt * K * V + k * V) * elem, (size_t)V * elem);
  return 0;
}
