/* w4a16.c -- CPU restatement of the reference's int4 weight-only decode path.
 * TEST INFRASTRUCTURE: only tests, the smoke check and the CPU baseline of the
 * benchmark may use it.
 *
 *  pack:   tools/buddy-codegen/import_model.py:810-815  (two int4 per byte,
 *          element 2i in the low nibble, 2i+1 in the high one; for a row-major
 *          [K, N] matrix that is channel n even -> low, n odd -> high)
 *  kernel: midend/lib/Conversion/MatMulOptimization/
 *          Int4DequantMatMulVectorizationDecode.cpp:385-468: per channel,
 *          sequential over k, in f16:
 *              acc = fma(a[k], f16(w[k][n]), acc)          (:438-446)
 *              C[n] = C[n] + acc * scale[n]                (:449-470)
 *          with low = ((b & 0x0F) << 4) >> 4 (arithmetic, i8), high = b >> 4
 *          (:404-416).
 * f16 arithmetic on the reference's x86 target is f32 arithmetic on the
 * extended operands, rounded back to f16 after every operation (there is no
 * native f16 FMA/ADD/MUL without AVX512-FP16); the same is written out here with
 * the F16C conversions.
 */
#include "oracle.h"

#include <immintrin.h>
#include <math.h>

static inline float h2f(uint16_t h) { return _cvtsh_ss(h); }
static inline uint16_t f2h(float f) {
  return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
}

void oracle_f32_to_f16(const float *x, int64_t n, uint16_t *y) {
  for (int64_t i = 0; i < n; ++i)
    y[i] = f2h(x[i]);
}
void oracle_f16_to_f32(const uint16_t *x, int64_t n, float *y) {
  for (int64_t i = 0; i < n; ++i)
    y[i] = h2f(x[i]);
}

/* import_model.py:810-815 */
int oracle_pack_int4(const int8_t *q, int64_t n, int8_t *packed) {
  if (n % 2)
    return -1;
  for (int64_t i = 0; i < n / 2; ++i) {
    const uint8_t lo = (uint8_t)q[2 * i] & 0x0F;
    const uint8_t hi = (uint8_t)(((uint8_t)q[2 * i + 1] & 0x0F) << 4);
    packed[i] = (int8_t)(lo | hi);
  }
  return 0;
}

/* Int4DequantMatMulVectorizationDecode.cpp:404-416 */
void oracle_unpack_int4(const int8_t *packed, int64_t n, int8_t *q) {
  for (int64_t i = 0; i < n / 2; ++i) {
    const int8_t b = packed[i];
    q[2 * i] = (int8_t)((int8_t)((b & 0x0F) << 4) >> 4);
    q[2 * i + 1] = (int8_t)(b >> 4);
  }
}

/* C[n] = C[n] + (sum_k a[k] * w[k][n]) * scale[n], all in f16, k in order. */
void oracle_w4a16_gemv(const uint16_t *a, const int8_t *packed, const uint16_t *scale,
                       uint16_t *c, int64_t K, int64_t N) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    uint16_t acc = 0;
    for (int64_t k = 0; k < K; ++k) {
      const int8_t b = packed[k * (N / 2) + n / 2];
      const int8_t w = (n & 1) ? (int8_t)(b >> 4) : (int8_t)((int8_t)((b & 0x0F) << 4) >> 4);
      const float wf = h2f(f2h((float)w)); /* sitofp i8 -> f16 (exact) */
      acc = f2h(fmaf(h2f(a[k]), wf, h2f(acc)));
    }
    const uint16_t scaled = f2h(h2f(acc) * h2f(scale[n]));
    c[n] = f2h(h2f(c[n]) + h2f(scaled));
  }
}
