/* TEST INFRASTRUCTURE: CPU restatement of the reference decode GEMV kernels.
 * Not part of the shipped library. */
#include "oracle.h"
#include <math.h>
#include <omp.h>

int oracle_num_threads(void) { return omp_get_max_threads(); }

#define VEC 32

/* DequantMatMulVectorizationDecode.cpp:250-321.
 *   scf.parallel n0 = 0..N step 32                       (:250-254)
 *     acc = 0                                            (:239-242,260)
 *     scf.for k: acc = fma(bcast(A[0,k]), sitofp(W[k,n0:+32]), acc)  (:259-283)
 *     C[0,n0:+32] = C[0,n0:+32] + acc * scale[0,n0:+32]  (:287-320)
 * The pattern emits full 32-wide vector loads with no tail handling; a ragged
 * last panel is restated lane-wise (the values of in-range lanes are the same).
 */
void oracle_dequant_gemv_w8a32(const float *A, const int8_t *W,
                               const float *scale, float *C, int64_t K,
                               int64_t N) {
#pragma omp parallel for schedule(static)
  for (int64_t n0 = 0; n0 < N; n0 += VEC) {
    int64_t w = N - n0 < VEC ? N - n0 : VEC;
    float acc[VEC];
    for (int v = 0; v < VEC; ++v)
      acc[v] = 0.0f;
    for (int64_t k = 0; k < K; ++k) {
      const float a = A[k];
      const int8_t *row = W + k * N + n0;
      for (int64_t v = 0; v < w; ++v)
        acc[v] = fmaf(a, (float)row[v], acc[v]);
    }
    for (int64_t v = 0; v < w; ++v) {
      float scaled = acc[v] * scale[n0 + v];
      C[n0 + v] = C[n0 + v] + scaled;
    }
  }
}

/* Same loop nest over an int8 matrix stored in the reference's panel order
 * flat[n0*K + k*32 + v] (MatMulVectorizationDecodePacked.cpp:224-240 address
 * arithmetic applied to int8; the reference refuses this combination,
 * tools/buddy-codegen/gen_config.py:366-370).  Used as the "not a straw man"
 * CPU baseline only. */
void oracle_dequant_gemv_w8a32_panels(const float *A, const int8_t *Wp,
                                      const float *scale, float *C, int64_t K,
                                      int64_t N) {
#pragma omp parallel for schedule(static)
  for (int64_t n0 = 0; n0 < N; n0 += VEC) {
    float acc[VEC];
    for (int v = 0; v < VEC; ++v)
      acc[v] = 0.0f;
    const int8_t *panel = Wp + n0 * K;
    for (int64_t k = 0; k < K; ++k) {
      const float a = A[k];
      const int8_t *row = panel + k * VEC;
      for (int v = 0; v < VEC; ++v)
        acc[v] = fmaf(a, (float)row[v], acc[v]);
    }
    for (int v = 0; v < VEC; ++v) {
      float scaled = acc[v] * scale[n0 + v];
      C[n0 + v] = C[n0 + v] + scaled;
    }
  }
}

/* MatMulVectorizationDecodePacked.cpp:207-248: the accumulator is seeded with
 * C (or with zero when the pass proved C zero-initialised, :209-222) and the
 * result is stored straight back -- no separate add.  linOffset = n0*K + k*V
 * (:224-240). */
void oracle_gemv_packed_f32(const float *A, const float *flatB, float *C,
                            int64_t K, int64_t N, int64_t V, int zero_init) {
#pragma omp parallel for schedule(static)
  for (int64_t n0 = 0; n0 < N; n0 += V) {
    for (int64_t v = 0; v < V; ++v) {
      float acc = zero_init ? 0.0f : C[n0 + v];
      for (int64_t k = 0; k < K; ++k)
        acc = fmaf(A[k], flatB[n0 * K + k * V + v], acc);
      C[n0 + v] = acc;
    }
  }
}

/* MatMulVectorizationDecode.cpp:142-175: same loop with B[k, n0:n0+V]
 * addressing (:158-171). */
void oracle_gemv_f32(const float *A, const float *B, float *C, int64_t K,
                     int64_t N, int64_t V, int zero_init) {
#pragma omp parallel for schedule(static)
  for (int64_t n0 = 0; n0 < N; n0 += V) {
    int64_t w = N - n0 < V ? N - n0 : V;
    for (int64_t v = 0; v < w; ++v) {
      float acc = zero_init ? 0.0f : C[n0 + v];
      for (int64_t k = 0; k < K; ++k)
        acc = fmaf(A[k], B[k * N + n0 + v], acc);
      C[n0 + v] = acc;
    }
  }
}
