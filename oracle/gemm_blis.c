/* TEST INFRASTRUCTURE: CPU restatement of the reference BLIS-style prefill
 * GEMM with the int8 dequantisation fused into B packing.  Not part of the
 * shipped library. */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>

/* MatMulBlisVectorization.cpp:351-360 */
enum { NC = 256, KC = 128, MC = 64, MR = 8, NR = 32 };

static inline int64_t imin(int64_t a, int64_t b) { return a < b ? a : b; }

/* One (jc, pc) block against every ic block.  Bp is the packed [kc, nc] f32
 * panel.  C is updated once per kc block: C += sum (:755-811), so partial sums
 * are rounded into C every 128 k.
 *   full 8x32 tile: 8 accumulators, acc = fma(bcast(A[i,k]), Bp[k, j:j+32], acc)
 *                   seeded with zero (:628-740), then C = C + acc.
 *   ragged rows (<8) of a full 32-column strip: scalar sum = sum + a*b with an
 *                   unfused mulf/addf (:815-876).
 *   ragged columns (<32): scalar, unfused, every row (:880-942). */
static void block_update(const float *A, int64_t lda, const float *Bp,
                         int64_t ncA, int64_t kcA, float *C, int64_t ldc,
                         int64_t M, int64_t jc, int64_t pc) {
#pragma omp parallel for schedule(static)
  for (int64_t ic = 0; ic < M; ic += MC) {
    int64_t mcA = imin(MC, M - ic);
    /* A packing (:569-584) is a plain copy; index A directly. */
    const float *Ap = A + ic * lda + pc;
    for (int64_t jr = 0; jr < ncA; jr += NR) {
      int64_t nrA = imin(NR, ncA - jr);
      /* the "micro blocks" loop (:598-606) runs once: nIdx = 0 */
      if (nrA >= NR) {
        for (int64_t ir = 0; ir < mcA; ir += MR) {
          int64_t mrA = imin(MR, mcA - ir);
          if (mrA >= MR) {
            float acc[MR][NR];
            for (int r = 0; r < MR; ++r)
              for (int v = 0; v < NR; ++v)
                acc[r][v] = 0.0f;
            for (int64_t k = 0; k < kcA; ++k) {
              const float *b = Bp + k * ncA + jr;
              for (int r = 0; r < MR; ++r) {
                const float a = Ap[(ir + r) * lda + k];
                for (int v = 0; v < NR; ++v)
                  acc[r][v] = fmaf(a, b[v], acc[r][v]);
              }
            }
            for (int r = 0; r < MR; ++r) {
              float *c = C + (ic + ir + r) * ldc + jc + jr;
              for (int v = 0; v < NR; ++v)
                c[v] = c[v] + acc[r][v];
            }
          } else {
            for (int64_t jj = 0; jj < NR; ++jj)
              for (int64_t ii = ir; ii < ir + mrA; ++ii) {
                float sum = 0.0f;
                for (int64_t k = 0; k < kcA; ++k) {
                  float prod = Ap[ii * lda + k] * Bp[k * ncA + jr + jj];
                  sum = sum + prod;
                }
                float *c = C + (ic + ii) * ldc + jc + jr + jj;
                *c = *c + sum;
              }
          }
        }
      } else {
        for (int64_t jt = 0; jt < nrA; ++jt)
          for (int64_t ii = 0; ii < mcA; ++ii) {
            float sum = 0.0f;
            for (int64_t k = 0; k < kcA; ++k) {
              float prod = Ap[ii * lda + k] * Bp[k * ncA + jr + jt];
              sum = sum + prod;
            }
            float *c = C + (ic + ii) * ldc + jc + jr + jt;
            *c = *c + sum;
          }
      }
    }
  }
}

/* The reference parallelises jc (scf.parallel, :400) and ic (:544).  Each jc
 * block owns disjoint columns of C, so running jc serially here and ic in
 * parallel produces the same values. */
static void blis(const float *A, const float *B, const int8_t *W,
                 const float *scale, float *C, int64_t M, int64_t N,
                 int64_t K) {
  float *Bp = (float *)malloc(sizeof(float) * NC * KC);
  for (int64_t jc = 0; jc < N; jc += NC) {
    int64_t ncA = imin(NC, N - jc);
    for (int64_t pc = 0; pc < K; pc += KC) {
      int64_t kcA = imin(KC, K - pc);
      /* B packing with fused dequant (:484-531):
       *   Bp[kp, j] = sitofp(W[pc+kp, jc+j]) * scale[jc+j]   (mulf, rounded) */
      for (int64_t kp = 0; kp < kcA; ++kp)
        for (int64_t j = 0; j < ncA; ++j) {
          if (W) {
            float wf = (float)W[(pc + kp) * N + jc + j];
            Bp[kp * ncA + j] = wf * scale[jc + j];
          } else {
            Bp[kp * ncA + j] = B[(pc + kp) * N + jc + j];
          }
        }
      block_update(A, K, Bp, ncA, kcA, C, N, M, jc, pc);
    }
  }
  free(Bp);
}

void oracle_blis_gemm_f32(const float *A, const float *B, float *C, int64_t M,
                          int64_t N, int64_t K) {
  blis(A, B, NULL, NULL, C, M, N, K);
}

void oracle_blis_gemm_w8a32(const float *A, const int8_t *W,
                            const float *scale, float *C, int64_t M, int64_t N,
                            int64_t K) {
  blis(A, NULL, W, scale, C, M, N, K);
}
