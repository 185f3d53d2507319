/* TEST INFRASTRUCTURE: CPU restatement of the reference attention kernels.
 * Not part of the shipped library. */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define SEED_M (-1.0e30f) /* tosa.py:13971 ; finite on purpose (:14242-14243) */

/* 16-lane dot product with the reference's shape: one vector<16xf32>
 * accumulator fma'd over d in steps of 16, then vector.reduction<add>
 * (tosa.py:14289-14336).  The reduction order of the 16 lanes is
 * backend-defined; lanes are summed in index order here. */
static float dot16(const float *a, const float *b, int64_t d) {
  float lane[16];
  for (int i = 0; i < 16; ++i)
    lane[i] = 0.0f;
  for (int64_t j = 0; j < d; j += 16)
    for (int i = 0; i < 16; ++i)
      lane[i] = fmaf(a[j + i], b[j + i], lane[i]);
  float s = 0.0f;
  for (int i = 0; i < 16; ++i)
    s = s + lane[i];
  return s;
}

/* frontend/Python/ops/tosa.py:14130-14600.
 * Pass 1, parallel over (head, split) (:14149-14181): k-blocks of 16
 * (:14259); per block
 *   score[j] = scale*dot(Q[h], K[h/group, k]) + mask[k]        (:14289-14351)
 *   m_block = max_j score ; new_m = m_block > m ? m_block : m   (:14355-14366)
 *   alpha = exp(m - new_m) ; p[j] = exp(score[j] - new_m)       (:14371-14382)
 *   l = l*alpha + sum_j p[j]                                    (:14383-14390)
 *   acc_block = sum_j fma(V[k], p[j], acc_block)  (seeded 0)    (:14392-14436)
 *   acc = fma(acc, alpha, acc_block)                            (:14439-14449)
 * Pass 2, serial combine over splits (:14485-14568):
 *   m_new = m_s > m_run ? m_s : m_run ; a = exp(m_run-m_new) ; b = exp(m_s-m_new)
 *   l = l*a + l_s*b ; acc = fma(acc_s, b, acc*a)
 * out = acc / l ; lse = m + log(l)                              (:14576-14594)
 * num_splits = 4 unless cache_len % 64 != 0 (:14087-14089); the caller passes
 * it so that the reference's stated split counts can be checked. */
void oracle_gqa_decode_attention(const float *q, const float *kcache,
                                 const float *vcache, const float *mask,
                                 float *out, float *lse, int64_t n_heads,
                                 int64_t n_kv_heads, int64_t cache_len,
                                 int64_t head_dim, float scale,
                                 int64_t num_splits) {
  const int64_t group = n_heads / n_kv_heads;
  if (num_splits < 1 || cache_len % (num_splits * 16) != 0)
    num_splits = 1;
  const int64_t split_len = cache_len / num_splits;
  const int64_t D = head_dim;
  float *pm = (float *)malloc(sizeof(float) * n_heads * num_splits);
  float *pl = (float *)malloc(sizeof(float) * n_heads * num_splits);
  float *pacc = (float *)malloc(sizeof(float) * n_heads * num_splits * D);

#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t h = 0; h < n_heads; ++h)
    for (int64_t s = 0; s < num_splits; ++s) {
      const int64_t hkv = h / group;
      const float *Q = q + h * D;
      const float *Kc = kcache + hkv * cache_len * D;
      const float *Vc = vcache + hkv * cache_len * D;
      float m = SEED_M, l = 0.0f;
      float *acc = pacc + (h * num_splits + s) * D;
      float accb[512];
      for (int64_t d = 0; d < D; ++d)
        acc[d] = 0.0f;
      /* a ragged last block cannot occur: split_len % 16 == 0 or splits == 1
       * with the cache length a multiple of 16 in every reference config; a
       * shorter tail is handled lane-wise. */
      for (int64_t kb = s * split_len; kb < (s + 1) * split_len; kb += 16) {
        int64_t bl = (s + 1) * split_len - kb < 16 ? (s + 1) * split_len - kb : 16;
        float score[16];
        float m_block = -INFINITY;
        for (int64_t j = 0; j < bl; ++j) {
          float dot = dot16(Q, Kc + (kb + j) * D, D);
          float scaled = dot * scale;
          score[j] = mask ? scaled + mask[kb + j] : scaled;
          if (j == 0 || score[j] > m_block)
            m_block = score[j];
        }
        float new_m = m_block > m ? m_block : m;
        float alpha = expf(m - new_m);
        float l_block = 0.0f;
        float p[16];
        for (int64_t j = 0; j < bl; ++j) {
          p[j] = expf(score[j] - new_m);
          l_block = l_block + p[j];
        }
        l = l * alpha + l_block;
        for (int64_t d = 0; d < D; ++d)
          accb[d] = 0.0f;
        for (int64_t j = 0; j < bl; ++j) {
          const float *vrow = Vc + (kb + j) * D;
          for (int64_t d = 0; d < D; ++d)
            accb[d] = fmaf(vrow[d], p[j], accb[d]);
        }
        for (int64_t d = 0; d < D; ++d)
          acc[d] = fmaf(acc[d], alpha, accb[d]);
        m = new_m;
      }
      pm[h * num_splits + s] = m;
      pl[h * num_splits + s] = l;
    }

  for (int64_t h = 0; h < n_heads; ++h) {
    float m_run = SEED_M, l_run = 0.0f;
    float acc[512];
    for (int64_t d = 0; d < D; ++d)
      acc[d] = 0.0f;
    for (int64_t s = 0; s < num_splits; ++s) {
      float m_s = pm[h * num_splits + s], l_s = pl[h * num_splits + s];
      float m_new = m_s > m_run ? m_s : m_run;
      float a = expf(m_run - m_new);
      float b = expf(m_s - m_new);
      l_run = l_run * a + l_s * b;
      const float *as = pacc + (h * num_splits + s) * D;
      for (int64_t d = 0; d < D; ++d) {
        float rescaled = acc[d] * a;
        acc[d] = fmaf(as[d], b, rescaled);
      }
      m_run = m_new;
    }
    if (lse)
      lse[h] = m_run + logf(l_run);
    for (int64_t d = 0; d < D; ++d)
      out[h * D + d] = acc[d] / l_run;
  }
  free(pm);
  free(pl);
  free(pacc);
}

/* frontend/Python/ops/tosa.py:4431-4799.  q-blocks of 16, kv-blocks of 64
 * (:4415-4416); per (head, q-block): m = -1e30, l = 0, acc = 0 (:4491-4511);
 * per kv-block (declared affine.parallel at :4513-4524 but it carries m/l/acc
 * through memrefs, so it is restated as the sequential loop it has to be):
 *   s[qi,kj] = dot16(Q, K)*scale + mask[qi,kj]                  (:4552-4623)
 *   m_block = max_kj s  (seeded -1e30, ogt)                     (:4625-4652)
 *   p = exp(s - m_block) ; l_block += p ; acc_block = fma(V, p, acc_block)
 *                                                               (:4667-4721)
 *   m_new = m_block > m ? m_block : m ; alpha = exp(m - m_new) ;
 *   beta = exp(m_block - m_new) ; acc = acc*alpha + acc_block*beta (unfused) ;
 *   l = l*alpha + l_block*beta                                  (:4722-4763)
 * out = acc / l (:4767-4795).  K and V are indexed by the query head (:4578,
 * :4700): they were already repeated to n_heads upstream. */
void oracle_prefill_flash_attention(const float *q, const float *k,
                                    const float *v, const float *mask,
                                    float *out, int64_t n_heads, int64_t q_len,
                                    int64_t k_len, int64_t head_dim,
                                    float scale) {
  const int64_t D = head_dim, BQ = 16, BKV = 64;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (int64_t h = 0; h < n_heads; ++h)
    for (int64_t qb = 0; qb < q_len; qb += BQ) {
      const float *Q = q + h * q_len * D;
      const float *Kh = k + h * k_len * D;
      const float *Vh = v + h * k_len * D;
      int64_t nq = q_len - qb < BQ ? q_len - qb : BQ;
      float m_i[16], l_i[16];
      float *acc = (float *)malloc(sizeof(float) * BQ * D);
      float *accb = (float *)malloc(sizeof(float) * D);
      float st[16][64];
      for (int i = 0; i < BQ; ++i) {
        m_i[i] = SEED_M;
        l_i[i] = 0.0f;
      }
      memset(acc, 0, sizeof(float) * BQ * D);
      for (int64_t kb = 0; kb < k_len; kb += BKV) {
        int64_t nk = k_len - kb < BKV ? k_len - kb : BKV;
        for (int64_t qi = 0; qi < nq; ++qi)
          for (int64_t kj = 0; kj < nk; ++kj) {
            float dot = dot16(Q + (qb + qi) * D, Kh + (kb + kj) * D, D);
            float scaled = dot * scale;
            st[qi][kj] = mask ? scaled + mask[(qb + qi) * k_len + kb + kj]
                              : scaled;
          }
        for (int64_t qi = 0; qi < nq; ++qi) {
          float m_block = SEED_M;
          for (int64_t kj = 0; kj < nk; ++kj)
            if (st[qi][kj] > m_block)
              m_block = st[qi][kj];
          for (int64_t d = 0; d < D; ++d)
            accb[d] = 0.0f;
          float l_block = 0.0f;
          for (int64_t kj = 0; kj < nk; ++kj) {
            float p = expf(st[qi][kj] - m_block);
            l_block = l_block + p;
            const float *vrow = Vh + (kb + kj) * D;
            for (int64_t d = 0; d < D; ++d)
              accb[d] = fmaf(vrow[d], p, accb[d]);
          }
          float m_new = m_block > m_i[qi] ? m_block : m_i[qi];
          float alpha = expf(m_i[qi] - m_new);
          float beta = expf(m_block - m_new);
          float *a = acc + qi * D;
          for (int64_t d = 0; d < D; ++d) {
            float am = a[d] * alpha;
            float bm = accb[d] * beta;
            a[d] = am + bm;
          }
          float la = l_i[qi] * alpha;
          float lb = l_block * beta;
          l_i[qi] = la + lb;
          m_i[qi] = m_new;
        }
      }
      for (int64_t qi = 0; qi < nq; ++qi)
        for (int64_t d = 0; d < D; ++d)
          out[(h * q_len + qb + qi) * D + d] = acc[qi * D + d] / l_i[qi];
      free(acc);
      free(accb);
    }
}
