// attn_prefill.hip -- causal GQA attention over a block of prompt tokens, and
// the RoPE + KV-cache write in front of it.
//
// Replaces flash_attention_for_cpu_prefill_op
// (frontend/Python/ops/tosa.py:4326-4810: q-blocks of 16, kv-blocks of 64,
// online softmax with m seeded at -1e30, out = acc / l) and, for a block of
// tokens, the RoPE / cache write of
// examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:51-59,88-142.
//
// The reference kernel is handed K and V already repeated to one copy per query
// head (tosa.py:4578-4579,4700); here the KV head is h / group, so the cache is
// read in place.  The causal structure is exploited: key tiles that lie wholly
// in a query tile's future are skipped (they are exactly zero after softmax).
// Arithmetic is f32 throughout.
#include "attn.h"

namespace bh {
namespace {

constexpr int kD = 128;
constexpr int TQ = 32, TK = 32;  // query / key rows per tile
constexpr int LDR = kD + 4;      // padded row length in LDS (floats)
constexpr float kSeedM = -1.0e30f; // tosa.py:4383

struct PrefillArgs {
  const float *q;   // token t, head h at q + t*q_stride + h*q_hstride
  const float *k, *v; // [kv_heads, kv_stride rows, D]
  const float *mask;  // additive [q_len, k_len] or null (causal)
  float *out;         // token t, head h at out + t*o_stride + h*o_hstride
  int64_t q_stride, q_hstride, o_stride, o_hstride, kv_stride;
  int heads, group, q_len, k_len, q_offset; // query i sits at key position q_offset + i
  float scale;
};

__global__ void __launch_bounds__(256) attn_prefill_kernel(PrefillArgs a) {
  __shared__ float q_s[TQ][LDR];
  __shared__ float k_s[TK][LDR];
  __shared__ float v_s[TK][LDR];
  __shared__ float p_s[TQ][TK + 1];

  const int tid = threadIdx.x;
  const int h = blockIdx.y, kvh = h / a.group;
  const int q0 = blockIdx.x * TQ;
  const int nq = min(TQ, a.q_len - q0);
  const int qi = tid >> 3, sub = tid & 7; // 8 threads per query row

  for (int i = tid; i < TQ * (kD / 4); i += 256) {
    const int r = i / (kD / 4), c = (i % (kD / 4)) * 4;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (r < nq)
      v = *reinterpret_cast<const float4 *>(a.q + (int64_t)(q0 + r) * a.q_stride +
                                            (int64_t)h * a.q_hstride + c);
    *reinterpret_cast<float4 *>(&q_s[r][c]) = v;
  }

  float m_run = kSeedM, l_run = 0.f;
  float acc[16];
#pragma unroll
  for (int d = 0; d < 16; ++d)
    acc[d] = 0.f;

  // last key any query of this tile may see
  const int k_last = a.mask ? a.k_len - 1
                            : min(a.k_len - 1, a.q_offset + q0 + nq - 1);
  const float *kbase = a.k + (int64_t)kvh * a.kv_stride * kD;
  const float *vbase = a.v + (int64_t)kvh * a.kv_stride * kD;

  for (int k0 = 0; k0 <= k_last; k0 += TK) {
    const int nk = min(TK, a.k_len - k0);
    __syncthreads(); // previous tile consumed (and q_s written, first time)
    for (int i = tid; i < TK * (kD / 4); i += 256) {
      const int r = i / (kD / 4), c = (i % (kD / 4)) * 4;
      float4 kv = make_float4(0.f, 0.f, 0.f, 0.f), vv = kv;
      if (r < nk) {
        kv = *reinterpret_cast<const float4 *>(kbase + (int64_t)(k0 + r) * kD + c);
        vv = *reinterpret_cast<const float4 *>(vbase + (int64_t)(k0 + r) * kD + c);
      }
      *reinterpret_cast<float4 *>(&k_s[r][c]) = kv;
      *reinterpret_cast<float4 *>(&v_s[r][c]) = vv;
    }
    __syncthreads();
    // scores of query qi against keys sub, sub+8, sub+16, sub+24
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    for (int d = 0; d < kD; d += 4) {
      const float4 qv = *reinterpret_cast<const float4 *>(&q_s[qi][d]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4 kv = *reinterpret_cast<const float4 *>(&k_s[sub + 8 * j][d]);
        s[j] = fmaf(qv.x, kv.x, s[j]);
        s[j] = fmaf(qv.y, kv.y, s[j]);
        s[j] = fmaf(qv.z, kv.z, s[j]);
        s[j] = fmaf(qv.w, kv.w, s[j]);
      }
    }
    float m_blk = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kj = sub + 8 * j, kp = k0 + kj;
      float sc = s[j] * a.scale;
      bool ok = qi < nq && kj < nk;
      if (ok) {
        if (a.mask)
          sc += a.mask[(int64_t)(q0 + qi) * a.k_len + kp];
        else
          ok = kp <= a.q_offset + q0 + qi;
      }
      s[j] = ok ? sc : -INFINITY;
      m_blk = fmaxf(m_blk, s[j]);
    }
    m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 1, 64));
    m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 2, 64));
    m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 4, 64));
    const float m_new = fmaxf(m_run, m_blk); // m_run is finite, so m_new is
    const float alpha = expf(m_run - m_new);
    float l_blk = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float p = expf(s[j] - m_new);
      p_s[qi][sub + 8 * j] = p;
      l_blk += p;
    }
    l_blk += __shfl_xor(l_blk, 1, 64);
    l_blk += __shfl_xor(l_blk, 2, 64);
    l_blk += __shfl_xor(l_blk, 4, 64);
    l_run = l_run * alpha + l_blk;
    m_run = m_new;
    __syncthreads(); // p_s complete
    // acc[d] for d = sub*16 .. +16
#pragma unroll
    for (int d = 0; d < 16; ++d)
      acc[d] *= alpha;
    for (int kj = 0; kj < nk; ++kj) {
      const float p = p_s[qi][kj];
#pragma unroll
      for (int d = 0; d < 16; d += 4) {
        const float4 vv = *reinterpret_cast<const float4 *>(&v_s[kj][sub * 16 + d]);
        acc[d] = fmaf(vv.x, p, acc[d]);
        acc[d + 1] = fmaf(vv.y, p, acc[d + 1]);
        acc[d + 2] = fmaf(vv.z, p, acc[d + 2]);
        acc[d + 3] = fmaf(vv.w, p, acc[d + 3]);
      }
    }
  }
  if (qi < nq) {
    float *o = a.out + (int64_t)(q0 + qi) * a.o_stride + (int64_t)h * a.o_hstride + sub * 16;
#pragma unroll
    for (int d = 0; d < 16; d += 4)
      *reinterpret_cast<float4 *>(o + d) =
          make_float4(acc[d] / l_run, acc[d + 1] / l_run, acc[d + 2] / l_run,
                      acc[d + 3] / l_run);
  }
}

// One workgroup per token: rotate q in place, rotate k into the cache, copy v.
__global__ void __launch_bounds__(256)
rope_kv_write_kernel(float *qkv, int64_t row_stride, const float *inv_freq,
                     float *kcache, float *vcache, int heads, int kv_heads,
                     int max_len, int start_pos) {
  __shared__ float cs[kD / 2], sn[kD / 2];
  const int t = blockIdx.x, pos = start_pos + t;
  if (threadIdx.x < kD / 2) {
    float s, c;
    sincosf(inv_freq[threadIdx.x] * (float)pos, &s, &c);
    cs[threadIdx.x] = c;
    sn[threadIdx.x] = s;
  }
  __syncthreads();
  float *row = qkv + (int64_t)t * row_stride;
  const int half = kD / 2;
  for (int i = threadIdx.x; i < (heads + kv_heads) * half; i += 256) {
    const int hh = i / half, j = i % half;
    float *v = row + (int64_t)hh * kD; // q heads first, then k heads
    const float lo = v[j], hi = v[j + half];
    const float nlo = lo * cs[j] + (-hi) * sn[j];
    const float nhi = hi * cs[j] + lo * sn[j];
    if (hh < heads) {
      v[j] = nlo;
      v[j + half] = nhi;
    } else {
      float *dst = kcache + ((int64_t)(hh - heads) * max_len + pos) * kD;
      dst[j] = nlo;
      dst[j + half] = nhi;
    }
  }
  const float *vsrc = row + (int64_t)(heads + kv_heads) * kD;
  for (int i = threadIdx.x; i < kv_heads * kD; i += 256)
    vcache[((int64_t)(i / kD) * max_len + pos) * kD + i % kD] = vsrc[i];
}

} // namespace

int launch_attn_prefill(const AttnPrefillArgs &in, hipStream_t stream) {
  BH_REQUIRE(in.q && in.k && in.v && in.out, "attn_prefill: null pointer");
  BH_REQUIRE(in.head_dim == kD, "attn_prefill: head_dim %d (only %d is built)",
             in.head_dim, kD);
  BH_REQUIRE(in.kv_heads > 0 && in.heads % in.kv_heads == 0,
             "attn_prefill: heads=%d kv_heads=%d", in.heads, in.kv_heads);
  BH_REQUIRE(in.q_len > 0 && in.k_len > 0 && in.kv_stride >= in.k_len,
             "attn_prefill: q_len=%d k_len=%d kv_stride=%lld", in.q_len, in.k_len,
             (long long)in.kv_stride);
  BH_REQUIRE(in.q_stride >= kD && in.o_stride >= kD && in.q_hstride >= kD &&
                 in.o_hstride >= kD && in.q_stride % 4 == 0 && in.o_stride % 4 == 0 &&
                 in.q_hstride % 4 == 0 && in.o_hstride % 4 == 0,
             "attn_prefill: bad strides");
  PrefillArgs a;
  a.q = in.q;
  a.k = in.k;
  a.v = in.v;
  a.mask = in.mask;
  a.out = in.out;
  a.q_stride = in.q_stride;
  a.q_hstride = in.q_hstride;
  a.o_stride = in.o_stride;
  a.o_hstride = in.o_hstride;
  a.kv_stride = in.kv_stride;
  a.heads = in.heads;
  a.group = in.heads / in.kv_heads;
  a.q_len = in.q_len;
  a.k_len = in.k_len;
  a.q_offset = in.k_len - in.q_len; // the last query sees every key
  a.scale = in.scale;
  hipLaunchKernelGGL(attn_prefill_kernel, dim3((unsigned)ceil_div(in.q_len, TQ), in.heads),
                     dim3(256), 0, stream, a);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_rope_kv_write(float *qkv, int64_t row_stride, const float *inv_freq,
                         float *kcache, float *vcache, int heads, int kv_heads,
                         int head_dim, int max_len, int start_pos, int n_tokens,
                         hipStream_t stream) {
  BH_REQUIRE(qkv && inv_freq && kcache && vcache, "rope_kv_write: null pointer");
  BH_REQUIRE(head_dim == kD, "rope_kv_write: head_dim %d", head_dim);
  BH_REQUIRE(n_tokens > 0 && start_pos >= 0 && start_pos + n_tokens <= max_len,
             "rope_kv_write: tokens %d..%d outside the cache (max_len %d)",
             start_pos, start_pos + n_tokens - 1, max_len);
  hipLaunchKernelGGL(rope_kv_write_kernel, dim3(n_tokens), dim3(256), 0, stream,
                     qkv, row_stride, inv_freq, kcache, vcache, heads, kv_heads,
                     max_len, start_pos);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace bh

extern "C" {

int buddy_hip_prefill_attention(const float *q, const float *k, const float *v,
                                const float *mask, float *out, int heads,
                                int kv_heads, int head_dim, int q_len, int k_len,
                                float scale, buddy_hip_stream stream) {
  // the reference operator's layout: [heads, len, head_dim] for q/out,
  // [kv_heads, len, head_dim] for k/v
  bh::AttnPrefillArgs a;
  a.q = q;
  a.k = k;
  a.v = v;
  a.mask = mask;
  a.out = out;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.head_dim = head_dim;
  a.q_len = q_len;
  a.k_len = k_len;
  a.scale = scale;
  a.kv_stride = k_len;
  a.q_stride = head_dim;
  a.q_hstride = (int64_t)q_len * head_dim;
  a.o_stride = head_dim;
  a.o_hstride = (int64_t)q_len * head_dim;
  return bh::launch_attn_prefill(a, bh::as_stream(stream));
}
}
