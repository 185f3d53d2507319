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
// read in place.  The causal structure is exploited: key blocks that lie wholly
// in a query block's future are skipped (they are exactly zero after softmax).
// Arithmetic is f32 throughout, on the f32 matrix cores.
#include "attn.h"

#include <type_traits>

namespace bh {
namespace {

constexpr int kD = 128;
constexpr int kQB = 16;            // query rows per workgroup
constexpr int kKB = 16;            // key positions per step of a wavefront
constexpr int kAttnWaves = 4;      // wavefronts per workgroup; they split the keys
constexpr float kSeedM = -1.0e30f; // tosa.py:4383

typedef float f32x4 __attribute__((ext_vector_type(4)));

struct PrefillArgs {
  const float *q;   // token t, head h at q + t*q_stride + h*q_hstride
  const float *k, *v; // [kv_heads, kv_stride rows, D]
  const float *mask;  // additive [q_len, k_len] or null (causal)
  float *out;         // token t, head h at out + t*o_stride + h*o_hstride
  int64_t q_stride, q_hstride, o_stride, o_hstride, kv_stride;
  int heads, group, q_len, k_len, q_offset; // query i sits at key position q_offset + i
  float scale;
};

// One workgroup: 16 query rows of one head.  Its four wavefronts take the 16-key
// blocks round robin, each with its own running (max, sum, output), and merge
// at the end.  All products run on the f32 matrix cores (16x16x4), operands
// straight from global memory in fragment layout:
//   S^T[key, query] = K . Q^T   (contraction over d; in step 4J + e a lane
//                                supplies d = 16 J + 4 (lane/16) + e, for K and
//                                Q alike: the four lane groups of a load read 64
//                                contiguous bytes of a row, so a K load touches
//                                16 pieces of memory and not 64)
//   O^T[d, query]  += V^T . P^T (contraction over the key; the S^T accumulator
//                                registers ARE the P^T operand of step r: a
//                                lane holds keys 4*(lane/16) + r of query lane%16)
// so the scores never leave the registers between the two products.
__global__ void __launch_bounds__(kAttnWaves *kWave) __attribute__((amdgpu_waves_per_eu(2, 2)))
attn_prefill_kernel(PrefillArgs a) {
  __shared__ float o_s[kAttnWaves][32][kWave];
  __shared__ float m_s[kAttnWaves][kQB], l_s[kAttnWaves][kQB];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // workgroups start in id order: the last query blocks, which see the most
  // keys, come first for every head, the short ones fill the gaps at the end
  const int h = blockIdx.x, kvh = h / a.group;
  const int q0 = ((int)gridDim.y - 1 - (int)blockIdx.y) * kQB;
  const int nq = min(kQB, a.q_len - q0);
  const int qi = lane & 15, lg = lane >> 4; // query of this lane; lane group
  const int qrow = q0 + min(qi, nq - 1);    // rows past the end repeat the last

  // Q^T fragment: qf[4J + e] is d = 16 J + 4 lg + e
  float qf[32];
  {
    const float *src = a.q + (int64_t)qrow * a.q_stride + (int64_t)h * a.q_hstride + lg * 4;
#pragma unroll
    for (int j = 0; j < 32; j += 4) {
      const float4 v = *reinterpret_cast<const float4 *>(src + 4 * j);
      qf[j] = v.x;
      qf[j + 1] = v.y;
      qf[j + 2] = v.z;
      qf[j + 3] = v.w;
    }
  }
  // last key any query of this workgroup may see
  const int k_last = a.mask ? a.k_len - 1
                            : min(a.k_len - 1, a.q_offset + q0 + nq - 1);
  const int nblocks = k_last / kKB + 1;
  const float *kbase = a.k + (int64_t)kvh * a.kv_stride * kD;
  const float *vbase = a.v + (int64_t)kvh * a.kv_stride * kD;

  float m_run = kSeedM, l_run = 0.f; // l_run: this lane's share of the row sum
  f32x4 acc[8]; // O^T: acc[2*e + half][r] is d = 64*half + 4*(4*lg + r) + e
#pragma unroll
  for (int i = 0; i < 8; ++i)
    acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

  // K and V of a key block: 16 loads, issued by hand one block ahead of the
  // block being multiplied (the compiler sinks ordinary loads down to their
  // first use, which leaves the matrix cores waiting out every L2 round trip).
  // A fetch is always exactly 16 loads -- blocks past the end fetch the last
  // block again -- so that vmcnt(16) means "everything but the newest fetch has
  // arrived".  The registers of a fetch are only read after such a wait names
  // them; the build refuses scratch use in this file.
  struct Frag {
    f32x4 k[8], v[8];
  };
  auto issue = [](f32x4 &dst, const float *p) {
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
  };
  auto fetch = [&](int b, Frag &f) {
    const int p0 = min(b, nblocks - 1) * kKB;
    // K fragment: key p0 + lane%16, k[J] is d = 16 J + 4 lg + 0..3
    const float *ks = kbase + (int64_t)min(p0 + qi, a.k_len - 1) * kD + lg * 4;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      issue(f.k[j], ks + 16 * j);
    // V^T fragments: key p0 + 4*lg + r, d = 64*half + 4*(lane%16) + 0..3
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float *vs = vbase + (int64_t)min(p0 + 4 * lg + r, a.k_len - 1) * kD + 4 * qi;
      issue(f.v[2 * r], vs);
      issue(f.v[2 * r + 1], vs + 64);
    }
  };
  auto arrived = [](Frag &f, auto n_in_flight) { // at most N loads still in flight
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(decltype(n_in_flight)::value) : "memory");
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      asm volatile("" : "+v"(f.k[j])::"memory");
      asm volatile("" : "+v"(f.v[j])::"memory");
    }
  };
  auto block = [&](const Frag &f, int b) {
    // ---- S^T block: keys x queries ------------------------------------------
    // four independent partial sums: a matrix instruction that adds to the
    // result of the one before it cannot issue until that one has finished
    f32x4 sp[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      sp[e] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        sp[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.k[j][e], qf[4 * j + e], sp[e], 0, 0, 0);
    const f32x4 st = (sp[0] + sp[1]) + (sp[2] + sp[3]);
    // lane holds keys p0 + 4*lg + r of query q0 + qi
    const int p0 = b * kKB;
    float sc[4];
    float m_blk = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int kp = p0 + 4 * lg + r;
      float v = st[r] * a.scale;
      bool ok = qi < nq && kp < a.k_len;
      if (ok) {
        if (a.mask)
          v += a.mask[(int64_t)(q0 + qi) * a.k_len + kp];
        else
          ok = kp <= a.q_offset + q0 + qi;
      }
      sc[r] = ok ? v : -INFINITY;
      m_blk = fmaxf(m_blk, sc[r]);
    }
    m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 16, 64));
    m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32, 64));
    const float m_new = fmaxf(m_run, m_blk); // m_run is finite, so m_new is
    const float alpha = expf(m_run - m_new);
    float p[4];
    float l_blk = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      p[r] = expf(sc[r] - m_new);
      l_blk += p[r];
    }
    l_run = l_run * alpha + l_blk;
    m_run = m_new;
    // ---- O^T += V^T . P^T -----------------------------------------------------
#pragma unroll
    for (int i = 0; i < 8; ++i)
      acc[i] *= alpha;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const f32x4 vv = f.v[2 * r + half];
        acc[0 + half] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv[0], p[r], acc[0 + half], 0, 0, 0);
        acc[2 + half] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv[1], p[r], acc[2 + half], 0, 0, 0);
        acc[4 + half] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv[2], p[r], acc[4 + half], 0, 0, 0);
        acc[6 + half] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv[3], p[r], acc[6 + half], 0, 0, 0);
      }
    }
  };
  Frag fa, fb;
  fetch(wave, fa);
  for (int b = wave; b < nblocks; b += 2 * kAttnWaves) {
    fetch(b + kAttnWaves, fb);
    arrived(fa, std::integral_constant<int, 16>{});
    block(fa, b);
    fetch(b + 2 * kAttnWaves, fa);
    arrived(fb, std::integral_constant<int, 16>{});
    if (b + kAttnWaves < nblocks)
      block(fb, b + kAttnWaves);
  }
  // the last fetch (a repeated block) may still be in flight: its registers stay
  // allocated until it has landed
  arrived(fa, std::integral_constant<int, 0>{});
  arrived(fb, std::integral_constant<int, 0>{});
  // this wavefront's row sums: the four lane groups hold different keys
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);

  // ---- merge the wavefronts (the reference's combine rule, in wave order) ----
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      o_s[wave][i * 4 + r][lane] = acc[i][r];
  if (lg == 0) {
    m_s[wave][qi] = m_run;
    l_s[wave][qi] = l_run;
  }
  __syncthreads();
  float m_all = m_s[0][qi];
#pragma unroll
  for (int w = 1; w < kAttnWaves; ++w)
    m_all = fmaxf(m_all, m_s[w][qi]);
  float wgt[kAttnWaves], l_all = 0.f;
#pragma unroll
  for (int w = 0; w < kAttnWaves; ++w) {
    wgt[w] = expf(m_s[w][qi] - m_all);
    l_all = fmaf(l_s[w][qi], wgt[w], l_all);
  }
  if (qi >= nq)
    return;
  const float inv = 1.0f / l_all;
  float *o = a.out + (int64_t)(q0 + qi) * a.o_stride + (int64_t)h * a.o_hstride;
  // wavefront w finishes accumulators 2w and 2w+1 (e = w, both halves)
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int i = 2 * wave + half;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < kAttnWaves; ++w)
        sum = fmaf(o_s[w][i * 4 + r][lane], wgt[w], sum);
      o[64 * half + 4 * (4 * lg + r) + wave] = sum * inv;
    }
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

BH_VARIANT_FAMILY(AttnPrefillFamily, "attn_prefill_kernel");

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
  BH_REQUIRE(ceil_div(in.q_len, kQB) <= 65535, "attn_prefill: q_len %d too long", in.q_len);
  BH_NOTE_VARIANT(AttnPrefillFamily);
  hipLaunchKernelGGL(attn_prefill_kernel, dim3(in.heads, (unsigned)ceil_div(in.q_len, kQB)),
                     dim3(kAttnWaves * kWave), 0, stream, a);
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
                                float scale, buddy_hip_stream stream) try {
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
} BH_CATCH_INT("buddy_hip_prefill_attention")
}
