// elementwise.hip -- the small kernels around the matmuls of a decode step:
// embedding gather, greedy argmax, and stand-alone RMSNorm / RoPE / SiLU*mul
// (the decode step itself runs those three fused into the GEMV and attention
// kernels; the stand-alone forms exist for operator-level callers and tests).
//
// Formulas and constants: examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir
// :46-48 (gather), :60-72 (RMSNorm), :51-59,:88-107 (RoPE), :225-232 (SiLU*mul);
// argmax tie rule: runtime/include/buddy/runtime/llm/Sampler.h:101-104.
#include "elementwise.h"

namespace bh {
namespace {

__global__ void __launch_bounds__(256)
embedding_kernel(const float *__restrict__ table, const int *__restrict__ token,
                 int64_t hidden, int64_t vocab, float *__restrict__ out) {
  int64_t t = *token;
  if (t < 0 || t >= vocab)
    t = 0; // an out-of-range id must not read outside the table
  const float *row = table + t * hidden;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < hidden;
       i += (int64_t)gridDim.x * blockDim.x)
    out[i] = row[i];
}

// y = w * (x * rsqrt(sum(x^2) * inv_n + eps)), one workgroup per row
__global__ void __launch_bounds__(256)
rmsnorm_kernel(const float *__restrict__ x, const float *__restrict__ w,
               float *__restrict__ y, int n, float inv_n, float eps) {
  __shared__ float red[4];
  const float *xr = x + (size_t)blockIdx.x * n;
  float *yr = y + (size_t)blockIdx.x * n;
  float s = 0.f;
  for (int i = threadIdx.x; i < n; i += 256)
    s = fmaf(xr[i], xr[i], s);
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0)
    red[threadIdx.x >> 6] = s;
  __syncthreads();
  const float tot = (red[0] + red[1]) + (red[2] + red[3]);
  const float r = 1.0f / sqrtf(tot * inv_n + eps);
  for (int i = threadIdx.x; i < n; i += 256)
    yr[i] = w[i] * (xr[i] * r);
}

// rotate-half RoPE in place on [n_heads, head_dim]
__global__ void __launch_bounds__(256)
rope_kernel(float *__restrict__ x, const float *__restrict__ inv_freq,
            const int *__restrict__ pos_ptr, int n_heads, int head_dim) {
  const int half = head_dim / 2;
  const float p = (float)*pos_ptr;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n_heads * half;
       i += gridDim.x * 256) {
    const int h = i / half, j = i % half;
    const float ang = inv_freq[j] * p;
    const float c = cosf(ang), s = sinf(ang);
    float *v = x + (size_t)h * head_dim;
    const float lo = v[j], hi = v[j + half];
    v[j] = lo * c + (-hi) * s;
    v[j + half] = hi * c + lo * s;
  }
}

__global__ void __launch_bounds__(256)
silu_mul_kernel(const float *__restrict__ g, const float *__restrict__ u,
                float *__restrict__ h, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * 256) {
    const float sig = 1.0f / (1.0f + expf(-g[i]));
    h[i] = (g[i] * sig) * u[i];
  }
}

// (value, index) with "larger value, then smaller index" order = the first
// maximum, like std::max_element
__device__ __forceinline__ void amax_merge(float &v, int &i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) {
    v = ov;
    i = oi;
  }
}

__global__ void __launch_bounds__(256)
argmax_partial_kernel(const float *__restrict__ x, int n,
                      float *__restrict__ pv, int *__restrict__ pi) {
  __shared__ float sv[4];
  __shared__ int si[4];
  float v = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256)
    amax_merge(v, idx, x[i], i);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1)
    amax_merge(v, idx, __shfl_xor(v, o, 64), __shfl_xor(idx, o, 64));
  if ((threadIdx.x & 63) == 0) {
    sv[threadIdx.x >> 6] = v;
    si[threadIdx.x >> 6] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      amax_merge(v, idx, sv[w], si[w]);
    pv[blockIdx.x] = v;
    pi[blockIdx.x] = idx;
  }
}

__global__ void __launch_bounds__(256)
argmax_final_kernel(const float *__restrict__ pv, const int *__restrict__ pi,
                    int nparts, int *__restrict__ out_token,
                    int *__restrict__ token_log, int *__restrict__ step_ptr) {
  __shared__ float sv[4];
  __shared__ int si[4];
  float v = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = threadIdx.x; i < nparts; i += 256)
    amax_merge(v, idx, pv[i], pi[i]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1)
    amax_merge(v, idx, __shfl_xor(v, o, 64), __shfl_xor(idx, o, 64));
  if ((threadIdx.x & 63) == 0) {
    sv[threadIdx.x >> 6] = v;
    si[threadIdx.x >> 6] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      amax_merge(v, idx, sv[w], si[w]);
    if (idx == 0x7fffffff)
      idx = 0; // all NaN / empty: max_element would return begin()
    *out_token = idx;
    if (token_log && step_ptr)
      token_log[*step_ptr] = idx;
  }
}

// Last kernel of a decode step: picks the greedy token from the per-workgroup
// candidates, logs it, advances position and step, then prepares the next step:
// its embedding row and the cos/sin table of its position (shared by every
// layer's attention kernel).  One workgroup.
__global__ void __launch_bounds__(1024)
finish_step_kernel(const float *__restrict__ pv, const int *__restrict__ pi,
                   int nparts, int *__restrict__ state, int *__restrict__ token_log,
                   const float *__restrict__ table, int64_t hidden, int64_t vocab,
                   float *__restrict__ x, const float *__restrict__ inv_freq,
                   int half, float *__restrict__ rope, int advance, int log_cap) {
  __shared__ float sv[16];
  __shared__ int si[16];
  __shared__ int s_tok, s_pos;
  const int threads = blockDim.x; // 256, or 1024 for thousands of candidates
  // token, position and step count: asked for with the first loads, not behind
  // the pick (only thread 0 uses them)
  int st_tok = 0, st_pos = 0, st_step = 0;
  if (threadIdx.x == 0) {
    st_tok = state[0];
    st_pos = state[1];
    st_step = state[2];
  }
  if (nparts > 0) {
    float v = -INFINITY;
    int idx = 0x7fffffff;
    // ten candidates per thread in flight at once: the 9496 group maxima of a
    // 151936-word vocabulary cost 1024 threads one trip to memory, not three
    constexpr int kInFlight = 10;
    for (int i0 = threadIdx.x; i0 < nparts; i0 += kInFlight * threads) {
      float cv[kInFlight];
      int ci[kInFlight];
#pragma unroll
      for (int j = 0; j < kInFlight; ++j) {
        const int i = min(i0 + j * threads, nparts - 1);
        cv[j] = pv[i];
        ci[j] = pi[i];
      }
#pragma unroll
      for (int j = 0; j < kInFlight; ++j)
        if (i0 + j * threads < nparts)
          amax_merge(v, idx, cv[j], ci[j]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
      amax_merge(v, idx, __shfl_xor(v, o, 64), __shfl_xor(idx, o, 64));
    if ((threadIdx.x & 63) == 0) {
      sv[threadIdx.x >> 6] = v;
      si[threadIdx.x >> 6] = idx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int w = 1; w < threads / 64; ++w)
        amax_merge(v, idx, sv[w], si[w]);
      if (idx == 0x7fffffff)
        idx = 0;
      // the host bounds the step count; a counter outside the log writes nothing
      if ((unsigned)st_step < (unsigned)log_cap)
        token_log[st_step] = idx;
      state[0] = idx;
      st_tok = idx;
    }
  }
  if (threadIdx.x == 0) {
    if (advance) {
      st_pos += 1;
      st_step += 1;
      state[1] = st_pos;
      state[2] = st_step;
    }
    s_tok = st_tok;
    s_pos = st_pos;
  }
  __syncthreads();
  int64_t t = s_tok;
  if (t < 0 || t >= vocab)
    t = 0;
  const float *row = table + t * hidden;
  for (int64_t i = threadIdx.x; i < hidden; i += threads)
    x[i] = row[i];
  if (threadIdx.x < half) {
    float sn, cs;
    sincosf(inv_freq[threadIdx.x] * (float)s_pos, &sn, &cs);
    rope[threadIdx.x] = cs;
    rope[half + threadIdx.x] = sn;
  }
}

} // namespace

int launch_finish_step(const float *cand_v, const int *cand_i, int nparts, int *state,
                       int *token_log, const float *table, int64_t hidden, int64_t vocab,
                       float *x, const float *inv_freq, int head_dim, float *rope,
                       bool advance, int token_log_cap, hipStream_t stream) {
  BH_REQUIRE(state && table && x && inv_freq && rope && head_dim > 0 &&
                 head_dim / 2 <= 256 && (nparts == 0 || (cand_v && cand_i && token_log)),
             "finish_step: bad argument");
  hipLaunchKernelGGL(finish_step_kernel, dim3(1), dim3(nparts > 1024 ? 1024 : 256), 0, stream,
                     cand_v, cand_i, nparts, state, token_log, table, hidden, vocab, x,
                     inv_freq, head_dim / 2, rope, advance ? 1 : 0, token_log_cap);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_argmax_partial(const float *x, int n, void *workspace, int *nparts_out,
                          hipStream_t stream) {
  BH_REQUIRE(x && workspace && n > 0, "argmax: bad argument");
  float *pv = static_cast<float *>(workspace);
  int *pi = reinterpret_cast<int *>(pv + kArgmaxParts);
  int parts = (int)ceil_div(n, 1024);
  if (parts > kArgmaxParts)
    parts = kArgmaxParts;
  hipLaunchKernelGGL(argmax_partial_kernel, dim3(parts), dim3(256), 0, stream, x, n, pv, pi);
  BH_CHECK_HIP(hipGetLastError());
  *nparts_out = parts;
  return BUDDY_HIP_OK;
}

int launch_embedding(const float *table, const int *token, int64_t hidden,
                     int64_t vocab, float *out, hipStream_t stream) {
  BH_REQUIRE(table && token && out && hidden > 0 && vocab > 0,
             "embedding: bad argument");
  hipLaunchKernelGGL(embedding_kernel, dim3((unsigned)ceil_div(hidden, 256)),
                     dim3(256), 0, stream, table, token, hidden, vocab, out);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_rmsnorm(const float *x, const float *w, float *y, int rows, int n,
                   float eps, hipStream_t stream) {
  BH_REQUIRE(x && w && y && rows > 0 && n > 0, "rmsnorm: bad argument");
  hipLaunchKernelGGL(rmsnorm_kernel, dim3(rows), dim3(256), 0, stream, x, w, y,
                     n, 1.0f / (float)n, eps);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_rope(float *x, const float *inv_freq, const int *pos, int n_heads,
                int head_dim, hipStream_t stream) {
  BH_REQUIRE(x && inv_freq && pos && n_heads > 0 && head_dim > 0 &&
                 head_dim % 2 == 0,
             "rope: bad argument");
  hipLaunchKernelGGL(rope_kernel,
                     dim3((unsigned)ceil_div((int64_t)n_heads * head_dim / 2, 256)),
                     dim3(256), 0, stream, x, inv_freq, pos, n_heads, head_dim);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

int launch_silu_mul(const float *g, const float *u, float *h, int64_t n,
                    hipStream_t stream) {
  BH_REQUIRE(g && u && h && n > 0, "silu_mul: bad argument");
  int64_t blocks = ceil_div(n, 256);
  if (blocks > 4096)
    blocks = 4096;
  hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     stream, g, u, h, n);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

size_t argmax_workspace_bytes() { return kArgmaxParts * (sizeof(float) + sizeof(int)); }

int launch_argmax(const float *x, int n, void *workspace, int *out_token,
                  int *token_log, int *step_ptr, hipStream_t stream) {
  BH_REQUIRE(x && workspace && out_token && n > 0, "argmax: bad argument");
  float *pv = static_cast<float *>(workspace);
  int *pi = reinterpret_cast<int *>(pv + kArgmaxParts);
  int parts = (int)ceil_div(n, 1024);
  if (parts > kArgmaxParts)
    parts = kArgmaxParts;
  hipLaunchKernelGGL(argmax_partial_kernel, dim3(parts), dim3(256), 0, stream, x,
                     n, pv, pi);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(256), 0, stream, pv, pi,
                     parts, out_token, token_log, step_ptr);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace bh

extern "C" {

int buddy_hip_rmsnorm(const float *x, const float *w, float *y, int rows, int n,
                      float eps, buddy_hip_stream stream) try {
  return bh::launch_rmsnorm(x, w, y, rows, n, eps, bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_rmsnorm")

int buddy_hip_rope(float *x, const float *inv_freq, const int *pos, int n_heads,
                   int head_dim, buddy_hip_stream stream) try {
  return bh::launch_rope(x, inv_freq, pos, n_heads, head_dim,
                         bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_rope")

int buddy_hip_silu_mul(const float *g, const float *u, float *h, int64_t n,
                       buddy_hip_stream stream) try {
  return bh::launch_silu_mul(g, u, h, n, bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_silu_mul")

size_t buddy_hip_argmax_workspace_bytes(void) {
  return bh::argmax_workspace_bytes();
}

int buddy_hip_argmax(const float *x, int n, void *workspace, int *out_index,
                     buddy_hip_stream stream) try {
  return bh::launch_argmax(x, n, workspace, out_index, nullptr, nullptr,
                           bh::as_stream(stream));
} BH_CATCH_INT("buddy_hip_argmax")
}
