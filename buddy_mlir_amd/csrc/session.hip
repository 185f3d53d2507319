// session.hip -- a Qwen2-shaped int8 (w8a32) decoder resident on one GPU.
//
// Takes the place of the generated ModelSession + compiled forward_decode
// (tools/buddy-codegen/gen_session.py:1381-1452 calling
// _mlir_ciface_forward_decode, whose body is the op sequence of
// examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:46-260,4986-5004) and
// of the greedy part of the decode loop
// (runtime/llm/TextGeneration.cpp:215-266, Sampler.h:101-104).
//
// Weights are repacked once into wave tiles and stay in HBM together with the
// f32 KV cache; a decode step is 5 kernels per layer on one stream:
//   [RMSNorm + q|k|v GEMV] -> [RoPE + KV write + attention partials] ->
//   [fold partials + o_proj GEMV + residual] ->
//   [RMSNorm + gate|up GEMV + SiLU*mul] -> [down GEMV + residual]
// followed by [RMSNorm + lm_head GEMV], a two-stage argmax and a bookkeeping
// kernel.  Token id, position and step counter live in device memory, so the
// whole step is captured once into a hipGraph and replayed; greedy decoding
// feeds the argmax straight into the next step's embedding gather without a
// host round trip.
#include "attn.h"
#include "elementwise.h"
#include "gemm.h"
#include "gemv_w8a32.h"
#include "kv_cache.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <new>
#include <map>
#include <vector>

namespace bh {

// defined in gemv_f32.hip / matmul_f32.hip
int launch_tile_f32(const float *B, int64_t K, int64_t N, int64_t ldb, float *T,
                    hipStream_t stream);
int launch_gemv_f32_tiles(const float *x, const float *T, const float *bias,
                          const float *norm_w, float norm_eps, float *y, int64_t K,
                          int64_t N, bool accumulate, hipStream_t stream);
int launch_gemv_f32(const float *x, const float *B, const float *bias, float *y,
                    int64_t K, int64_t N, int64_t ldb, bool accumulate,
                    hipStream_t stream);
int launch_bias_rows(float *C, const float *bias, int64_t M, int64_t N,
                     hipStream_t stream);
int launch_matmul_f32(const float *A, const float *B, float *C, int64_t M,
                      int64_t N, int64_t K, int64_t lda, int64_t ldb,
                      int64_t ldc, bool accumulate, hipStream_t stream);

namespace {

struct PackedLinear {
  int8_t *w = nullptr; // wave tiles
  float *s = nullptr;  // scales
  float *b = nullptr;  // bias or null
  int64_t K = 0, N = 0;
};

struct Layer {
  float *ln1 = nullptr, *ln2 = nullptr;
  PackedLinear qkv, o, gate, up, down;
  // gate and up share one allocation (up right behind gate): when the
  // intermediate size is a multiple of 16 the two are also one packed matrix of
  // 2 * inter channels, which the prefill multiplies in one launch
  bool gate_up_joint = false;
  // the reference's shipped w8a32 build keeps q/k/v in f32 with a bias
  // (they import as AddMMOp, which the quantizer does not touch):
  float *qkv_f32 = nullptr; // [hidden, q|k|v] dense, or null when int8
  float *qkv_f32_tiles = nullptr; // the same matrix in 1 KiB tiles for the decode GEMV
  float *kc = nullptr, *vc = nullptr; // [kv_heads, max_len, D]
  bool set = false;
};

// x[t, :] = table[token[t], :]
__global__ void __launch_bounds__(256)
embedding_rows_kernel(const float *__restrict__ table, const int *__restrict__ tokens,
                      int64_t hidden, int64_t vocab, float *__restrict__ out) {
  int64_t t = tokens[blockIdx.x];
  if (t < 0 || t >= vocab)
    t = 0;
  const float *row = table + t * hidden;
  float *dst = out + (int64_t)blockIdx.x * hidden;
  for (int64_t i = threadIdx.x; i < hidden; i += 256)
    dst[i] = row[i];
}

} // namespace

struct Session {
  buddy_hip_model_shape shape{};
  hipStream_t stream = nullptr;
  bool own_stream = false;
  std::vector<Layer> layers;
  const float *embed = nullptr; // borrowed: [vocab, hidden] f32
  float *ln_f = nullptr, *inv_freq = nullptr;
  float *rope = nullptr; // [cos | sin] of the step's position
  std::vector<float> inv_freq_host; // for the key re-rotation after a discard
  PackedLinear lm;
  // activations
  float *x = nullptr, *xn = nullptr, *qkv = nullptr, *att = nullptr,
        *h = nullptr, *logits = nullptr;
  void *attn_ws = nullptr, *amax_ws = nullptr;
  float *group_max_v = nullptr; // first maxima of lm_head's channel groups: values,
  int *group_max_i = nullptr;   // indices
  size_t attn_ws_bytes = 0;
  int *state = nullptr;     // device: token, pos, step
  int *token_log = nullptr; // device: greedy tokens by step
  int token_log_cap = 0;
  int *host_state = nullptr; // pinned staging for token/pos/step
  // Host-side mirror of the device's (position, step): what the next enqueued
  // step will use.  -1 until set_state; every step advances both on the device,
  // so the host can refuse steps that would leave the cache or the token log.
  int next_pos = -1, next_step = 0;
  // One captured step per (attention chunk size, chunks covered): the host knows
  // the position of the step it launches and picks the graph.  A cache of up to
  // 1152 positions only ever has one.
  struct StepGraph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
  };
  std::map<std::pair<int, int>, StepGraph> graphs;
  static constexpr size_t kMaxStepGraphs = 8;
  bool use_graph = true;
  std::vector<void *> owned;
  // prefill activations, grown on demand: rows = tokens per prefill call
  int pf_rows = 0;
  float *pf_x = nullptr, *pf_xn = nullptr, *pf_qkv = nullptr, *pf_att = nullptr,
        *pf_g = nullptr, *pf_u = nullptr;
  int *pf_tokens = nullptr;
  float *kv_rows = nullptr; // staging of get_kv_rows, grown on demand
  size_t kv_rows_cap = 0;
  unsigned short *pf_xn_bf = nullptr, *pf_g_bf = nullptr; // bf16 matmul inputs
  unsigned short *pf_att_dg = nullptr; // digit planes of the attention output (o_proj's input)
  int gemm_terms = 3; // bf16 terms per activation in the prefill matmuls (3 = exact)
  int gemm_digits = 3; // int8 digit planes instead of bf16 terms when not 0

  template <typename T> int alloc(T **p, size_t n) {
    void *q = nullptr;
    BH_CHECK_HIP(hipMalloc(&q, n * sizeof(T)));
    owned.push_back(q);
    *p = static_cast<T *>(q);
    return BUDDY_HIP_OK;
  }

  int pack_into(const int8_t *W, const float *scale, const float *bias,
                int64_t K, int64_t N, int8_t *dst_w, float *dst_s, float *dst_b) {
    int rc = buddy_hip_pack_w8(W, K, N, dst_w, stream);
    if (rc)
      return rc;
    BH_CHECK_HIP(hipMemcpyAsync(dst_s, scale, sizeof(float) * N,
                                hipMemcpyDefault, stream));
    if (bias && dst_b)
      BH_CHECK_HIP(hipMemcpyAsync(dst_b, bias, sizeof(float) * N,
                                  hipMemcpyDefault, stream));
    return BUDDY_HIP_OK;
  }

  int make_linear(PackedLinear &L, const int8_t *W, const float *scale,
                  int64_t K, int64_t N) {
    BH_REQUIRE(W && scale, "session: null weight or scale");
    L.K = K;
    L.N = N;
    int rc = alloc(&L.w, buddy_hip_w8_packed_bytes(K, N));
    if (rc)
      return rc;
    rc = alloc(&L.s, (size_t)N);
    if (rc)
      return rc;
    return pack_into(W, scale, nullptr, K, N, L.w, L.s, nullptr);
  }

  void drop_graph() {
    for (auto &kv : graphs) {
      if (kv.second.exec)
        (void)hipGraphExecDestroy(kv.second.exec);
      if (kv.second.graph)
        (void)hipGraphDestroy(kv.second.graph);
    }
    graphs.clear();
  }

  int gemv(const float *A, const PackedLinear &W0, const PackedLinear *W1,
           const float *norm_w, float *C, int epi) {
    GemvArgs g;
    g.A = A;
    g.lda = W0.K;
    g.W0 = W0.w;
    g.s0 = W0.s;
    if (W1) {
      g.W1 = W1->w;
      g.s1 = W1->s;
    }
    g.bias = epi == kEpiStore ? W0.b : nullptr;
    g.norm_w = norm_w;
    g.norm_eps = shape.rms_eps;
    g.norm_inv_k = 1.0f / (float)W0.K;
    g.C = C;
    g.ldc = W0.N;
    g.M = 1;
    g.K = W0.K;
    g.N = W0.N;
    g.epilogue = epi;
    return launch_gemv(g, stream);
  }

  // Enqueues one decode step (reads token/pos from device state) with the cut
  // of the attention the host chose from the position.
  int enqueue_step(const AttnStepPlan &plan) {
    const int attn_chunk = plan.chunk, attn_used = plan.used;
    // x and the RoPE table were prepared by the previous step's last kernel (or
    // by prepare_step after the host set token and position)
    const auto &S = shape;
    int rc;
    const float scale = (float)(1.0 / std::sqrt((double)S.head_dim));
    for (int i = 0; i < S.layers; ++i) {
      Layer &L = layers[(size_t)i];
      if (L.qkv_f32) {
        if ((rc = launch_gemv_f32_tiles(x, L.qkv_f32_tiles, L.qkv.b, L.ln1, S.rms_eps,
                                        qkv, L.qkv.K, L.qkv.N, false, stream)))
          return rc;
      } else if ((rc = gemv(x, L.qkv, nullptr, L.ln1, qkv, kEpiStore))) {
        return rc;
      }
      AttnDecodeArgs a;
      a.qkv = qkv;
      a.inv_freq = inv_freq;
      a.rope_table = rope;
      a.pos_ptr = state + 1;
      a.kcache = L.kc;
      a.vcache = L.vc;
      a.out = att;
      a.heads = S.heads;
      a.kv_heads = S.kv_heads;
      a.head_dim = S.head_dim;
      a.max_len = S.max_len;
      a.scale = scale;
      a.workspace = attn_ws;
      a.workspace_bytes = attn_ws_bytes;
      // o_proj folds the partials while staging its input -- up to the 36 it
      // requests in one trip; far into a long cache (the plan says from where)
      // every one of its workgroups would repeat a fold that outgrows the
      // matrix, and a launch of its own folds them once
      const bool own_fold = plan.own_fold;
      a.combine = own_fold;
      a.wide_combine = own_fold;
      a.chunk = attn_chunk;
      a.chunks_used = attn_used;
      a.head_split = plan.head_split;
      if ((rc = launch_attn_decode(a, stream)))
        return rc;
      if (own_fold) {
        if ((rc = gemv(att, L.o, nullptr, nullptr, x, kEpiAccum)))
          return rc;
      } else {
        const AttnPartials parts =
            attn_partials(attn_ws, S.heads, S.head_dim, S.max_len, attn_chunk);
        GemvArgs g;
        g.attn_acc = parts.acc;
        g.attn_ml = parts.ml;
        g.attn_nchunks = parts.nchunks;
        g.attn_chunk = attn_chunk;
        g.attn_used = attn_used;
        g.head_dim = S.head_dim;
        g.pos_ptr = state + 1;
        g.W0 = L.o.w;
        g.s0 = L.o.s;
        g.C = x;
        g.ldc = L.o.N;
        g.M = 1;
        g.K = L.o.K;
        g.N = L.o.N;
        g.epilogue = kEpiAccum;
        if ((rc = launch_gemv(g, stream)))
          return rc;
      }
      if ((rc = gemv(x, L.gate, &L.up, L.ln2, h, kEpiSiluMul)))
        return rc;
      if ((rc = gemv(h, L.down, nullptr, nullptr, x, kEpiAccum)))
        return rc;
    }
    // lm_head leaves the first maximum of every 16 logits behind where its cut
    // allows it; otherwise a launch of its own scans the row
    int nparts = 0;
    {
      GemvArgs g;
      g.A = x;
      g.lda = lm.K;
      g.W0 = lm.w;
      g.s0 = lm.s;
      g.bias = lm.b;
      g.norm_w = ln_f;
      g.norm_eps = S.rms_eps;
      g.norm_inv_k = 1.0f / (float)lm.K;
      g.C = logits;
      g.ldc = lm.N;
      g.M = 1;
      g.K = lm.K;
      g.N = lm.N;
      g.epilogue = kEpiStore;
      g.argmax_v = group_max_v;
      g.argmax_i = group_max_i;
      g.argmax_groups = &nparts;
      if ((rc = launch_gemv(g, stream)))
        return rc;
    }
    if (nparts > 0)
      return launch_finish_step(group_max_v, group_max_i, nparts, state, token_log, embed,
                                S.hidden, S.vocab, x, inv_freq, S.head_dim, rope, true,
                                token_log_cap, stream);
    if ((rc = launch_argmax_partial(logits, S.vocab, amax_ws, &nparts, stream)))
      return rc;
    const float *pv = static_cast<const float *>(amax_ws);
    return launch_finish_step(pv, reinterpret_cast<const int *>(pv + kArgmaxParts), nparts,
                              state, token_log, embed, S.hidden, S.vocab, x, inv_freq,
                              S.head_dim, rope, true, token_log_cap, stream);
  }

  // After the host wrote token/position: embedding row and RoPE table of the step.
  int prepare_step() {
    const auto &S = shape;
    return launch_finish_step(nullptr, nullptr, 0, state, token_log, embed, S.hidden, S.vocab,
                              x, inv_freq, S.head_dim, rope, false, token_log_cap,
                              stream);
  }

  int ensure_prefill_buffers(int rows) {
    if (rows <= pf_rows)
      return BUDDY_HIP_OK;
    const auto &S = shape;
    const size_t QN = (size_t)S.heads * S.head_dim, KVN = (size_t)S.kv_heads * S.head_dim;
    for (float **p : {&pf_x, &pf_xn, &pf_qkv, &pf_att, &pf_g})
      if (*p) {
        (void)hipFree(*p);
        *p = nullptr;
      }
    if (pf_tokens) {
      (void)hipFree(pf_tokens);
      pf_tokens = nullptr;
    }
    for (unsigned short **p : {&pf_xn_bf, &pf_g_bf, &pf_att_dg})
      if (*p) {
        (void)hipFree(*p);
        *p = nullptr;
      }
    pf_rows = 0;
    BH_CHECK_HIP(hipMalloc((void **)&pf_x, sizeof(float) * rows * S.hidden));
    BH_CHECK_HIP(hipMalloc((void **)&pf_xn, sizeof(float) * rows * S.hidden));
    BH_CHECK_HIP(hipMalloc((void **)&pf_qkv, sizeof(float) * rows * (QN + 2 * KVN)));
    BH_CHECK_HIP(hipMalloc((void **)&pf_att, sizeof(float) * rows * QN));
    // gate | up side by side: rows of 2 * inter floats
    BH_CHECK_HIP(hipMalloc((void **)&pf_g, sizeof(float) * rows * 2 * S.inter));
    pf_u = pf_g + S.inter;
    BH_CHECK_HIP(hipMalloc((void **)&pf_tokens, sizeof(int) * rows));
    // bf16 staging of the matmul inputs that the norm and SiLU kernels write
    // directly (up to three terms)
    const GemmStagingLayout lx = gemm_staging_layout(rows, S.hidden),
                            lg = gemm_staging_layout(rows, S.inter);
    BH_CHECK_HIP(hipMalloc((void **)&pf_xn_bf, std::max(lx.bytes(3), lx.bytes_digits(3))));
    BH_CHECK_HIP(hipMalloc((void **)&pf_g_bf, std::max(lg.bytes(3), lg.bytes_digits(3))));
    BH_CHECK_HIP(hipMalloc((void **)&pf_att_dg, gemm_staging_layout(rows, QN).bytes_digits(3)));
    pf_rows = rows;
    return BUDDY_HIP_OK;
  }

  int gemm(const float *A, const PackedLinear &W, float *C, int64_t M, bool accumulate,
           bool same_input_as_before = false) {
    GemmW8Args g;
    g.A = A;
    g.lda = W.K;
    g.W = W.w;
    g.scale = W.s;
    g.bias = accumulate ? nullptr : W.b;
    g.C = C;
    g.ldc = W.N;
    g.M = M;
    g.K = W.K;
    g.N = W.N;
    g.accumulate = accumulate;
    g.terms = gemm_terms;
    g.digits = gemm_digits;
    g.reuse_staged_a = same_input_as_before;
    return launch_gemm_w8(g, stream);
  }
  // the same with the input already staged as bf16 terms
  int gemm_staged(const unsigned short *staged, const PackedLinear &W, float *C, int64_t M,
                  bool accumulate, int64_t ldc = 0, const float *then_norm_w = nullptr,
                  void *then_norm_staged = nullptr) {
    GemmW8Args g;
    g.then_norm_w = then_norm_w;
    g.then_norm_eps = shape.rms_eps;
    g.then_norm_staged = then_norm_staged;
    g.staged = staged;
    g.W = W.w;
    g.scale = W.s;
    g.bias = accumulate ? nullptr : W.b;
    g.C = C;
    g.ldc = ldc ? ldc : W.N;
    g.M = M;
    g.K = W.K;
    g.N = W.N;
    g.accumulate = accumulate;
    g.terms = gemm_terms;
    g.digits = gemm_digits;
    return launch_gemm_w8(g, stream);
  }
  // RMSNorm rows / SiLU(g) * u written straight into the matmul's input format
  int norm_to_staging(const float *x, const float *w, int rows, unsigned short *staged) {
    const auto &S = shape;
    if (gemm_digits)
      return launch_rmsnorm_to_digits(x, S.hidden, w, rows, S.hidden, S.rms_eps, gemm_digits,
                                      staged, stream);
    return launch_rmsnorm_to_staging(x, w, rows, S.hidden, S.rms_eps, gemm_terms, staged,
                                     stream);
  }
  int silu_mul_to_staging(const float *g, const float *u, int rows, unsigned short *staged) {
    const auto &S = shape;
    if (gemm_digits)
      return launch_silu_mul_to_digits(g, u, 2 * (int64_t)S.inter, rows, S.inter, gemm_digits,
                                       staged, stream);
    return launch_silu_mul_to_staging(g, u, 2 * (int64_t)S.inter, rows, S.inter, gemm_terms,
                                      staged, stream);
  }

  // Prompt processing for tokens already in pf_tokens: fills cache rows
  // start_pos .. start_pos+n-1 and leaves the final hidden states in pf_x
  // (op order of a layer: subgraph0_decode_simplify.mlir:60-232 over n rows).
  int enqueue_prefill(int n, int start_pos) {
    const auto &S = shape;
    const int64_t QKV = (int64_t)(S.heads + 2 * S.kv_heads) * S.head_dim;
    const float scale = (float)(1.0 / std::sqrt((double)S.head_dim));
    hipLaunchKernelGGL(embedding_rows_kernel, dim3(n), dim3(256), 0, stream, embed,
                       pf_tokens, (int64_t)S.hidden, (int64_t)S.vocab, pf_x);
    BH_CHECK_HIP(hipGetLastError());
    int rc;
    bool normed_ahead = false; // pf_xn_bf already holds this layer's normed input
    for (int i = 0; i < S.layers; ++i) {
      Layer &L = layers[(size_t)i];
      if (L.qkv_f32) {
        if ((rc = launch_rmsnorm(pf_x, L.ln1, pf_xn, n, S.hidden, S.rms_eps, stream)))
          return rc;
        if ((rc = launch_bias_rows(pf_qkv, L.qkv.b, n, L.qkv.N, stream)))
          return rc;
        if ((rc = launch_matmul_f32(pf_xn, L.qkv_f32, pf_qkv, n, L.qkv.N, L.qkv.K,
                                    L.qkv.K, L.qkv.N, L.qkv.N, true, stream)))
          return rc;
      } else {
        // the norm writes the matmul's input format directly (digit planes: the
        // previous layer's down matmul already has)
        if (!normed_ahead && (rc = norm_to_staging(pf_x, L.ln1, n, pf_xn_bf)))
          return rc;
        normed_ahead = false;
        if ((rc = gemm_staged(pf_xn_bf, L.qkv, pf_qkv, n, false)))
          return rc;
      }
      if ((rc = launch_rope_kv_write(pf_qkv, QKV, inv_freq, L.kc, L.vc, S.heads,
                                     S.kv_heads, S.head_dim, S.max_len, start_pos,
                                     n, stream)))
        return rc;
      AttnPrefillArgs a;
      a.q = pf_qkv;
      a.q_stride = QKV;
      a.q_hstride = S.head_dim;
      a.k = L.kc;
      a.v = L.vc;
      a.kv_stride = S.max_len;
      a.out = pf_att;
      a.o_stride = (int64_t)S.heads * S.head_dim;
      a.o_hstride = S.head_dim;
      a.heads = S.heads;
      a.kv_heads = S.kv_heads;
      a.head_dim = S.head_dim;
      a.q_len = n;
      a.k_len = start_pos + n;
      a.scale = scale;
      if ((rc = launch_attn_prefill(a, stream)))
        return rc;
      if (gemm_digits) {
        // o_proj's finished rows go on as the normed input of gate and up: where
        // the matmul splits K over workgroups, the kernel that adds the slices
        // holds whole rows and writes those digit planes itself
        if ((rc = launch_activations_to_digits(pf_att, (int64_t)S.heads * S.head_dim, n,
                                               (int64_t)S.heads * S.head_dim, gemm_digits,
                                               pf_att_dg, stream)))
          return rc;
        if ((rc = gemm_staged(reinterpret_cast<const unsigned short *>(pf_att_dg), L.o, pf_x, n,
                              true, 0, L.ln2, pf_xn_bf)))
          return rc;
      } else {
        if ((rc = gemm(pf_att, L.o, pf_x, n, true)))
          return rc;
        if ((rc = norm_to_staging(pf_x, L.ln2, n, pf_xn_bf)))
          return rc;
      }
      const int64_t ld_gu = 2 * (int64_t)S.inter;
      if (L.gate_up_joint && gemm_digits) {
        // gate and up in one launch whose workgroups hold matching tiles of
        // both: SiLU(gate) * up leaves the matmul, and one pass turns it into
        // the digit planes of down's input
        GemmW8Args g;
        g.staged = pf_xn_bf;
        g.W = L.gate.w;
        g.scale = L.gate.s;
        g.C = pf_g;
        g.ldc = S.inter;
        g.M = n;
        g.K = L.gate.K;
        g.N = 2 * L.gate.N;
        g.digits = gemm_digits;
        g.silu_pair = true;
        if ((rc = launch_gemm_w8(g, stream)))
          return rc;
        if ((rc = launch_activations_to_digits(pf_g, S.inter, n, S.inter, gemm_digits, pf_g_bf,
                                               stream)))
          return rc;
        // down's finished rows go on as the next layer's normed q|k|v input
        const Layer *nx = i + 1 < S.layers ? &layers[(size_t)i + 1] : nullptr;
        const bool ahead = nx && !nx->qkv_f32;
        if ((rc = gemm_staged(pf_g_bf, L.down, pf_x, n, true, 0, ahead ? nx->ln1 : nullptr,
                              ahead ? pf_xn_bf : nullptr)))
          return rc;
        normed_ahead = ahead;
        continue;
      }
      if (L.gate_up_joint) {
        // gate | up as one matrix of 2 * inter channels: one launch, whose second
        // round of tiles starts while the first one drains
        PackedLinear both = L.gate;
        both.N = 2 * L.gate.N;
        if ((rc = gemm_staged(pf_xn_bf, both, pf_g, n, false, ld_gu)))
          return rc;
      } else {
        if ((rc = gemm_staged(pf_xn_bf, L.gate, pf_g, n, false, ld_gu)))
          return rc;
        if ((rc = gemm_staged(pf_xn_bf, L.up, pf_u, n, false, ld_gu)))
          return rc;
      }
      if ((rc = silu_mul_to_staging(pf_g, pf_u, n, pf_g_bf)))
        return rc;
      if ((rc = gemm_staged(pf_g_bf, L.down, pf_x, n, true)))
        return rc;
    }
    return BUDDY_HIP_OK;
  }

  int ready() const {
    if (!embed || !ln_f || !lm.w)
      return fail(BUDDY_HIP_ERR_ARG, "session: embedding / head not set");
    for (size_t i = 0; i < layers.size(); ++i)
      if (!layers[i].set)
        return fail(BUDDY_HIP_ERR_ARG, "session: layer %zu not set", i);
    return BUDDY_HIP_OK;
  }

  // The position and step the device holds must stay inside the cache and the
  // token log for every one of `steps` further steps.
  int check_steps(int steps, const char *who) const {
    BH_REQUIRE(next_pos >= 0, "%s: no token / position set (set_state first)", who);
    BH_REQUIRE(steps > 0 && (int64_t)next_pos + steps <= shape.max_len,
               "%s: %d step(s) from position %d leave the cache (max_len %d)", who, steps,
               next_pos, shape.max_len);
    BH_REQUIRE((int64_t)next_step + steps <= token_log_cap,
               "%s: %d step(s) from step %d overflow the token log (%d entries)", who,
               steps, next_step, token_log_cap);
    return BUDDY_HIP_OK;
  }

  int run_step() {
    int rc = check_steps(1, "decode step");
    if (rc)
      return rc;
    const AttnStepPlan plan = attn_step_plan(next_pos, shape.max_len, shape.kv_heads);
    if (!use_graph) {
      rc = enqueue_step(plan);
    } else {
      // one captured step per cut of the attention; positions only move forward,
      // so a session far into a long cache keeps the last few and lets the rest go
      const std::pair<int, int> key{plan.chunk * 4 + plan.head_split,
                                    plan.own_fold ? -plan.used : plan.used};
      auto it = graphs.find(key);
      if (it == graphs.end()) {
        if (graphs.size() >= kMaxStepGraphs) {
          BH_CHECK_HIP(hipStreamSynchronize(stream)); // a replay may still be running
          drop_graph();
        }
        it = graphs.emplace(key, StepGraph{}).first;
      }
      StepGraph &g = it->second;
      if (!g.exec) {
        BH_CHECK_HIP(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
        rc = enqueue_step(plan);
        hipError_t e = hipStreamEndCapture(stream, &g.graph);
        if (!rc && e != hipSuccess)
          rc = fail(BUDDY_HIP_ERR_HIP, "hipStreamEndCapture: %s", hipGetErrorString(e));
        if (!rc && (e = hipGraphInstantiate(&g.exec, g.graph, nullptr, nullptr, 0)) != hipSuccess)
          rc = fail(BUDDY_HIP_ERR_HIP, "hipGraphInstantiate: %s", hipGetErrorString(e));
        if (rc) {
          drop_graph(); // a half-built graph is not kept
          return rc;
        }
      }
      BH_CHECK_HIP(hipGraphLaunch(g.exec, stream));
    }
    if (!rc) {
      ++next_pos;
      ++next_step;
    }
    return rc;
  }

  // The captured step has kernel arguments baked in (weight, cache and embedding
  // pointers): whoever may change one of them drops the graph first, and the
  // next step captures a new one.
  int invalidate_graph() {
    if (!graphs.empty()) {
      BH_CHECK_HIP(hipStreamSynchronize(stream));
      drop_graph();
    }
    return BUDDY_HIP_OK;
  }

  int set_state(int token, int pos, int step) {
    next_pos = pos;
    next_step = step;
    host_state[0] = token;
    host_state[1] = pos;
    host_state[2] = step;
    BH_CHECK_HIP(hipMemcpyAsync(state, host_state, 3 * sizeof(int),
                                hipMemcpyHostToDevice, stream));
    int rc = prepare_step();
    if (rc)
      return rc;
    // the pinned staging words are reused by the next call
    BH_CHECK_HIP(hipStreamSynchronize(stream));
    return BUDDY_HIP_OK;
  }
};

} // namespace bh

using bh::Session;

extern "C" {

buddy_hip_session *buddy_hip_session_create(const buddy_hip_model_shape *shape,
                                            buddy_hip_stream stream) try {
  if (!shape) {
    bh::fail(BUDDY_HIP_ERR_ARG, "session_create: null shape");
    return nullptr;
  }
  const auto &S = *shape;
  if (S.layers <= 0 || S.hidden <= 0 || S.heads <= 0 || S.kv_heads <= 0 ||
      S.head_dim != 128 || S.inter <= 0 || S.vocab <= 0 || S.max_len <= 0 ||
      S.heads % S.kv_heads != 0 || S.heads / S.kv_heads > 8) {
    bh::fail(BUDDY_HIP_ERR_ARG,
             "session_create: unsupported shape (head_dim must be 128, at most "
             "8 query heads per KV head)");
    return nullptr;
  }
  if (buddy_hip_device_count() == 0) {
    bh::fail(BUDDY_HIP_ERR_NO_DEVICE, "session_create: no HIP device");
    return nullptr;
  }
  if (S.max_len > bh::kAttnWideChunks * 256) {
    bh::fail(BUDDY_HIP_ERR_ARG, "session_create: max_len %d above %d positions", S.max_len,
             bh::kAttnWideChunks * 256);
    return nullptr;
  }
  Session *s = new (std::nothrow) Session();
  if (!s)
    return nullptr;
  s->shape = S;
  s->stream = bh::as_stream(stream);
  if (!s->stream) {
    if (hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking) != hipSuccess) {
      bh::fail(BUDDY_HIP_ERR_HIP, "session_create: cannot create a stream");
      delete s;
      return nullptr;
    }
    s->own_stream = true;
  }
  s->layers.resize((size_t)S.layers);
  const size_t QN = (size_t)S.heads * S.head_dim, KVN = (size_t)S.kv_heads * S.head_dim;
  int rc = 0;
  rc |= s->alloc(&s->x, (size_t)S.hidden);
  rc |= s->alloc(&s->xn, (size_t)S.hidden);
  rc |= s->alloc(&s->qkv, QN + 2 * KVN);
  rc |= s->alloc(&s->att, QN);
  rc |= s->alloc(&s->h, (size_t)S.inter);
  rc |= s->alloc(&s->logits, (size_t)S.vocab);
  rc |= s->alloc(&s->ln_f, (size_t)S.hidden);
  rc |= s->alloc(&s->inv_freq, (size_t)S.head_dim / 2);
  rc |= s->alloc(&s->rope, (size_t)S.head_dim);
  rc |= s->alloc(&s->state, 4);
  s->token_log_cap = 65536;
  rc |= s->alloc(&s->token_log, (size_t)s->token_log_cap);
  s->attn_ws_bytes = bh::attn_decode_workspace_bytes(S.heads, S.max_len);
  rc |= s->alloc((char **)&s->attn_ws, s->attn_ws_bytes);
  rc |= s->alloc((char **)&s->amax_ws, bh::argmax_workspace_bytes());
  {
    const size_t groups = (size_t)bh::ceil_div(S.vocab, bh::kTileN);
    rc |= s->alloc(&s->group_max_v, groups);
    rc |= s->alloc(&s->group_max_i, groups);
  }
  for (auto &L : s->layers) {
    rc |= s->alloc(&L.kc, KVN * (size_t)S.max_len);
    rc |= s->alloc(&L.vc, KVN * (size_t)S.max_len);
    rc |= s->alloc(&L.ln1, (size_t)S.hidden);
    rc |= s->alloc(&L.ln2, (size_t)S.hidden);
  }
  if (!rc && hipHostMalloc((void **)&s->host_state, 4 * sizeof(int)) != hipSuccess)
    rc = bh::fail(BUDDY_HIP_ERR_HIP, "session_create: pinned alloc failed");
  if (!rc) {
    for (auto &L : s->layers) {
      if (hipMemsetAsync(L.kc, 0, sizeof(float) * KVN * S.max_len, s->stream) != hipSuccess ||
          hipMemsetAsync(L.vc, 0, sizeof(float) * KVN * S.max_len, s->stream) != hipSuccess)
        rc = bh::fail(BUDDY_HIP_ERR_HIP, "session_create: cache clear failed");
    }
    if (hipMemsetAsync(s->state, 0, 4 * sizeof(int), s->stream) != hipSuccess)
      rc = BUDDY_HIP_ERR_HIP;
    (void)hipStreamSynchronize(s->stream);
  }
  if (rc) {
    buddy_hip_session_destroy(reinterpret_cast<buddy_hip_session *>(s));
    return nullptr;
  }
  return reinterpret_cast<buddy_hip_session *>(s);
} BH_CATCH_NULL("buddy_hip_session_create")

void buddy_hip_session_destroy(buddy_hip_session *hs) try {
  Session *s = reinterpret_cast<Session *>(hs);
  if (!s)
    return;
  if (s->stream)
    (void)hipStreamSynchronize(s->stream);
  s->drop_graph();
  for (void *p : s->owned)
    (void)hipFree(p);
  for (void *p : {(void *)s->pf_x, (void *)s->pf_xn, (void *)s->pf_qkv, (void *)s->pf_att,
                  (void *)s->pf_g, (void *)s->pf_tokens, (void *)s->kv_rows,
                  (void *)s->pf_xn_bf, (void *)s->pf_g_bf, (void *)s->pf_att_dg})
    if (p)
      (void)hipFree(p);
  if (s->host_state)
    (void)hipHostFree(s->host_state);
  bh::release_gemm_staging(s->stream);
  if (s->own_stream)
    (void)hipStreamDestroy(s->stream);
  delete s;
} BH_CATCH_VOID("buddy_hip_session_destroy")

int buddy_hip_session_set_globals(buddy_hip_session *hs, const float *embed,
                                  const float *inv_freq, const float *ln_f,
                                  const int8_t *w_lm, const float *s_lm) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s && embed && inv_freq && ln_f && w_lm && s_lm,
             "session_set_globals: null argument");
  const auto &S = s->shape;
  int rc0 = s->invalidate_graph(); // the embedding pointer is baked into it
  if (rc0)
    return rc0;
  s->embed = embed;
  BH_CHECK_HIP(hipMemcpyAsync(s->inv_freq, inv_freq, sizeof(float) * S.head_dim / 2,
                              hipMemcpyDefault, s->stream));
  s->inv_freq_host.resize((size_t)S.head_dim / 2);
  BH_CHECK_HIP(hipMemcpyAsync(s->inv_freq_host.data(), inv_freq,
                              sizeof(float) * S.head_dim / 2, hipMemcpyDefault,
                              s->stream));
  BH_CHECK_HIP(hipMemcpyAsync(s->ln_f, ln_f, sizeof(float) * S.hidden,
                              hipMemcpyDefault, s->stream));
  if (!s->lm.w) {
    int rc = s->make_linear(s->lm, w_lm, s_lm, S.hidden, S.vocab);
    if (rc)
      return rc;
  } else {
    int rc = s->pack_into(w_lm, s_lm, nullptr, S.hidden, S.vocab, s->lm.w,
                          s->lm.s, nullptr);
    if (rc)
      return rc;
  }
  BH_CHECK_HIP(hipStreamSynchronize(s->stream));
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_set_globals")

int buddy_hip_session_set_layer(buddy_hip_session *hs, int index,
                                const buddy_hip_layer_weights *w) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s && w, "session_set_layer: null argument");
  const auto &S = s->shape;
  BH_REQUIRE(index >= 0 && index < S.layers, "session_set_layer: index %d", index);
  const bool f32_qkv = w->fq != nullptr;
  BH_REQUIRE(w->ln1 && w->ln2 && w->wo && w->wg && w->wu && w->wd && w->so &&
                 w->sg && w->su && w->sd,
             "session_set_layer: null weight");
  BH_REQUIRE(f32_qkv ? (w->fk && w->fv && w->bq && !w->wq && !w->wk && !w->wv)
                     : (w->wq && w->wk && w->wv && w->sq && w->sk && w->sv &&
                        !w->fk && !w->fv),
             "session_set_layer: q/k/v must be all int8 (+scales) or all f32 "
             "(+biases)");
  BH_REQUIRE((w->bq != nullptr) == (w->bk != nullptr) &&
                 (w->bq != nullptr) == (w->bv != nullptr),
             "session_set_layer: q/k/v biases must come together");
  bh::Layer &L = s->layers[(size_t)index];
  const int64_t H = S.hidden, QN = (int64_t)S.heads * S.head_dim,
                KVN = (int64_t)S.kv_heads * S.head_dim, I = S.inter;
  int rc = s->invalidate_graph();
  if (rc)
    return rc;
  if (!L.set) {
    // q|k|v share one packed matrix: channel groups are independent, so the
    // three packed blocks simply follow each other
    L.qkv.K = H;
    L.qkv.N = QN + 2 * KVN;
    if (f32_qkv) {
      rc |= s->alloc(&L.qkv_f32, (size_t)H * L.qkv.N);
      rc |= s->alloc(&L.qkv_f32_tiles, buddy_hip_f32_tiles_bytes(H, L.qkv.N) / sizeof(float));
    } else {
      rc |= s->alloc(&L.qkv.w, buddy_hip_w8_packed_bytes(H, L.qkv.N));
      rc |= s->alloc(&L.qkv.s, (size_t)L.qkv.N);
    }
    if (w->bq)
      rc |= s->alloc(&L.qkv.b, (size_t)L.qkv.N);
    L.o.K = QN; L.o.N = H;
    L.gate.K = H; L.gate.N = I;
    L.up.K = H; L.up.N = I;
    L.down.K = I; L.down.N = H;
    for (bh::PackedLinear *P : {&L.o, &L.down}) {
      rc |= s->alloc(&P->w, buddy_hip_w8_packed_bytes(P->K, P->N));
      rc |= s->alloc(&P->s, (size_t)P->N);
    }
    const size_t gate_bytes = buddy_hip_w8_packed_bytes(H, I);
    rc |= s->alloc(&L.gate.w, 2 * gate_bytes);
    rc |= s->alloc(&L.gate.s, (size_t)(2 * I));
    if (!rc) {
      L.up.w = L.gate.w + gate_bytes;
      L.up.s = L.gate.s + I;
      L.gate_up_joint = I % bh::kTileN == 0; // no padding channels between the two
    }
    if (rc)
      return rc;
  }
  BH_REQUIRE(QN % 16 == 0 && KVN % 16 == 0, "session_set_layer: head sizes");
  const size_t kp = (size_t)bh::round_up(H, bh::kTileK);
  BH_REQUIRE(f32_qkv == (L.qkv_f32 != nullptr),
             "session_set_layer: layer %d was created with the other q/k/v type", index);
  if (f32_qkv) {
    // [H, QN] | [H, KVN] | [H, KVN] side by side in one [H, QN + 2 KVN] matrix
    const size_t ld = (size_t)L.qkv.N * sizeof(float);
    BH_CHECK_HIP(hipMemcpy2DAsync(L.qkv_f32, ld, w->fq, QN * sizeof(float),
                                  QN * sizeof(float), H, hipMemcpyDefault, s->stream));
    BH_CHECK_HIP(hipMemcpy2DAsync(L.qkv_f32 + QN, ld, w->fk, KVN * sizeof(float),
                                  KVN * sizeof(float), H, hipMemcpyDefault, s->stream));
    BH_CHECK_HIP(hipMemcpy2DAsync(L.qkv_f32 + QN + KVN, ld, w->fv, KVN * sizeof(float),
                                  KVN * sizeof(float), H, hipMemcpyDefault, s->stream));
    if ((rc = bh::launch_tile_f32(L.qkv_f32, H, L.qkv.N, L.qkv.N, L.qkv_f32_tiles, s->stream)))
      return rc;
    BH_CHECK_HIP(hipMemcpyAsync(L.qkv.b, w->bq, QN * sizeof(float), hipMemcpyDefault, s->stream));
    BH_CHECK_HIP(hipMemcpyAsync(L.qkv.b + QN, w->bk, KVN * sizeof(float), hipMemcpyDefault, s->stream));
    BH_CHECK_HIP(hipMemcpyAsync(L.qkv.b + QN + KVN, w->bv, KVN * sizeof(float), hipMemcpyDefault, s->stream));
  } else {
    rc |= s->pack_into(w->wq, w->sq, w->bq, H, QN, L.qkv.w, L.qkv.s, L.qkv.b);
    rc |= s->pack_into(w->wk, w->sk, w->bk, H, KVN, L.qkv.w + kp * QN,
                       L.qkv.s + QN, L.qkv.b ? L.qkv.b + QN : nullptr);
    rc |= s->pack_into(w->wv, w->sv, w->bv, H, KVN, L.qkv.w + kp * (QN + KVN),
                       L.qkv.s + QN + KVN, L.qkv.b ? L.qkv.b + QN + KVN : nullptr);
  }
  rc |= s->pack_into(w->wo, w->so, nullptr, QN, H, L.o.w, L.o.s, nullptr);
  rc |= s->pack_into(w->wg, w->sg, nullptr, H, I, L.gate.w, L.gate.s, nullptr);
  rc |= s->pack_into(w->wu, w->su, nullptr, H, I, L.up.w, L.up.s, nullptr);
  rc |= s->pack_into(w->wd, w->sd, nullptr, I, H, L.down.w, L.down.s, nullptr);
  if (rc)
    return rc;
  BH_CHECK_HIP(hipMemcpyAsync(L.ln1, w->ln1, sizeof(float) * H, hipMemcpyDefault, s->stream));
  BH_CHECK_HIP(hipMemcpyAsync(L.ln2, w->ln2, sizeof(float) * H, hipMemcpyDefault, s->stream));
  BH_CHECK_HIP(hipStreamSynchronize(s->stream));
  L.set = true;
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_set_layer")

int buddy_hip_session_set_kv(buddy_hip_session *hs, int kv_index,
                             const float *src) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s && src, "session_set_kv: null argument");
  const auto &S = s->shape;
  BH_REQUIRE(kv_index >= 0 && kv_index < 2 * S.layers, "session_set_kv: index %d",
             kv_index);
  bh::Layer &L = s->layers[(size_t)(kv_index / 2)];
  float *dst = (kv_index & 1) ? L.vc : L.kc; // even = K, odd = V
  BH_CHECK_HIP(hipMemcpyAsync(dst, src,
                              sizeof(float) * (size_t)S.kv_heads * S.max_len * S.head_dim,
                              hipMemcpyDefault, s->stream));
  BH_CHECK_HIP(hipStreamSynchronize(s->stream));
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_set_kv")

int buddy_hip_session_get_kv(buddy_hip_session *hs, int kv_index, float *dst) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s && dst, "session_get_kv: null argument");
  const auto &S = s->shape;
  BH_REQUIRE(kv_index >= 0 && kv_index < 2 * S.layers, "session_get_kv: index %d",
             kv_index);
  bh::Layer &L = s->layers[(size_t)(kv_index / 2)];
  const float *src = (kv_index & 1) ? L.vc : L.kc;
  BH_CHECK_HIP(hipMemcpyAsync(dst, src,
                              sizeof(float) * (size_t)S.kv_heads * S.max_len * S.head_dim,
                              hipMemcpyDefault, s->stream));
  BH_CHECK_HIP(hipStreamSynchronize(s->stream));
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_get_kv")

int buddy_hip_session_get_kv_rows(buddy_hip_session *hs, int row0, int rows,
                                  float *dst) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s && dst, "session_get_kv_rows: null argument");
  const auto &S = s->shape;
  BH_REQUIRE(row0 >= 0 && rows > 0 && (int64_t)row0 + rows <= S.max_len,
             "session_get_kv_rows: rows %d..%d outside the cache (max_len %d)", row0,
             row0 + rows - 1, S.max_len);
  const size_t n = (size_t)2 * S.layers * S.kv_heads * rows * S.head_dim;
  if (n > s->kv_rows_cap) {
    BH_CHECK_HIP(hipStreamSynchronize(s->stream));
    if (s->kv_rows)
      (void)hipFree(s->kv_rows);
    s->kv_rows = nullptr;
    s->kv_rows_cap = 0;
    BH_CHECK_HIP(hipMalloc((void **)&s->kv_rows, sizeof(float) * n));
    s->kv_rows_cap = n;
  }
  std::vector<const float *> tensors;
  for (auto &L : s->layers) {
    tensors.push_back(L.kc);
    tensors.push_back(L.vc);
  }
  int rc = bh::launch_kv_gather_rows(tensors.data(), (int)tensors.size(), S.kv_heads,
                                     S.max_len, S.head_dim, row0, rows, s->kv_rows,
                                     s->stream);
  if (rc)
    return rc;
  BH_CHECK_HIP(hipMemcpyAsync(dst, s->kv_rows, sizeof(float) * n, hipMemcpyDefault,
                              s->stream));
  BH_CHECK_HIP(hipStreamSynchronize(s->stream));
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_get_kv_rows")

int buddy_hip_session_use_graph(buddy_hip_session *hs, int enable) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s, "session_use_graph: null session");
  s->use_graph = enable != 0;
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_use_graph")

int buddy_hip_session_decode_mirror(buddy_hip_session *hs, int token, int pos,
                                    float *logits_out, float *kv_rows_out,
                                    int *next_token) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s, "session_decode: null session");
  int rc = s->ready();
  if (rc)
    return rc;
  BH_REQUIRE(token >= 0 && token < s->shape.vocab, "session_decode: token %d", token);
  BH_REQUIRE(pos >= 0 && pos < s->shape.max_len,
             "session_decode: position %d outside the cache (max_len %d)", pos,
             s->shape.max_len);
  if ((rc = s->set_state(token, pos, 0)))
    return rc;
  if ((rc = s->run_step()))
    return rc;
  if (logits_out)
    BH_CHECK_HIP(hipMemcpyAsync(logits_out, s->logits,
                                sizeof(float) * s->shape.vocab, hipMemcpyDefault,
                                s->stream));
  BH_CHECK_HIP(hipMemcpyAsync(s->host_state, s->state, 3 * sizeof(int),
                              hipMemcpyDeviceToHost, s->stream));
  if (kv_rows_out) { // the cache rows this step wrote, all layers
    if ((rc = buddy_hip_session_get_kv_rows(hs, pos, 1, kv_rows_out)))
      return rc;
  }
  BH_CHECK_HIP(hipStreamSynchronize(s->stream));
  if (next_token)
    *next_token = s->host_state[0];
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_decode_mirror")

int buddy_hip_session_decode(buddy_hip_session *hs, int token, int pos,
                             float *logits_out, int *next_token) {
  return buddy_hip_session_decode_mirror(hs, token, pos, logits_out, nullptr, next_token);
}

int buddy_hip_session_decode_greedy(buddy_hip_session *hs, int first_token,
                                    int start_pos, int steps, int *tokens_out) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s && tokens_out, "session_decode_greedy: null argument");
  int rc = s->ready();
  if (rc)
    return rc;
  BH_REQUIRE(first_token >= 0 && first_token < s->shape.vocab,
             "session_decode_greedy: token %d", first_token);
  BH_REQUIRE(steps > 0 && steps <= s->token_log_cap,
             "session_decode_greedy: steps %d", steps);
  BH_REQUIRE(start_pos >= 0 && start_pos + steps <= s->shape.max_len,
             "session_decode_greedy: positions %d..%d outside the cache (max_len %d)",
             start_pos, start_pos + steps - 1, s->shape.max_len);
  if ((rc = s->set_state(first_token, start_pos, 0)))
    return rc;
  for (int i = 0; i < steps; ++i)
    if ((rc = s->run_step()))
      return rc;
  BH_CHECK_HIP(hipMemcpyAsync(tokens_out, s->token_log, sizeof(int) * steps,
                              hipMemcpyDefault, s->stream));
  BH_CHECK_HIP(hipStreamSynchronize(s->stream));
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_decode_greedy")

int buddy_hip_session_prefill(buddy_hip_session *hs, const int *tokens,
                              int n_tokens, int start_pos, float *logits_out,
                              int *next_token) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s && tokens, "session_prefill: null argument");
  int rc = s->ready();
  if (rc)
    return rc;
  const auto &S = s->shape;
  BH_REQUIRE(n_tokens > 0 && start_pos >= 0 && start_pos + n_tokens <= S.max_len,
             "session_prefill: tokens %d..%d outside the cache (max_len %d)",
             start_pos, start_pos + n_tokens - 1, S.max_len);
  if ((rc = s->ensure_prefill_buffers(n_tokens)))
    return rc;
  BH_CHECK_HIP(hipMemcpyAsync(s->pf_tokens, tokens, sizeof(int) * n_tokens,
                              hipMemcpyDefault, s->stream));
  if ((rc = s->enqueue_prefill(n_tokens, start_pos)))
    return rc;
  // logits of the last prompt token only: RMSNorm + lm_head as in a decode step
  {
    bh::GemvArgs g;
    g.A = s->pf_x + (size_t)(n_tokens - 1) * S.hidden;
    g.lda = S.hidden;
    g.W0 = s->lm.w;
    g.s0 = s->lm.s;
    g.norm_w = s->ln_f;
    g.norm_eps = S.rms_eps;
    g.norm_inv_k = 1.0f / (float)S.hidden;
    g.C = s->logits;
    g.ldc = S.vocab;
    g.M = 1;
    g.K = S.hidden;
    g.N = S.vocab;
    g.epilogue = bh::kEpiStore;
    if ((rc = bh::launch_gemv(g, s->stream)))
      return rc;
  }
  if ((rc = bh::launch_argmax(s->logits, S.vocab, s->amax_ws, s->state, nullptr,
                              nullptr, s->stream)))
    return rc;
  if (logits_out)
    BH_CHECK_HIP(hipMemcpyAsync(logits_out, s->logits, sizeof(float) * S.vocab,
                                hipMemcpyDefault, s->stream));
  BH_CHECK_HIP(hipMemcpyAsync(s->host_state, s->state, sizeof(int),
                              hipMemcpyDeviceToHost, s->stream));
  BH_CHECK_HIP(hipStreamSynchronize(s->stream));
  if (next_token)
    *next_token = s->host_state[0];
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_prefill")

int buddy_hip_session_prefill_all_logits(buddy_hip_session *hs, const int *tokens,
                                         int n_tokens, int start_pos,
                                         float *logits_out) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s && tokens && logits_out, "session_prefill_all_logits: null argument");
  int rc = s->ready();
  if (rc)
    return rc;
  const auto &S = s->shape;
  BH_REQUIRE(n_tokens > 0 && start_pos >= 0 && start_pos + n_tokens <= S.max_len,
             "session_prefill_all_logits: tokens %d..%d outside the cache (max_len %d)",
             start_pos, start_pos + n_tokens - 1, S.max_len);
  if ((rc = s->ensure_prefill_buffers(n_tokens)))
    return rc;
  BH_CHECK_HIP(hipMemcpyAsync(s->pf_tokens, tokens, sizeof(int) * n_tokens,
                              hipMemcpyDefault, s->stream));
  if ((rc = s->enqueue_prefill(n_tokens, start_pos)))
    return rc;
  if ((rc = bh::launch_rmsnorm(s->pf_x, s->ln_f, s->pf_xn, n_tokens, S.hidden,
                               S.rms_eps, s->stream)))
    return rc;
  float *dev_logits = nullptr;
  BH_CHECK_HIP(hipMalloc((void **)&dev_logits, sizeof(float) * (size_t)n_tokens * S.vocab));
  rc = s->gemm(s->pf_xn, s->lm, dev_logits, n_tokens, false);
  if (!rc && hipMemcpyAsync(logits_out, dev_logits, sizeof(float) * (size_t)n_tokens * S.vocab,
                            hipMemcpyDefault, s->stream) != hipSuccess)
    rc = bh::fail(BUDDY_HIP_ERR_HIP, "session_prefill_all_logits: copy failed");
  (void)hipStreamSynchronize(s->stream);
  (void)hipFree(dev_logits);
  return rc;
} BH_CATCH_INT("buddy_hip_session_prefill_all_logits")

void buddy_hip_session_adopt(buddy_hip_session *hs, void *device_ptr) try {
  Session *s = reinterpret_cast<Session *>(hs);
  if (s && device_ptr)
    s->owned.push_back(device_ptr);
} BH_CATCH_VOID("buddy_hip_session_adopt")

int buddy_hip_session_set_prefill_precision(buddy_hip_session *hs, int mode) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s, "session_set_prefill_precision: null session");
  BH_REQUIRE(mode >= 0 && mode <= 3, "session_set_prefill_precision: mode %d outside 0..3",
             mode);
  s->gemm_terms = mode == 1 ? 3 : 1;
  s->gemm_digits = mode == 2 ? 3 : mode == 3 ? 2 : 0;
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_set_prefill_precision")

int buddy_hip_session_enqueue_steps(buddy_hip_session *hs, int steps) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s && steps > 0, "session_enqueue_steps: bad argument");
  int rc = s->ready();
  if (rc)
    return rc;
  // refused as a whole: no step is enqueued when the last one would not fit
  if ((rc = s->check_steps(steps, "session_enqueue_steps")))
    return rc;
  for (int i = 0; i < steps; ++i)
    if ((rc = s->run_step()))
      return rc;
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_enqueue_steps")

int buddy_hip_session_set_state(buddy_hip_session *hs, int token, int pos) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s, "session_set_state: null session");
  BH_REQUIRE(token >= 0 && token < s->shape.vocab && pos >= 0 &&
                 pos < s->shape.max_len,
             "session_set_state: token %d / position %d out of range", token, pos);
  int rc = s->ready();
  if (rc)
    return rc;
  return s->set_state(token, pos, 0);
} BH_CATCH_INT("buddy_hip_session_set_state")

const float *buddy_hip_session_logits(buddy_hip_session *hs) {
  Session *s = reinterpret_cast<Session *>(hs);
  return s ? s->logits : nullptr;
}

int buddy_hip_session_discard_kv_freqs(buddy_hip_session *hs, int keep, int discard,
                                       int count, const float *inv_freq) try {
  Session *s = reinterpret_cast<Session *>(hs);
  BH_REQUIRE(s, "session_discard_kv: null session");
  int rc = s->ready();
  if (rc)
    return rc;
  const auto &S = s->shape;
  std::vector<float *> tensors;
  for (auto &L : s->layers) {
    tensors.push_back(L.kc);
    tensors.push_back(L.vc);
  }
  rc = bh::launch_kv_discard(tensors.data(), (int)tensors.size(), S.kv_heads, S.max_len,
                             S.head_dim, keep, discard, count,
                             inv_freq ? inv_freq : s->inv_freq_host.data(), s->stream);
  if (rc)
    return rc;
  BH_CHECK_HIP(hipStreamSynchronize(s->stream));
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_session_discard_kv_freqs")

int buddy_hip_session_discard_kv(buddy_hip_session *hs, int keep, int discard,
                                 int count) try {
  return buddy_hip_session_discard_kv_freqs(hs, keep, discard, count, nullptr);
} BH_CATCH_INT("buddy_hip_session_discard_kv")

int buddy_hip_session_vocab(buddy_hip_session *hs) try {
  Session *s = reinterpret_cast<Session *>(hs);
  return s ? s->shape.vocab : 0;
} BH_CATCH_INT("buddy_hip_session_vocab")

buddy_hip_stream buddy_hip_session_stream(buddy_hip_session *hs) {
  Session *s = reinterpret_cast<Session *>(hs);
  return s ? reinterpret_cast<buddy_hip_stream>(s->stream) : nullptr;
}
}
