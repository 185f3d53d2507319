// ciface_model.cpp -- `_mlir_ciface_forward_prefill` / `_mlir_ciface_forward_decode`
// with the argument lists the generated ModelSession binds with dlsym
// (tools/buddy-codegen/gen_session.py:974-1007, 1127-1143), for the
// DeepSeek-R1-Distill-Qwen-1.5B w8a32 package the reference ships
// (models/deepseek_r1/specs/w8a32.json; examples/BuddyDeepSeekR1/
// buddy-deepseek-r1-w8a32-main.cpp:32-39).
//
// The caller keeps weights and KV cache in host memory.  On the first call the
// two weight blobs are cut into tensors, uploaded and repacked into a resident
// device session keyed by the blob addresses (weights are immutable after
// loadWeights, gen_session.py:1301-1331); after that a decode call moves one
// token id in and one row of logits out.  The KV cache lives on the device;
// result descriptors for the KV tensors alias the caller's own buffers, which
// the caller recognises and neither copies nor frees
// (gen_session.py:1421-1442).
//
// Layout of the blobs (order of the parameters inside arg0-w8a32-f32.data /
// arg0-w8a32-i8.data): taken from the argument list of
// examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:4 (embed, inv_freq,
// then per layer ln1, q_bias, q_w, k_bias, k_w, v_bias, v_w, o_w, ln2, gate, up,
// down, finally the last norm and lm_head), split by dtype with the scalers
// appended after all original f32 parameters in weight order
// (frontend/Python/graph/transform/quantization/quantize.py:561-590).  The
// element counts this gives are exactly the reference's constants
// F32ParamsSize = 322338752 and I8ParamsSize = 1455489024; the order itself has
// not been checked against a blob written by the reference importer.
#include "common.h"

#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <vector>

namespace bh {
namespace {

constexpr int kLayers = 28; // fixed by the argument list of the generated ABI

struct ModelState {
  std::mutex mu;
  buddy_hip_session *sess = nullptr;
  const void *f32_key = nullptr, *i8_key = nullptr;
  buddy_hip_model_shape shape{};
  float *dev_f32 = nullptr; // the f32 blob on the device (embedding is borrowed)
  float *pinned_logits = nullptr; // [vocab]: the logits row lands here first
  float *pinned_rows = nullptr;   // [2 * layers, kv_heads, head_dim]: a step's new cache rows
  bool kv_on_device = false;
  // The position the next decode call is expected to carry when the caller just
  // goes on generating; -1: any (after a prefill, whose prompt length only the
  // caller knows, and after a device-side discard).  A call with another
  // position means the caller edited its host tensors (the generated
  // ModelSession::handleKVCacheOverflow shifts and re-rotates them and lowers
  // its position, gen_session.py:1471-1511): the device cache is then reloaded
  // from them.
  long long expected_pos = -1;
  // Set by a device-side discard (buddy_hip_forward_discard_kv): the caller's
  // tensors were not shifted, so from then on only the device cache is whole
  // and a decode at any position keeps it.  Cleared by invalidate_kv, reset
  // and a prefill.
  bool device_is_truth = false;
};

// malloc'd host memory that is freed unless handed over
struct HostBuf {
  void *p = nullptr;
  explicit HostBuf(size_t bytes) : p(malloc(bytes)) {}
  HostBuf(const HostBuf &) = delete;
  HostBuf &operator=(const HostBuf &) = delete;
  ~HostBuf() { free(p); }
  template <typename T> T *as() const { return static_cast<T *>(p); }
  template <typename T> T *release() {
    T *q = static_cast<T *>(p);
    p = nullptr;
    return q;
  }
};

ModelState &state() {
  static ModelState s;
  return s;
}

buddy_hip_model_shape default_shape(int kv_heads, int max_len, int head_dim) {
  buddy_hip_model_shape s{};
  s.layers = kLayers;
  s.hidden = 1536;
  s.heads = 12;
  s.kv_heads = kv_heads;
  s.head_dim = head_dim;
  s.inter = 8960;
  s.vocab = 151936;
  s.max_len = max_len;
  s.rms_eps = 1e-6f;
  return s;
}

// The parameters of the reference's w8a32 package in the order they lie in the
// two blobs, with running element offsets per dtype.
//  * Parameters keep their trace order = the order of the function arguments of
//    examples/BuddyDeepSeekR1/subgraph0_decode_simplify.mlir:4 with the run-time
//    inputs (token, positions, KV caches) left out; packing walks them in that
//    order and advances one running offset per dtype
//    (frontend/Python/graph/graph.py:848-863, 1001-1018).
//  * The weights of plain matmuls (o_proj, gate, up, down, lm_head) are int8,
//    the q/k/v weights, which feed a matmul + bias add, stay f32
//    (frontend/Python/graph/transform/quantization/weight_only_channel_wise.py
//    :366-461).
//  * One f32 scaler vector per int8 weight follows all original parameters, in
//    the order of the weights
//    (frontend/Python/graph/transform/quantization/quantize.py:561-590).
std::vector<buddy_hip_blob_entry> blob_layout(const buddy_hip_model_shape &S) {
  const int64_t H = S.hidden, QN = (int64_t)S.heads * S.head_dim,
                KVN = (int64_t)S.kv_heads * S.head_dim, I = S.inter, V = S.vocab;
  std::vector<buddy_hip_blob_entry> t;
  int64_t off[2] = {0, 0};
  auto add = [&](int param, int layer, int dtype, int64_t rows, int64_t cols) {
    buddy_hip_blob_entry e;
    e.param = param;
    e.layer = layer;
    e.dtype = dtype;
    e.reserved = 0;
    e.rows = rows;
    e.cols = cols;
    e.offset = off[dtype];
    e.count = rows * cols;
    off[dtype] += e.count;
    t.push_back(e);
  };
  constexpr int F = BUDDY_HIP_BLOB_F32, Q = BUDDY_HIP_BLOB_I8;
  add(BUDDY_HIP_PARAM_EMBED, -1, F, V, H);
  add(BUDDY_HIP_PARAM_INV_FREQ, -1, F, 1, S.head_dim / 2);
  for (int l = 0; l < S.layers; ++l) {
    add(BUDDY_HIP_PARAM_LN1, l, F, 1, H);
    add(BUDDY_HIP_PARAM_Q_BIAS, l, F, 1, QN);
    add(BUDDY_HIP_PARAM_Q_W, l, F, H, QN);
    add(BUDDY_HIP_PARAM_K_BIAS, l, F, 1, KVN);
    add(BUDDY_HIP_PARAM_K_W, l, F, H, KVN);
    add(BUDDY_HIP_PARAM_V_BIAS, l, F, 1, KVN);
    add(BUDDY_HIP_PARAM_V_W, l, F, H, KVN);
    add(BUDDY_HIP_PARAM_O_W, l, Q, QN, H);
    add(BUDDY_HIP_PARAM_LN2, l, F, 1, H);
    add(BUDDY_HIP_PARAM_GATE_W, l, Q, H, I);
    add(BUDDY_HIP_PARAM_UP_W, l, Q, H, I);
    add(BUDDY_HIP_PARAM_DOWN_W, l, Q, I, H);
  }
  add(BUDDY_HIP_PARAM_LN_F, -1, F, 1, H);
  add(BUDDY_HIP_PARAM_LM_HEAD_W, -1, Q, H, V);
  for (int l = 0; l < S.layers; ++l) { // scalers, in weight order
    add(BUDDY_HIP_PARAM_O_SCALE, l, F, 1, H);
    add(BUDDY_HIP_PARAM_GATE_SCALE, l, F, 1, I);
    add(BUDDY_HIP_PARAM_UP_SCALE, l, F, 1, I);
    add(BUDDY_HIP_PARAM_DOWN_SCALE, l, F, 1, H);
  }
  add(BUDDY_HIP_PARAM_LM_HEAD_SCALE, -1, F, 1, V);
  return t;
}

struct BlobSizes {
  int64_t f32, i8;
};
BlobSizes blob_sizes(const buddy_hip_model_shape &S) {
  BlobSizes b{0, 0};
  for (const buddy_hip_blob_entry &e : blob_layout(S))
    (e.dtype == BUDDY_HIP_BLOB_F32 ? b.f32 : b.i8) += e.count;
  return b;
}

void destroy_locked(ModelState &m) {
  if (m.sess)
    buddy_hip_session_destroy(m.sess);
  if (m.dev_f32)
    (void)hipFree(m.dev_f32);
  if (m.pinned_logits)
    (void)hipHostFree(m.pinned_logits);
  if (m.pinned_rows)
    (void)hipHostFree(m.pinned_rows);
  m.pinned_rows = nullptr;
  m.expected_pos = -1;
  m.device_is_truth = false;
  m.sess = nullptr;
  m.dev_f32 = nullptr;
  m.pinned_logits = nullptr;
  m.f32_key = m.i8_key = nullptr;
  m.kv_on_device = false;
}

// Builds a resident session from the two host blobs.  *dev_f32_out receives the
// device copy of the f32 blob, which the session borrows the embedding from.
int session_from_blobs(const float *f32, int64_t n_f32, const int8_t *i8,
                       int64_t n_i8, const buddy_hip_model_shape &S,
                       buddy_hip_session **sess_out, float **dev_f32_out) {
  const BlobSizes want = blob_sizes(S);
  BH_REQUIRE(f32 && i8, "w8a32 blobs: null pointer");
  BH_REQUIRE(n_f32 == want.f32 && n_i8 == want.i8,
             "w8a32 blobs hold %lld f32 / %lld int8 elements, this shape needs "
             "%lld / %lld",
             (long long)n_f32, (long long)n_i8, (long long)want.f32,
             (long long)want.i8);
  buddy_hip_session *sess = buddy_hip_session_create(&S, nullptr);
  if (!sess)
    return BUDDY_HIP_ERR_HIP;
  float *dev_f32 = nullptr;
  int8_t *dev_i8 = nullptr;
  auto cleanup = [&](int code) {
    buddy_hip_session_destroy(sess);
    if (dev_f32)
      (void)hipFree(dev_f32);
    if (dev_i8)
      (void)hipFree(dev_i8);
    return code;
  };
  if (hipMalloc((void **)&dev_f32, sizeof(float) * (size_t)n_f32) != hipSuccess ||
      hipMalloc((void **)&dev_i8, (size_t)n_i8) != hipSuccess ||
      hipMemcpy(dev_f32, f32, sizeof(float) * (size_t)n_f32, hipMemcpyDefault) != hipSuccess ||
      hipMemcpy(dev_i8, i8, (size_t)n_i8, hipMemcpyDefault) != hipSuccess)
    return cleanup(fail(BUDDY_HIP_ERR_HIP, "w8a32 blobs: upload failed: %s",
                        hipGetErrorString(hipGetLastError())));

  // cut the blobs into tensors by the one layout table
  const std::vector<buddy_hip_blob_entry> table = blob_layout(S);
  const float *embed = nullptr, *inv_freq = nullptr, *ln_f = nullptr, *s_lm = nullptr;
  const int8_t *w_lm = nullptr;
  std::vector<buddy_hip_layer_weights> lw((size_t)S.layers);
  for (auto &w : lw)
    std::memset(&w, 0, sizeof(w));
  for (const buddy_hip_blob_entry &e : table) {
    const float *pf = dev_f32 + e.offset;
    const int8_t *pi = dev_i8 + e.offset;
    buddy_hip_layer_weights *w = e.layer >= 0 ? &lw[(size_t)e.layer] : nullptr;
    switch (e.param) {
    case BUDDY_HIP_PARAM_EMBED:    embed = pf; break;
    case BUDDY_HIP_PARAM_INV_FREQ: inv_freq = pf; break;
    case BUDDY_HIP_PARAM_LN1:      w->ln1 = pf; break;
    case BUDDY_HIP_PARAM_Q_BIAS:   w->bq = pf; break;
    case BUDDY_HIP_PARAM_Q_W:      w->fq = pf; break;
    case BUDDY_HIP_PARAM_K_BIAS:   w->bk = pf; break;
    case BUDDY_HIP_PARAM_K_W:      w->fk = pf; break;
    case BUDDY_HIP_PARAM_V_BIAS:   w->bv = pf; break;
    case BUDDY_HIP_PARAM_V_W:      w->fv = pf; break;
    case BUDDY_HIP_PARAM_O_W:      w->wo = pi; break;
    case BUDDY_HIP_PARAM_LN2:      w->ln2 = pf; break;
    case BUDDY_HIP_PARAM_GATE_W:   w->wg = pi; break;
    case BUDDY_HIP_PARAM_UP_W:     w->wu = pi; break;
    case BUDDY_HIP_PARAM_DOWN_W:   w->wd = pi; break;
    case BUDDY_HIP_PARAM_LN_F:     ln_f = pf; break;
    case BUDDY_HIP_PARAM_LM_HEAD_W: w_lm = pi; break;
    case BUDDY_HIP_PARAM_O_SCALE:    w->so = pf; break;
    case BUDDY_HIP_PARAM_GATE_SCALE: w->sg = pf; break;
    case BUDDY_HIP_PARAM_UP_SCALE:   w->su = pf; break;
    case BUDDY_HIP_PARAM_DOWN_SCALE: w->sd = pf; break;
    case BUDDY_HIP_PARAM_LM_HEAD_SCALE: s_lm = pf; break;
    default:
      return cleanup(fail(BUDDY_HIP_ERR_ARG, "w8a32 blobs: unknown parameter %d", e.param));
    }
  }
  int rc = buddy_hip_session_set_globals(sess, embed, inv_freq, ln_f, w_lm, s_lm);
  for (int i = 0; !rc && i < S.layers; ++i)
    rc = buddy_hip_session_set_layer(sess, i, &lw[(size_t)i]);
  if (rc)
    return cleanup(rc);
  (void)hipFree(dev_i8); // the int8 weights now live in the session's packed copy
  *sess_out = sess;
  *dev_f32_out = dev_f32;
  return BUDDY_HIP_OK;
}

int build_session(ModelState &m, const float *f32, int64_t n_f32, const int8_t *i8,
                  int64_t n_i8, const buddy_hip_model_shape &S) {
  destroy_locked(m);
  int rc = session_from_blobs(f32, n_f32, i8, n_i8, S, &m.sess, &m.dev_f32);
  if (rc)
    return rc;
  m.shape = S;
  m.f32_key = f32;
  m.i8_key = i8;
  return BUDDY_HIP_OK;
}

struct KVArgs {
  buddy_memref_f32_4d *kv[2 * kLayers];
  buddy_memref_i64_1d *dummy[kLayers - 1];
};

int ensure_session(ModelState &m, buddy_memref_f32_1d *f32, buddy_memref_i8_1d *i8,
                   int kv_heads, int max_len, int head_dim) {
  BH_REQUIRE(f32 && i8 && f32->aligned && i8->aligned, "forward: null weight blob");
  const float *pf = f32->aligned + f32->offset;
  const int8_t *pi = i8->aligned + i8->offset;
  if (m.sess && m.f32_key == pf && m.i8_key == pi && m.shape.max_len == max_len &&
      m.shape.kv_heads == kv_heads)
    return BUDDY_HIP_OK;
  return build_session(m, pf, f32->sizes[0], pi, i8->sizes[0],
                       default_shape(kv_heads, max_len, head_dim));
}

int check_kv(const KVArgs &a, int *kv_heads, int *max_len, int *head_dim) {
  for (int i = 0; i < 2 * kLayers; ++i) {
    const buddy_memref_f32_4d *k = a.kv[i];
    BH_REQUIRE(k && k->aligned, "forward_decode: null KV tensor %d", i);
    BH_REQUIRE(k->sizes[0] == 1 && k->strides[3] == 1 &&
                   k->strides[2] == k->sizes[3] &&
                   k->strides[1] == k->sizes[2] * k->sizes[3],
               "forward_decode: KV tensor %d is not a dense [1,h,len,d] tensor", i);
    BH_REQUIRE(k->sizes[1] == a.kv[0]->sizes[1] && k->sizes[2] == a.kv[0]->sizes[2] &&
                   k->sizes[3] == a.kv[0]->sizes[3],
               "forward_decode: KV tensors differ in shape");
  }
  *kv_heads = (int)a.kv[0]->sizes[1];
  *max_len = (int)a.kv[0]->sizes[2];
  *head_dim = (int)a.kv[0]->sizes[3];
  return BUDDY_HIP_OK;
}

// DecodeABI (gen_session.py:924-932): [pos_out][kv0][kv1]([dummy][kv][kv]) x 27
// [logits {1,1,V}]
struct DecodeResult {
  buddy_memref_i64_1d pos_out;
  buddy_memref_f32_4d kv0, kv1;
  struct {
    buddy_memref_i64_1d dummy;
    buddy_memref_f32_4d k, v;
  } rest[kLayers - 1];
  buddy_memref_f32_3d logits;
};
static_assert(sizeof(DecodeResult) == 40 + 2 * 88 + (kLayers - 1) * (40 + 2 * 88) + 72,
              "DecodeABI layout");

// The result block of the hand-written example program for the same model
// (examples/BuddyDeepSeekR1/buddy-deepseek-r1-w8a32-main.cpp:163-249) keeps the
// 27 position copies together: [pos_out][kv0][kv1][dummy x 27][kv2 .. kv55]
// [logits].  Same members, same size, another order; the caller says which one
// it reads with BUDDY_HIP_DECODE_RESULT_LAYOUT=grouped in the environment.
struct DecodeResultGrouped {
  buddy_memref_i64_1d pos_out;
  buddy_memref_f32_4d kv0, kv1;
  buddy_memref_i64_1d dummy[kLayers - 1];
  buddy_memref_f32_4d kv[2 * (kLayers - 1)];
  buddy_memref_f32_3d logits;
};
static_assert(sizeof(DecodeResultGrouped) == sizeof(DecodeResult), "same members");

bool grouped_result_layout() {
  static const bool v = [] {
    const char *e = getenv("BUDDY_HIP_DECODE_RESULT_LAYOUT");
    return e && std::strcmp(e, "grouped") == 0;
  }();
  return v;
}

// PrefillABI (gen_session.py:908-911): [kv0 .. kv55][logits {1,max_len,V}]
struct PrefillResult {
  buddy_memref_f32_4d kv[2 * kLayers];
  buddy_memref_f32_3d logits;
};
static_assert(sizeof(PrefillResult) == 2 * kLayers * 88 + 72, "PrefillABI layout");

int forward_decode(DecodeResult *res, buddy_memref_f32_1d *f32, buddy_memref_i8_1d *i8,
                   buddy_memref_i64_2d *tok, buddy_memref_i64_1d *pos, const KVArgs &a) {
  ModelState &m = state();
  std::lock_guard<std::mutex> lock(m.mu);
  BH_REQUIRE(res && tok && pos && tok->aligned && pos->aligned,
             "forward_decode: null argument");
  int kv_heads, max_len, head_dim;
  int rc = check_kv(a, &kv_heads, &max_len, &head_dim);
  if (rc)
    return rc;
  if ((rc = ensure_session(m, f32, i8, kv_heads, max_len, head_dim)))
    return rc;
  const long long token = tok->aligned[tok->offset];
  const long long position = pos->aligned[pos->offset];
  BH_REQUIRE(token >= 0 && token < m.shape.vocab && position >= 0 &&
                 position < m.shape.max_len,
             "forward_decode: token %lld / position %lld out of range", token, position);
  // The caller's host tensors and the device cache are kept equal: every step
  // writes its new rows through to the caller's tensors (below), so the caller
  // may edit them between calls.  It has done so when the position is not the
  // one that follows the last step; the device copy is then loaded again.
  if (m.kv_on_device && !m.device_is_truth && m.expected_pos >= 0 &&
      position != m.expected_pos)
    m.kv_on_device = false;
  if (!m.kv_on_device) { // the caller's cache is the truth
    for (int i = 0; i < 2 * kLayers; ++i)
      if ((rc = buddy_hip_session_set_kv(m.sess, i, a.kv[i]->aligned + a.kv[i]->offset)))
        return rc;
    m.kv_on_device = true;
  }
  const int64_t V = m.shape.vocab;
  const size_t row_elems = (size_t)m.shape.kv_heads * m.shape.head_dim;
  // the row crosses PCIe into pinned memory (a copy into pageable memory is
  // staged by the runtime and several times slower) and is handed over in a
  // malloc'd buffer, which is what the caller frees
  if (!m.pinned_logits)
    BH_CHECK_HIP(hipHostMalloc((void **)&m.pinned_logits, sizeof(float) * (size_t)V));
  if (!m.pinned_rows)
    BH_CHECK_HIP(hipHostMalloc((void **)&m.pinned_rows,
                               sizeof(float) * 2 * kLayers * row_elems));
  if ((rc = buddy_hip_session_decode_mirror(m.sess, (int)token, (int)position,
                                            m.pinned_logits, m.pinned_rows, nullptr)))
    return rc;
  m.expected_pos = position + 1;
  // write-through: row `position` of every cache, as the compiled model leaves
  // it in the caller's tensors (index_put, subgraph0_decode_simplify.mlir:108-142)
  for (int i = 0; i < 2 * kLayers; ++i) {
    float *host = a.kv[i]->aligned + a.kv[i]->offset;
    for (int h = 0; h < m.shape.kv_heads; ++h)
      memcpy(host + ((size_t)h * m.shape.max_len + (size_t)position) * m.shape.head_dim,
             m.pinned_rows + ((size_t)i * m.shape.kv_heads + h) * m.shape.head_dim,
             sizeof(float) * m.shape.head_dim);
  }
  HostBuf logits_buf(sizeof(float) * (size_t)V);
  BH_REQUIRE(logits_buf.p, "forward_decode: out of host memory");
  memcpy(logits_buf.p, m.pinned_logits, sizeof(float) * (size_t)V);
  // results: state tensors alias the caller's, logits are handed over.  The
  // descriptors are read before any is written: the caller may pass members of
  // the result block itself as arguments.
  const buddy_memref_i64_1d pos_d = *pos;
  buddy_memref_f32_4d kv_d[2 * kLayers];
  buddy_memref_i64_1d dummy_d[kLayers - 1];
  for (int i = 0; i < 2 * kLayers; ++i)
    kv_d[i] = *a.kv[i];
  for (int i = 0; i < kLayers - 1; ++i)
    dummy_d[i] = *a.dummy[i];
  buddy_memref_f32_3d *lg;
  if (grouped_result_layout()) {
    DecodeResultGrouped *g = reinterpret_cast<DecodeResultGrouped *>(res);
    // that program owns every member of its result block and frees each at
    // exit: the position comes back in a buffer of its own, not as an alias of
    // the caller's cache_position tensor
    long long *own = static_cast<long long *>(malloc(sizeof(long long)));
    if (!own)
      return fail(BUDDY_HIP_ERR_HOST, "forward_decode: out of host memory");
    *own = position;
    g->pos_out = pos_d;
    g->pos_out.allocated = own;
    g->pos_out.aligned = own;
    g->pos_out.offset = 0;
    g->kv0 = kv_d[0];
    g->kv1 = kv_d[1];
    for (int i = 0; i < kLayers - 1; ++i)
      g->dummy[i] = dummy_d[i];
    for (int i = 0; i < 2 * (kLayers - 1); ++i)
      g->kv[i] = kv_d[2 + i];
    lg = &g->logits;
  } else {
    res->pos_out = pos_d;
    res->kv0 = kv_d[0];
    res->kv1 = kv_d[1];
    for (int i = 0; i < kLayers - 1; ++i) {
      res->rest[i].dummy = dummy_d[i];
      res->rest[i].k = kv_d[2 + 2 * i];
      res->rest[i].v = kv_d[3 + 2 * i];
    }
    lg = &res->logits;
  }
  float *logits = logits_buf.release<float>();
  lg->allocated = logits;
  lg->aligned = logits;
  lg->offset = 0;
  lg->sizes[0] = 1;
  lg->sizes[1] = 1;
  lg->sizes[2] = V;
  lg->strides[0] = V;
  lg->strides[1] = V;
  lg->strides[2] = 1;
  return BUDDY_HIP_OK;
}

int forward_prefill(PrefillResult *res, buddy_memref_f32_1d *f32,
                    buddy_memref_i8_1d *i8, buddy_memref_i64_2d *tokens) {
  ModelState &m = state();
  std::lock_guard<std::mutex> lock(m.mu);
  BH_REQUIRE(res && tokens && tokens->aligned, "forward_prefill: null argument");
  const int max_len = (int)tokens->sizes[1];
  BH_REQUIRE(tokens->sizes[0] == 1 && max_len > 0, "forward_prefill: tokens must be [1, max_len]");
  int rc = ensure_session(m, f32, i8, 2, max_len, 128);
  if (rc)
    return rc;
  const auto &S = m.shape;
  std::vector<int> toks((size_t)max_len);
  const long long *src = tokens->aligned + tokens->offset;
  for (int i = 0; i < max_len; ++i) {
    const long long t = src[(int64_t)i * tokens->strides[1]];
    toks[(size_t)i] = (t >= 0 && t < S.vocab) ? (int)t : 0;
  }
  // the compiled graph is static: every one of the max_len rows is processed
  // (rows past the prompt are padding; causality keeps them from mattering)
  const size_t kv_elems = (size_t)S.kv_heads * S.max_len * S.head_dim;
  const size_t logit_elems = (size_t)S.max_len * S.vocab;
  HostBuf logits_buf(sizeof(float) * logit_elems);
  BH_REQUIRE(logits_buf.p, "forward_prefill: out of host memory");
  std::vector<std::unique_ptr<HostBuf>> kvbuf;
  kvbuf.reserve(2 * kLayers);
  if ((rc = buddy_hip_session_prefill_all_logits(m.sess, toks.data(), max_len, 0,
                                                 logits_buf.as<float>())))
    return rc;
  for (int i = 0; i < 2 * kLayers; ++i) {
    kvbuf.emplace_back(new HostBuf(sizeof(float) * kv_elems));
    BH_REQUIRE(kvbuf.back()->p, "forward_prefill: out of host memory");
    if ((rc = buddy_hip_session_get_kv(m.sess, i, kvbuf.back()->as<float>())))
      return rc;
  }
  // nothing below can fail: the buffers now belong to the caller
  float *logits = logits_buf.release<float>();
  m.expected_pos = -1; // the prompt length is the caller's knowledge
  m.device_is_truth = false; // the caller receives the whole cache below
  m.kv_on_device = true;
  for (int i = 0; i < 2 * kLayers; ++i) {
    buddy_memref_f32_4d &d = res->kv[i];
    d.allocated = d.aligned = kvbuf[(size_t)i]->release<float>();
    d.offset = 0;
    d.sizes[0] = 1;
    d.sizes[1] = S.kv_heads;
    d.sizes[2] = S.max_len;
    d.sizes[3] = S.head_dim;
    d.strides[3] = 1;
    d.strides[2] = S.head_dim;
    d.strides[1] = (intptr_t)S.max_len * S.head_dim;
    d.strides[0] = (intptr_t)S.kv_heads * S.max_len * S.head_dim;
  }
  res->logits.allocated = res->logits.aligned = logits;
  res->logits.offset = 0;
  res->logits.sizes[0] = 1;
  res->logits.sizes[1] = S.max_len;
  res->logits.sizes[2] = S.vocab;
  res->logits.strides[2] = 1;
  res->logits.strides[1] = S.vocab;
  res->logits.strides[0] = (intptr_t)S.max_len * S.vocab;
  return BUDDY_HIP_OK;
}

} // namespace
} // namespace bh

#define BH_KV(n) , buddy_memref_f32_4d *k##n, buddy_memref_f32_4d *v##n
#define BH_DKV(n) , buddy_memref_i64_1d *d##n BH_KV(n)
#define BH_PUT(n)                                                              \
  a.kv[2 * n] = k##n;                                                          \
  a.kv[2 * n + 1] = v##n;
#define BH_PUTD(n)                                                             \
  a.dummy[n - 1] = d##n;                                                       \
  BH_PUT(n)

extern "C" {

void _mlir_ciface_forward_decode(
    void *result, buddy_memref_f32_1d *f32_params, buddy_memref_i8_1d *i8_params,
    buddy_memref_i64_2d *token, buddy_memref_i64_1d *cache_position BH_KV(0)
    BH_DKV(1) BH_DKV(2) BH_DKV(3) BH_DKV(4) BH_DKV(5) BH_DKV(6) BH_DKV(7) BH_DKV(8)
    BH_DKV(9) BH_DKV(10) BH_DKV(11) BH_DKV(12) BH_DKV(13) BH_DKV(14) BH_DKV(15)
    BH_DKV(16) BH_DKV(17) BH_DKV(18) BH_DKV(19) BH_DKV(20) BH_DKV(21) BH_DKV(22)
    BH_DKV(23) BH_DKV(24) BH_DKV(25) BH_DKV(26) BH_DKV(27)) try {
  bh::KVArgs a;
  BH_PUT(0)
  BH_PUTD(1) BH_PUTD(2) BH_PUTD(3) BH_PUTD(4) BH_PUTD(5) BH_PUTD(6) BH_PUTD(7)
  BH_PUTD(8) BH_PUTD(9) BH_PUTD(10) BH_PUTD(11) BH_PUTD(12) BH_PUTD(13) BH_PUTD(14)
  BH_PUTD(15) BH_PUTD(16) BH_PUTD(17) BH_PUTD(18) BH_PUTD(19) BH_PUTD(20) BH_PUTD(21)
  BH_PUTD(22) BH_PUTD(23) BH_PUTD(24) BH_PUTD(25) BH_PUTD(26) BH_PUTD(27)
  for (int i = 0; i < bh::kLayers - 1; ++i)
    if (!a.dummy[i]) {
      bh::fail(BUDDY_HIP_ERR_ARG, "forward_decode: null position copy %d", i);
      return;
    }
  (void)bh::forward_decode(static_cast<bh::DecodeResult *>(result), f32_params,
                           i8_params, token, cache_position, a);
} BH_CATCH_VOID("_mlir_ciface_forward_decode")

void _mlir_ciface_forward_prefill(void *result, buddy_memref_f32_1d *f32_params,
                                  buddy_memref_i8_1d *i8_params,
                                  buddy_memref_i64_2d *tokens) try {
  (void)bh::forward_prefill(static_cast<bh::PrefillResult *>(result), f32_params,
                            i8_params, tokens);
} BH_CATCH_VOID("_mlir_ciface_forward_prefill")

buddy_hip_session *buddy_hip_session_create_from_w8a32_blobs(
    const buddy_hip_model_shape *shape, const float *f32_params, int64_t n_f32,
    const int8_t *i8_params, int64_t n_i8) try {
  if (!shape) {
    bh::fail(BUDDY_HIP_ERR_ARG, "create_from_w8a32_blobs: null shape");
    return nullptr;
  }
  buddy_hip_session *sess = nullptr;
  float *dev_f32 = nullptr;
  if (bh::session_from_blobs(f32_params, n_f32, i8_params, n_i8, *shape, &sess, &dev_f32))
    return nullptr;
  buddy_hip_session_adopt(sess, dev_f32); // freed with the session
  return sess;
} BH_CATCH_NULL("buddy_hip_session_create_from_w8a32_blobs")

int64_t buddy_hip_w8a32_blob_layout(const buddy_hip_model_shape *shape,
                                    buddy_hip_blob_entry *entries, int64_t capacity) try {
  if (!shape)
    return 0;
  const std::vector<buddy_hip_blob_entry> t = bh::blob_layout(*shape);
  for (int64_t i = 0; entries && i < capacity && i < (int64_t)t.size(); ++i)
    entries[i] = t[(size_t)i];
  return (int64_t)t.size();
} catch (...) {
  return 0;
}

void buddy_hip_w8a32_blob_sizes(const buddy_hip_model_shape *shape, int64_t *n_f32,
                                int64_t *n_i8) try {
  if (!shape)
    return;
  const bh::BlobSizes b = bh::blob_sizes(*shape);
  if (n_f32)
    *n_f32 = b.f32;
  if (n_i8)
    *n_i8 = b.i8;
} BH_CATCH_VOID("buddy_hip_w8a32_blob_sizes")

void buddy_hip_forward_reset(void) try {
  bh::ModelState &m = bh::state();
  std::lock_guard<std::mutex> lock(m.mu);
  bh::destroy_locked(m);
} BH_CATCH_VOID("buddy_hip_forward_reset")

int buddy_hip_forward_discard_kv(int keep, int discard, int count) try {
  bh::ModelState &m = bh::state();
  std::lock_guard<std::mutex> lock(m.mu);
  if (!m.sess || !m.kv_on_device)
    return bh::fail(BUDDY_HIP_ERR_ARG,
                    "forward_discard_kv: no device-resident KV cache yet");
  int rc = buddy_hip_session_discard_kv(m.sess, keep, discard, count);
  if (!rc) { // the device cache is now ahead of the caller's tensors: never reload
    m.expected_pos = -1;
    m.device_is_truth = true;
  }
  return rc;
} BH_CATCH_INT("buddy_hip_forward_discard_kv")

void buddy_hip_forward_invalidate_kv(void) try {
  bh::ModelState &m = bh::state();
  std::lock_guard<std::mutex> lock(m.mu);
  m.kv_on_device = false;
  m.device_is_truth = false;
  m.expected_pos = -1;
} BH_CATCH_VOID("buddy_hip_forward_invalidate_kv")
}
