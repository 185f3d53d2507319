// ciface_ops.cpp -- operator-level `_mlir_ciface_*` entry points.
//
// Convention followed (runtime/external_kernels/matmul/MatmulTorq.cpp:116-166,
// examples/BuddyOneDNN/onednn_ops.cpp:213-258): arguments are pointers to
// memref descriptors; a result-returning function receives the result
// descriptor uninitialised as its first argument, malloc()s the buffer and
// fills the descriptor; strided inputs are compacted; errors go to stderr and
// the function returns with the result left null.
#include "common.h"
#include "gemm.h"
#include "gemv_w8a32.h"

#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <tuple>
#include <vector>

namespace bh {
namespace {

bool is_device_pointer(const void *p) {
  if (!p)
    return false;
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, p);
  if (e != hipSuccess) {
    (void)hipGetLastError(); // plain host memory: clear the sticky error
    return false;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

struct DeviceBuffer {
  void *ptr = nullptr;
  size_t bytes = 0;
  int reserve(size_t n) {
    if (n <= bytes)
      return BUDDY_HIP_OK;
    if (ptr)
      (void)hipFree(ptr);
    ptr = nullptr;
    bytes = 0;
    BH_CHECK_HIP(hipMalloc(&ptr, n));
    bytes = n;
    return BUDDY_HIP_OK;
  }
};

struct CachedWeight {
  int8_t *packed = nullptr;
  float *scale = nullptr;
  uint64_t fingerprint = 0; // of the caller's W and scale when it was packed
  size_t bytes = 0;         // device bytes held
  uint64_t last_use = 0;    // the context's call counter at the last hit
};

// What the weight cache compares on every hit: up to 64 leading elements of
// four rows of W (first, 1/3, 2/3, last) and the first and last 16 scales,
// folded with the shape.  A buffer that was freed and reused at the same
// address with other contents almost surely differs in one of them; a change
// confined to bytes that are not sampled is not seen (the documented remedy is
// buddy_hip_clear_weight_cache).
constexpr int kFpRowBytes = 64;
constexpr int kFpRows = 4;
constexpr int kFpScales = 16;

struct OpContext {
  std::mutex mu;
  hipStream_t stream = nullptr;
  DeviceBuffer a_buf, c_buf, w_stage;
  std::map<std::tuple<const void *, const void *, int64_t, int64_t>,
           CachedWeight>
      weights;
  size_t cache_bytes = 0;            // sum of the entries' device bytes
  size_t cache_limit = default_cache_limit();
  uint64_t calls = 0, uploads = 0, evictions = 0;
  unsigned char *fp_stage = nullptr; // pinned: samples of device-resident operands

  static size_t default_cache_limit() {
    if (const char *e = std::getenv("BUDDY_HIP_WEIGHT_CACHE_BYTES")) {
      char *end = nullptr;
      const unsigned long long v = std::strtoull(e, &end, 10);
      if (end != e)
        return (size_t)v;
    }
    return (size_t)16 << 30; // a Llama-3-8B-sized int8 model twice over
  }

  int ensure_stream() {
    if (stream)
      return BUDDY_HIP_OK;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n == 0)
      return fail(BUDDY_HIP_ERR_NO_DEVICE, "no HIP device available");
    BH_CHECK_HIP(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    return BUDDY_HIP_OK;
  }
};

OpContext &ctx() {
  static OpContext c;
  return c;
}

template <typename T> const T *data_of(const T *aligned, intptr_t offset) {
  return aligned + offset;
}

// Copies a strided 2-D view into a dense row-major host vector when it is not
// dense already (MatmulTorq.cpp:134-147 does the same for A and B).
template <typename T>
const T *compact_host(const T *src, int64_t rows, int64_t cols, intptr_t s0,
                      intptr_t s1, std::vector<T> &tmp) {
  if (s1 == 1 && s0 == cols)
    return src;
  tmp.resize((size_t)(rows * cols));
  for (int64_t i = 0; i < rows; ++i)
    for (int64_t j = 0; j < cols; ++j)
      tmp[(size_t)(i * cols + j)] = src[i * s0 + j * s1];
  return tmp.data();
}

// Brings a dense [rows, cols] matrix to the device (no copy if it is there).
template <typename T>
int to_device(OpContext &c, const T *src, bool src_on_device, int64_t rows,
              int64_t cols, intptr_t s0, intptr_t s1, DeviceBuffer &buf,
              const T **out) {
  const size_t bytes = sizeof(T) * (size_t)(rows * cols);
  if (src_on_device) {
    if (s1 == 1 && s0 == cols) {
      *out = src;
      return BUDDY_HIP_OK;
    }
    BH_REQUIRE(s1 == 1, "device operand with non-unit inner stride");
    int rc = buf.reserve(bytes);
    if (rc)
      return rc;
    BH_CHECK_HIP(hipMemcpy2DAsync(buf.ptr, sizeof(T) * cols, src,
                                  sizeof(T) * s0, sizeof(T) * cols, rows,
                                  hipMemcpyDeviceToDevice, c.stream));
    *out = static_cast<const T *>(buf.ptr);
    return BUDDY_HIP_OK;
  }
  std::vector<T> tmp;
  const T *dense = compact_host(src, rows, cols, s0, s1, tmp);
  int rc = buf.reserve(bytes);
  if (rc)
    return rc;
  BH_CHECK_HIP(hipMemcpyAsync(buf.ptr, dense, bytes, hipMemcpyHostToDevice,
                              c.stream));
  // the staging vector dies with this scope
  BH_CHECK_HIP(hipStreamSynchronize(c.stream));
  *out = static_cast<const T *>(buf.ptr);
  return BUDDY_HIP_OK;
}

// Packed copy of a dense device matrix and a dense copy of its scales.
int fill_weight(OpContext &c, const int8_t *w_dev, const float *s, intptr_t sstride,
                int64_t K, int64_t N, CachedWeight *cw) {
  BH_CHECK_HIP(hipMalloc((void **)&cw->packed, buddy_hip_w8_packed_bytes(K, N)));
  BH_CHECK_HIP(hipMalloc((void **)&cw->scale, sizeof(float) * (size_t)N));
  int rc = buddy_hip_pack_w8(w_dev, K, N, cw->packed, c.stream);
  if (rc)
    return rc;
  if (is_device_pointer(s)) {
    BH_CHECK_HIP(hipMemcpy2DAsync(cw->scale, sizeof(float), s, sizeof(float) * sstride,
                                  sizeof(float), N, hipMemcpyDeviceToDevice, c.stream));
  } else {
    std::vector<float> dense((size_t)N);
    for (int64_t n = 0; n < N; ++n)
      dense[(size_t)n] = s[n * sstride];
    BH_CHECK_HIP(hipMemcpyAsync(cw->scale, dense.data(), sizeof(float) * N,
                                hipMemcpyHostToDevice, c.stream));
    BH_CHECK_HIP(hipStreamSynchronize(c.stream)); // `dense` dies with this scope
  }
  BH_CHECK_HIP(hipStreamSynchronize(c.stream));
  return BUDDY_HIP_OK;
}

uint64_t fold(uint64_t h, const void *data, size_t n) { // FNV-1a
  const unsigned char *b = static_cast<const unsigned char *>(data);
  for (size_t i = 0; i < n; ++i)
    h = (h ^ b[i]) * 0x100000001b3ull;
  return h;
}

// Fingerprint of the caller's operands as they are now (see kFpRowBytes).
int fingerprint_of(OpContext &c, const int8_t *w, intptr_t ws0, intptr_t ws1, const float *s,
                   intptr_t sstride, int64_t K, int64_t N, uint64_t *out) {
  const int64_t rows[kFpRows] = {0, K / 3, (2 * K) / 3, K - 1};
  const int64_t nb = N < kFpRowBytes ? N : kFpRowBytes;
  const int64_t ns = N < kFpScales ? N : kFpScales;
  int8_t wsample[kFpRows * kFpRowBytes] = {};
  float ssample[2 * kFpScales] = {};
  const bool w_dev = is_device_pointer(w), s_dev = is_device_pointer(s);
  if (w_dev || s_dev) {
    if (!c.fp_stage)
      BH_CHECK_HIP(hipHostMalloc((void **)&c.fp_stage, sizeof(wsample) + sizeof(ssample)));
  }
  if (w_dev) {
    BH_REQUIRE(ws1 == 1, "device operand with non-unit inner stride");
    for (int r = 0; r < kFpRows; ++r)
      BH_CHECK_HIP(hipMemcpyAsync(c.fp_stage + r * kFpRowBytes, w + rows[r] * ws0, (size_t)nb,
                                  hipMemcpyDeviceToHost, c.stream));
  } else {
    for (int r = 0; r < kFpRows; ++r)
      for (int64_t j = 0; j < nb; ++j)
        wsample[r * kFpRowBytes + j] = w[rows[r] * ws0 + j * ws1];
  }
  if (s_dev) {
    float *dst = reinterpret_cast<float *>(c.fp_stage + sizeof(wsample));
    BH_CHECK_HIP(hipMemcpy2DAsync(dst, sizeof(float), s, sizeof(float) * sstride, sizeof(float),
                                  (size_t)ns, hipMemcpyDeviceToHost, c.stream));
    BH_CHECK_HIP(hipMemcpy2DAsync(dst + kFpScales, sizeof(float), s + (N - ns) * sstride,
                                  sizeof(float) * sstride, sizeof(float), (size_t)ns,
                                  hipMemcpyDeviceToHost, c.stream));
  } else {
    for (int64_t j = 0; j < ns; ++j) {
      ssample[j] = s[j * sstride];
      ssample[kFpScales + j] = s[(N - ns + j) * sstride];
    }
  }
  if (w_dev || s_dev) {
    BH_CHECK_HIP(hipStreamSynchronize(c.stream));
    if (w_dev)
      std::memcpy(wsample, c.fp_stage, (size_t)kFpRows * kFpRowBytes);
    if (s_dev)
      std::memcpy(ssample, c.fp_stage + sizeof(wsample), sizeof(ssample));
  }
  uint64_t h = 0xcbf29ce484222325ull;
  h = fold(h, &K, sizeof(K));
  h = fold(h, &N, sizeof(N));
  h = fold(h, wsample, sizeof(wsample));
  h = fold(h, ssample, sizeof(ssample));
  *out = h;
  return BUDDY_HIP_OK;
}

void drop_entry(OpContext &c, CachedWeight &cw) {
  (void)hipFree(cw.packed);
  (void)hipFree(cw.scale);
  c.cache_bytes -= cw.bytes;
}

// Frees least recently used entries until `incoming` more bytes fit under the
// limit (or nothing is left: an entry larger than the limit is still kept for
// the call that needs it and goes first the next time).  The stream is idle:
// every operator call ends with a synchronisation.
void make_room(OpContext &c, size_t incoming) {
  while (!c.weights.empty() && c.cache_bytes + incoming > c.cache_limit) {
    auto oldest = c.weights.begin();
    for (auto it = c.weights.begin(); it != c.weights.end(); ++it)
      if (it->second.last_use < oldest->second.last_use)
        oldest = it;
    drop_entry(c, oldest->second);
    c.weights.erase(oldest);
    ++c.evictions;
  }
}

int get_weight(OpContext &c, buddy_memref_i8_2d *W, buddy_memref_f32_2d *scale,
               int64_t K, int64_t N, CachedWeight *out) {
  const int8_t *w = data_of(W->aligned, W->offset);
  const float *s = data_of(scale->aligned, scale->offset);
  // scale: N values along whichever axis is not 1
  const int64_t sn = (int64_t)scale->sizes[0] * (int64_t)scale->sizes[1];
  BH_REQUIRE(sn == N, "dequant_matmul: scale has %lld values, N=%lld",
             (long long)sn, (long long)N);
  const intptr_t sstride = scale->sizes[1] == N ? scale->strides[1]
                                                : scale->strides[0];
  uint64_t fp = 0;
  int rc = fingerprint_of(c, w, W->strides[0], W->strides[1], s, sstride, K, N, &fp);
  if (rc)
    return rc;
  ++c.calls;
  auto key = std::make_tuple((const void *)w, (const void *)s, K, N);
  auto it = c.weights.find(key);
  if (it != c.weights.end()) {
    if (it->second.fingerprint == fp) {
      it->second.last_use = c.calls;
      *out = it->second;
      return BUDDY_HIP_OK;
    }
    // same addresses, other contents: the buffer was rewritten or reused
    drop_entry(c, it->second);
    c.weights.erase(it);
  }
  CachedWeight cw;
  cw.fingerprint = fp;
  cw.last_use = c.calls;
  cw.bytes = buddy_hip_w8_packed_bytes(K, N) + sizeof(float) * (size_t)N;
  make_room(c, cw.bytes);
  const int8_t *w_dev = nullptr;
  rc = to_device(c, w, is_device_pointer(w), K, N, W->strides[0],
                 W->strides[1], c.w_stage, &w_dev);
  if (rc)
    return rc;
  rc = fill_weight(c, w_dev, s, sstride, K, N, &cw);
  if (rc) { // nothing half-made stays behind
    if (cw.packed)
      (void)hipFree(cw.packed);
    if (cw.scale)
      (void)hipFree(cw.scale);
    return rc;
  }
  c.weights.emplace(key, cw);
  c.cache_bytes += cw.bytes;
  ++c.uploads;
  *out = cw;
  return BUDDY_HIP_OK;
}

// C (host or device, dense rows with stride ldc) <- / += A * dequant(W).
int dequant_matmul(buddy_memref_f32_2d *A, buddy_memref_i8_2d *W,
                   buddy_memref_f32_2d *scale, float *c_host_or_dev,
                   bool c_on_device, int64_t ldc, bool accumulate) {
  OpContext &c = ctx();
  std::lock_guard<std::mutex> lock(c.mu);
  int rc = c.ensure_stream();
  if (rc)
    return rc;
  BH_REQUIRE(A && W && scale && A->aligned && W->aligned && scale->aligned,
             "dequant_matmul: null descriptor or data");
  const int64_t M = A->sizes[0], K = A->sizes[1], N = W->sizes[1];
  BH_REQUIRE(M > 0 && K > 0 && N > 0, "dequant_matmul: empty operand");
  BH_REQUIRE(W->sizes[0] == K, "dequant_matmul: A is [%lld,%lld], W is [%lld,%lld]",
             (long long)M, (long long)K, (long long)W->sizes[0], (long long)N);
  CachedWeight cw;
  rc = get_weight(c, W, scale, K, N, &cw);
  if (rc)
    return rc;
  const float *a = data_of(A->aligned, A->offset);
  const float *a_dev = nullptr;
  rc = to_device(c, a, is_device_pointer(a), M, K, A->strides[0], A->strides[1],
                 c.a_buf, &a_dev);
  if (rc)
    return rc;
  float *c_dev = c_host_or_dev;
  int64_t ldc_dev = ldc;
  if (!c_on_device) {
    rc = c.c_buf.reserve(sizeof(float) * (size_t)(M * N));
    if (rc)
      return rc;
    c_dev = static_cast<float *>(c.c_buf.ptr);
    ldc_dev = N;
    if (accumulate)
      BH_CHECK_HIP(hipMemcpy2DAsync(c_dev, sizeof(float) * N, c_host_or_dev,
                                    sizeof(float) * ldc, sizeof(float) * N, M,
                                    hipMemcpyHostToDevice, c.stream));
  }
  if (M > 16) {
    // a block of rows (the prefill shape): the matrix-core matmul, with every
    // bit of the f32 activations carried (three bf16 terms), so that NaN and
    // infinity propagate as they do in the reference's f32 arithmetic
    GemmW8Args g;
    g.A = a_dev;
    g.lda = K;
    g.W = cw.packed;
    g.scale = cw.scale;
    g.C = c_dev;
    g.ldc = ldc_dev;
    g.M = M;
    g.K = K;
    g.N = N;
    g.accumulate = accumulate;
    g.terms = 3;
    rc = launch_gemm_w8(g, c.stream);
    if (rc)
      return rc;
  }
  for (int64_t m0 = 0; M <= 16 && m0 < M; m0 += 16) {
    GemvArgs g;
    g.A = a_dev + m0 * K;
    g.lda = K;
    g.W0 = cw.packed;
    g.s0 = cw.scale;
    g.C = c_dev + m0 * ldc_dev;
    g.ldc = ldc_dev;
    g.M = (int)(M - m0 < 16 ? M - m0 : 16);
    g.K = K;
    g.N = N;
    g.epilogue = accumulate ? kEpiAccum : kEpiStore;
    rc = launch_gemv(g, c.stream);
    if (rc)
      return rc;
  }
  if (!c_on_device)
    BH_CHECK_HIP(hipMemcpy2DAsync(c_host_or_dev, sizeof(float) * ldc, c_dev,
                                  sizeof(float) * N, sizeof(float) * N, M,
                                  hipMemcpyDeviceToHost, c.stream));
  BH_CHECK_HIP(hipStreamSynchronize(c.stream));
  return BUDDY_HIP_OK;
}

void fill_result(buddy_memref_f32_2d *r, float *data, int64_t M, int64_t N) {
  r->allocated = data;
  r->aligned = data;
  r->offset = 0;
  r->sizes[0] = M;
  r->sizes[1] = N;
  r->strides[0] = N;
  r->strides[1] = 1;
}

} // namespace
} // namespace bh

extern "C" {

void _mlir_ciface_buddy_dequant_matmul_i8_f32(buddy_memref_f32_2d *result,
                                              buddy_memref_f32_2d *A,
                                              buddy_memref_i8_2d *W,
                                              buddy_memref_f32_2d *scale) try {
  if (!result)
    return;
  result->allocated = nullptr;
  result->aligned = nullptr;
  if (!A || !W) {
    bh::fail(BUDDY_HIP_ERR_ARG, "dequant_matmul: null descriptor");
    return;
  }
  const int64_t M = A->sizes[0], N = W->sizes[1];
  if (M <= 0 || N <= 0) {
    bh::fail(BUDDY_HIP_ERR_ARG, "dequant_matmul: empty operand");
    return;
  }
  // freed again unless the product succeeds (also when an exception passes by)
  std::unique_ptr<float, decltype(&free)> out(
      static_cast<float *>(malloc(sizeof(float) * (size_t)(M * N))), &free);
  if (!out) {
    bh::fail(BUDDY_HIP_ERR_HOST, "dequant_matmul: out of host memory");
    return;
  }
  if (bh::dequant_matmul(A, W, scale, out.get(), false, N, false) != BUDDY_HIP_OK)
    return;
  bh::fill_result(result, out.release(), M, N);
} BH_CATCH_VOID("_mlir_ciface_buddy_dequant_matmul_i8_f32")

void _mlir_ciface_buddy_dequant_matmul_i8_f32_acc(buddy_memref_f32_2d *C,
                                                  buddy_memref_f32_2d *A,
                                                  buddy_memref_i8_2d *W,
                                                  buddy_memref_f32_2d *scale) try {
  if (!C || !C->aligned || !A || !W) {
    bh::fail(BUDDY_HIP_ERR_ARG, "dequant_matmul_acc: null descriptor");
    return;
  }
  if (C->strides[1] != 1 || C->sizes[0] != A->sizes[0] ||
      C->sizes[1] != W->sizes[1]) {
    bh::fail(BUDDY_HIP_ERR_ARG,
             "dequant_matmul_acc: C must be [M,N] with unit inner stride");
    return;
  }
  float *c = C->aligned + C->offset;
  (void)bh::dequant_matmul(A, W, scale, c, bh::is_device_pointer(c),
                           C->strides[0], true);
} BH_CATCH_VOID("_mlir_ciface_buddy_dequant_matmul_i8_f32_acc")

void buddy_hip_clear_weight_cache(void) try {
  bh::OpContext &c = bh::ctx();
  std::lock_guard<std::mutex> lock(c.mu);
  if (c.stream)
    (void)hipStreamSynchronize(c.stream);
  for (auto &kv : c.weights)
    bh::drop_entry(c, kv.second);
  c.weights.clear();
} BH_CATCH_VOID("buddy_hip_clear_weight_cache")

void buddy_hip_set_weight_cache_limit(size_t bytes) try {
  bh::OpContext &c = bh::ctx();
  std::lock_guard<std::mutex> lock(c.mu);
  if (c.stream)
    (void)hipStreamSynchronize(c.stream);
  c.cache_limit = bytes;
  bh::make_room(c, 0);
} BH_CATCH_VOID("buddy_hip_set_weight_cache_limit")

void buddy_hip_weight_cache_stats(buddy_hip_weight_cache_info *info) try {
  if (!info)
    return;
  bh::OpContext &c = bh::ctx();
  std::lock_guard<std::mutex> lock(c.mu);
  info->entries = (int64_t)c.weights.size();
  info->bytes = (int64_t)c.cache_bytes;
  info->limit_bytes = (int64_t)c.cache_limit;
  info->uploads = (int64_t)c.uploads;
  info->evictions = (int64_t)c.evictions;
} BH_CATCH_VOID("buddy_hip_weight_cache_stats")
}
