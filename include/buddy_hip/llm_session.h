/*
 * llm_session.h -- buddy::runtime::LLMSession over libbuddy_hip.
 *
 * The reference's generation loop (runtime/llm/TextGeneration.cpp:157-277), its
 * REPL and its CLI talk to a model through the abstract class
 * buddy::runtime::LLMSession (runtime/include/buddy/runtime/llm/LLMSession.h:
 * 38-88); the class its code generator writes for a model
 * (tools/buddy-codegen/gen_session.py:1301-1511) is one implementation.  This
 * header is another: the same eight virtuals over the C interface of
 * buddy_hip.h, with the weights, the KV cache and every kernel on the GPU.  It
 * is meant to be compiled inside the reference tree (it includes the
 * reference's own headers) and linked with libbuddy_hip.so; nothing else of the
 * library depends on it.
 *
 *   buddy_hip::HipLLMSession session(shape);          // shape.max_len = cache rows
 *   session.loadWeights({"arg0-w8a32-f32.data", "arg0-w8a32-i8.data"});
 *   buddy::runtime::runGeneration(prompt, session, vocab, maxNewTokens, stops,
 *                                 sampler, codec, quiet);
 *
 * Behaviour follows the generated class: prefill() leaves the logits of every
 * prompt row for logitsData(row) and sets the position to the token count
 * (gen_session.py:1345-1369); decode() runs one step at the current position
 * and advances it (:1381-1452); handleKVCacheOverflow() acts once the position
 * has reached the cache length, keeps the clamped prefix, drops half of the
 * rest and re-rotates the moved keys with kvcache::buildInverseRopeFreqs(
 * ropeTheta, head_dim) (:1471-1511) -- here as one kernel on the device-resident
 * cache.  Failures throw std::runtime_error with the library's message, as the
 * generated class does for its own.
 */
#ifndef BUDDY_HIP_LLM_SESSION_H
#define BUDDY_HIP_LLM_SESSION_H

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

#include "buddy/runtime/llm/KVCacheManager.h"
#include "buddy/runtime/llm/LLMSession.h"
#include "buddy_hip/buddy_hip.h"

namespace buddy_hip {

class HipLLMSession : public buddy::runtime::LLMSession {
public:
  explicit HipLLMSession(const buddy_hip_model_shape &shape) : shape_(shape) {}
  ~HipLLMSession() override {
    if (session_)
      buddy_hip_session_destroy(session_);
  }

  /// {f32 file, int8 file}: the two parameter files of the w8a32 package
  /// (tools/buddy-codegen/gen_config.py:55-58).
  void loadWeights(const std::vector<std::string> &weightPaths) override {
    if (weightPaths.size() != 2)
      throw std::runtime_error("HipLLMSession: expected {f32 file, int8 file}");
    int64_t nF32 = 0, nI8 = 0;
    buddy_hip_w8a32_blob_sizes(&shape_, &nF32, &nI8);
    std::vector<float> f32((size_t)nF32);
    std::vector<int8_t> i8((size_t)nI8);
    readFile(weightPaths[0], f32.data(), sizeof(float) * (size_t)nF32);
    readFile(weightPaths[1], i8.data(), (size_t)nI8);
    if (session_)
      buddy_hip_session_destroy(session_);
    session_ =
        buddy_hip_session_create_from_w8a32_blobs(&shape_, f32.data(), nF32, i8.data(), nI8);
    if (!session_)
      fail("loadWeights");
    position_ = 0;
  }

  void prefill(buddy::Text<size_t, 2> &tokens) override {
    requireLoaded();
    const int n = (int)tokens.getTokenCnt();
    if (n <= 0 || n > shape_.max_len)
      throw std::runtime_error("HipLLMSession: prompt of " + std::to_string(n) +
                               " tokens does not fit the cache");
    std::vector<int> ids((size_t)n);
    const size_t *src = tokens.getData();
    for (int i = 0; i < n; ++i)
      ids[(size_t)i] = (int)src[i];
    logits_.resize((size_t)n * (size_t)shape_.vocab);
    if (buddy_hip_session_prefill_all_logits(session_, ids.data(), n, 0, logits_.data()))
      fail("prefill");
    position_ = n;
    rows_ = n;
  }

  void decode(int tokenId) override {
    requireLoaded();
    logits_.resize((size_t)shape_.vocab);
    if (buddy_hip_session_decode(session_, tokenId, position_, logits_.data(), nullptr))
      fail("decode");
    ++position_;
    rows_ = 1;
  }

  void resetPosition() override { position_ = 0; }
  int position() const override { return position_; }

  const float *logitsData(int tokenOffset = 0) const override {
    if (tokenOffset < 0 || tokenOffset >= rows_)
      throw std::runtime_error("HipLLMSession: no logits for row " +
                               std::to_string(tokenOffset));
    return logits_.data() + (size_t)tokenOffset * (size_t)shape_.vocab;
  }

  int vocabSize() const override { return shape_.vocab; }

  bool handleKVCacheOverflow(int keepTokenNum, float ropeTheta = 10000.0f) override {
    requireLoaded();
    if (position_ < shape_.max_len)
      return false;
    const int currentTokens = std::min(position_, shape_.max_len);
    keepTokenNum = std::clamp(keepTokenNum, 0, currentTokens - 1);
    const int discardLen = std::max(1, (currentTokens - keepTokenNum) / 2);
    const std::vector<float> inverseFreqs =
        buddy::kvcache::buildInverseRopeFreqs(ropeTheta, shape_.head_dim);
    if (buddy_hip_session_discard_kv_freqs(session_, keepTokenNum, discardLen, currentTokens,
                                           inverseFreqs.data()))
      fail("handleKVCacheOverflow");
    position_ = std::clamp(currentTokens - discardLen, 0, shape_.max_len);
    return true;
  }

private:
  void requireLoaded() const {
    if (!session_)
      throw std::runtime_error("HipLLMSession: loadWeights() has not been called");
  }
  [[noreturn]] static void fail(const char *what) {
    throw std::runtime_error(std::string("HipLLMSession::") + what + ": " +
                             buddy_hip_last_error());
  }
  static void readFile(const std::string &path, void *dst, size_t bytes) {
    FILE *f = std::fopen(path.c_str(), "rb");
    if (!f)
      throw std::runtime_error("Failed to open params file: " + path);
    const size_t got = std::fread(dst, 1, bytes, f);
    const bool more = got == bytes && std::fgetc(f) != EOF;
    std::fclose(f);
    if (got != bytes || more)
      throw std::runtime_error("params file " + path + " does not hold " +
                               std::to_string(bytes) + " bytes");
  }

  buddy_hip_model_shape shape_;
  buddy_hip_session *session_ = nullptr;
  int position_ = 0;
  int rows_ = 0; // rows of logits_ that are valid
  std::vector<float> logits_;
};

} // namespace buddy_hip

#endif // BUDDY_HIP_LLM_SESSION_H
