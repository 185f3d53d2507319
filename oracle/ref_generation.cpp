/*
 * ref_generation.cpp -- the reference's own generation loop over libbuddy_hip.
 *
 * Test harness: compiled together with the reference's
 * runtime/llm/TextGeneration.cpp (runGeneration, the streaming output) and its
 * header-only tokenizer, sampler and KV-cache manager, where they lie in the
 * reference tree; the model behind the reference's LLMSession interface is
 * buddy_hip::HipLLMSession (include/buddy_hip/llm_session.h).  What
 * examples/BuddyDeepSeekR1/buddy-deepseek-r1-main.cpp does around the generated
 * session, this does around the GPU one:
 *
 *   ref_generation --f32 F --i8 I --vocab V --prompt "text" --max-tokens N
 *                  [--max-len L --layers .. --hidden .. --heads .. --kv-heads ..
 *                   --inter .. --vocab-size ..]
 *                  [--temperature T --top-k K --top-p P --min-p P
 *                   --repeat-penalty R --repeat-last-n N --seed S]
 *
 * It prints the prompt's token ids ("[input ids] ...") and then the JSON lines
 * of the reference's own streaming mode, one per generated token.
 *
 * TEST INFRASTRUCTURE ONLY, like the rest of this directory.
 */
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <string>
#include <vector>

#include "buddy/runtime/llm/TextGeneration.h"
#include "buddy_hip/llm_session.h"

int main(int argc, char **argv) {
  buddy_hip_model_shape shape = {28, 1536, 12, 2, 128, 8960, 151936, 1024, 1e-6f};
  std::string f32, i8, vocab, prompt;
  int maxTokens = 64;
  buddy::SamplerConfig sc;
  for (int i = 1; i + 1 < argc; i += 2) {
    const std::string a = argv[i];
    const char *v = argv[i + 1];
    if (a == "--f32") f32 = v;
    else if (a == "--i8") i8 = v;
    else if (a == "--vocab") vocab = v;
    else if (a == "--prompt") prompt = v;
    else if (a == "--max-tokens") maxTokens = atoi(v);
    else if (a == "--max-len") shape.max_len = atoi(v);
    else if (a == "--layers") shape.layers = atoi(v);
    else if (a == "--hidden") shape.hidden = atoi(v);
    else if (a == "--heads") shape.heads = atoi(v);
    else if (a == "--kv-heads") shape.kv_heads = atoi(v);
    else if (a == "--inter") shape.inter = atoi(v);
    else if (a == "--vocab-size") shape.vocab = atoi(v);
    else if (a == "--temperature") sc.temperature = (float)atof(v);
    else if (a == "--top-k") sc.topK = atoi(v);
    else if (a == "--top-p") sc.topP = (float)atof(v);
    else if (a == "--min-p") sc.minP = (float)atof(v);
    else if (a == "--repeat-penalty") sc.repeatPenalty = (float)atof(v);
    else if (a == "--repeat-last-n") sc.repeatLastN = atoi(v);
    else if (a == "--seed") sc.seed = strtoull(v, nullptr, 10);
    else {
      fprintf(stderr, "unknown option %s\n", a.c_str());
      return 2;
    }
  }
  if (f32.empty() || i8.empty() || vocab.empty() || prompt.empty()) {
    fprintf(stderr, "--f32, --i8, --vocab and --prompt are required\n");
    return 2;
  }
  try {
    buddy_hip::HipLLMSession session(shape);
    session.loadWeights({f32, i8});

    const int maxLen = shape.max_len;
    buddy::runtime::TextCodec codec;
    codec.tokenize = [maxLen](buddy::Text<size_t, 2> &t, const std::string &vocabPath) {
      t.tokenizeDeepSeekR1(vocabPath, (size_t)maxLen);
    };
    codec.detokenize = [](buddy::Text<size_t, 2> &t) { return t.revertDeepSeekR1(); };
    codec.maxTokenLen = maxLen;

    { // the ids the loop is going to feed, for whoever checks the run
      buddy::Text<size_t, 2> probe(prompt);
      codec.tokenize(probe, vocab);
      std::cout << "[input ids]";
      for (size_t i = 0; i < probe.getTokenCnt(); ++i)
        std::cout << ' ' << probe.getData()[i];
      std::cout << std::endl;
    }

    buddy::Sampler sampler(sc);
    const std::vector<long long> stops = {151643};
    const buddy::runtime::GenerationResult r = buddy::runtime::runGeneration(
        prompt, session, vocab, maxTokens, stops, sampler, codec, /*suppress=*/true,
        /*streamJsonl=*/true);
    std::cout << "[generated] " << r.generatedTokens << " decode steps, final position "
              << session.position() << std::endl;
  } catch (const std::exception &e) {
    fprintf(stderr, "[Error] %s\n", e.what());
    return 1;
  }
  return 0;
}
