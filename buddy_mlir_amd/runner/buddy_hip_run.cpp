// buddy_hip_run -- runs a w8a32 weight package of the reference through
// libbuddy_hip: the two flat parameter files its importer writes
// (arg0-w8a32-f32.data, arg0-w8a32-i8.data; tools/buddy-codegen/gen_config.py:
// 55-58), a prompt given as token ids, block prefill, then greedy decoding.
//
// It follows the flow of the reference's own runner
// (examples/BuddyDeepSeekR1/buddy-deepseek-r1-w8a32-main.cpp:353-376 parameter
// loading, :505-506, :640-745 prefill, decode loop, end-of-text id 151643 and
// the closing report of prefill and decode tokens/s), without its tokenizer:
// token ids in, token ids out.
//
//   buddy_hip_run --f32 arg0-w8a32-f32.data --i8 arg0-w8a32-i8.data
//                 --tokens 151646,8948,... [--max-new 64] [--max-len 1024]
//                 [--eos 151643] [--layers 28 --hidden 1536 --heads 12
//                 --kv-heads 2 --inter 8960 --vocab 151936]
//                 [--temperature T --top-k K --top-p P --min-p P
//                  --repeat-penalty R --repeat-last-n N --seed S]
//
// With a temperature above 0 or a repetition penalty other than 1 the next
// token comes from the library's sampler
// (runtime/include/buddy/runtime/llm/Sampler.h:38-46 names the options),
// otherwise decoding is greedy on the device.
//
// Only the C interface of the library is used; nothing here touches the GPU
// directly.
#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "buddy_hip/buddy_hip.h"

namespace {

void usage(FILE *f) {
  fputs("usage: buddy_hip_run --f32 FILE --i8 FILE --tokens ID,ID,... [--max-new N]\n"
        "                     [--max-len N] [--eos ID] [--layers N --hidden N --heads N\n"
        "                     --kv-heads N --inter N --vocab N]\n"
        "                     [--temperature T --top-k K --top-p P --min-p P\n"
        "                      --repeat-penalty R --repeat-last-n N --seed S]\n"
        "Runs the reference's w8a32 parameter files (arg0-w8a32-f32.data,\n"
        "arg0-w8a32-i8.data) through libbuddy_hip: prefill of the prompt tokens, then\n"
        "greedy decoding, or sampling when a temperature or a repetition penalty is\n"
        "given.  Defaults are the DeepSeek-R1-Distill-Qwen-1.5B shape.\n",
        f);
}

// the whole file, or an empty vector with a message on stderr
template <typename T> bool read_file(const std::string &path, int64_t want, std::vector<T> &out) {
  FILE *f = fopen(path.c_str(), "rb");
  if (!f) {
    fprintf(stderr, "[Error] Failed to open params file: %s\n", path.c_str());
    return false;
  }
  fseek(f, 0, SEEK_END);
  const long long bytes = ftell(f);
  fseek(f, 0, SEEK_SET);
  if (bytes != (long long)(want * (int64_t)sizeof(T))) {
    fprintf(stderr, "[Error] %s holds %lld bytes, the model shape needs %lld\n", path.c_str(),
            bytes, (long long)(want * (int64_t)sizeof(T)));
    fclose(f);
    return false;
  }
  out.resize((size_t)want);
  const size_t got = fread(out.data(), sizeof(T), (size_t)want, f);
  fclose(f);
  if (got != (size_t)want) {
    fprintf(stderr, "[Error] Error occurred while reading params file %s\n", path.c_str());
    return false;
  }
  return true;
}

bool parse_tokens(const char *s, std::vector<int> &out) {
  while (*s) {
    char *end = nullptr;
    const long v = strtol(s, &end, 10);
    if (end == s || v < 0)
      return false;
    out.push_back((int)v);
    s = end;
    if (*s == ',')
      ++s;
    else if (*s)
      return false;
  }
  return !out.empty();
}

double seconds_since(std::chrono::steady_clock::time_point t0) {
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

} // namespace

int main(int argc, char **argv) {
  buddy_hip_model_shape shape = {28, 1536, 12, 2, 128, 8960, 151936, 1024, 1e-6f};
  std::string f32_path, i8_path;
  std::vector<int> prompt;
  int max_new = 64, eos = 151643;
  buddy_hip_sampler_config sampling = {0.0f, 0, 1.0f, 0.0f, 1.0f, 64, 0};
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    if (a == "--help" || a == "-h") {
      usage(stdout);
      return 0;
    }
    if (i + 1 >= argc) {
      usage(stderr);
      return 2;
    }
    const char *v = argv[++i];
    if (a == "--f32") f32_path = v;
    else if (a == "--i8") i8_path = v;
    else if (a == "--tokens") {
      if (!parse_tokens(v, prompt)) {
        fprintf(stderr, "[Error] --tokens wants a comma separated list of ids\n");
        return 2;
      }
    } else if (a == "--max-new") max_new = atoi(v);
    else if (a == "--max-len") shape.max_len = atoi(v);
    else if (a == "--eos") eos = atoi(v);
    else if (a == "--layers") shape.layers = atoi(v);
    else if (a == "--hidden") shape.hidden = atoi(v);
    else if (a == "--heads") shape.heads = atoi(v);
    else if (a == "--kv-heads") shape.kv_heads = atoi(v);
    else if (a == "--inter") shape.inter = atoi(v);
    else if (a == "--vocab") shape.vocab = atoi(v);
    else if (a == "--temperature") sampling.temperature = (float)atof(v);
    else if (a == "--top-k") sampling.top_k = atoi(v);
    else if (a == "--top-p") sampling.top_p = (float)atof(v);
    else if (a == "--min-p") sampling.min_p = (float)atof(v);
    else if (a == "--repeat-penalty") sampling.repeat_penalty = (float)atof(v);
    else if (a == "--repeat-last-n") sampling.repeat_last_n = atoi(v);
    else if (a == "--seed") sampling.seed = strtoull(v, nullptr, 10);
    else {
      usage(stderr);
      return 2;
    }
  }
  if (f32_path.empty() || i8_path.empty() || prompt.empty() || max_new < 1) {
    usage(stderr);
    return 2;
  }
  if ((int)prompt.size() + max_new > shape.max_len) {
    fprintf(stderr, "[Error] %zu prompt tokens + %d new ones do not fit a cache of %d positions\n",
            prompt.size(), max_new, shape.max_len);
    return 2;
  }
  for (int t : prompt)
    if (t >= shape.vocab) {
      fprintf(stderr, "[Error] token id %d outside the vocabulary (%d)\n", t, shape.vocab);
      return 2;
    }

  int64_t n_f32 = 0, n_i8 = 0;
  buddy_hip_w8a32_blob_sizes(&shape, &n_f32, &n_i8);
  auto t0 = std::chrono::steady_clock::now();
  std::vector<float> f32;
  std::vector<int8_t> i8;
  if (!read_file(f32_path, n_f32, f32) || !read_file(i8_path, n_i8, i8))
    return 1;
  printf("[Log] Params load time: %.3fs\n", seconds_since(t0));

  t0 = std::chrono::steady_clock::now();
  buddy_hip_session *s =
      buddy_hip_session_create_from_w8a32_blobs(&shape, f32.data(), n_f32, i8.data(), n_i8);
  if (!s) {
    fprintf(stderr, "[Error] %s\n", buddy_hip_last_error());
    return 1;
  }
  std::vector<int8_t>().swap(i8); // the session holds its own packed copy
  printf("[Log] Upload and packing: %.3fs\n", seconds_since(t0));

  const bool sampled = sampling.temperature > 0.0f || sampling.repeat_penalty != 1.0f;
  buddy_hip_sampler *sampler = nullptr;
  if (sampled && !(sampler = buddy_hip_sampler_create(&sampling))) {
    fprintf(stderr, "[Error] %s\n", buddy_hip_last_error());
    return 1;
  }

  // prefill: the prompt as one block; the token it predicts is the first output
  int next = -1;
  t0 = std::chrono::steady_clock::now();
  if (buddy_hip_session_prefill(s, prompt.data(), (int)prompt.size(), 0, nullptr, &next)) {
    fprintf(stderr, "[Error] %s\n", buddy_hip_last_error());
    return 1;
  }
  // the reference samples the first token from the prefill logits, with no
  // recent ids yet (runtime/llm/TextGeneration.cpp:191-196)
  if (sampled && buddy_hip_sampler_sample(sampler, buddy_hip_session_logits(s), shape.vocab,
                                          nullptr, 0, &next, buddy_hip_session_stream(s))) {
    fprintf(stderr, "[Error] %s\n", buddy_hip_last_error());
    return 1;
  }
  const double prefill_s = seconds_since(t0);

  // decode: greedy steps on the device, in runs of 16 so that an end-of-text id
  // stops the generation soon after it appears
  std::vector<int> out;
  out.push_back(next);
  int pos = (int)prompt.size();
  double decode_s = 0;
  int decoded = 0;
  while (sampled && (int)out.size() < max_new && out.back() != eos) {
    t0 = std::chrono::steady_clock::now();
    if (buddy_hip_session_decode_sample(s, sampler, out.back(), pos, out.data(), (int)out.size(),
                                        &next)) {
      fprintf(stderr, "[Error] %s\n", buddy_hip_last_error());
      return 1;
    }
    decode_s += seconds_since(t0);
    ++decoded;
    ++pos;
    out.push_back(next);
  }
  while ((int)out.size() < max_new && out.back() != eos) {
    const int run = std::min(16, max_new - (int)out.size());
    int buf[16];
    t0 = std::chrono::steady_clock::now();
    if (buddy_hip_session_decode_greedy(s, out.back(), pos, run, buf)) {
      fprintf(stderr, "[Error] %s\n", buddy_hip_last_error());
      return 1;
    }
    decode_s += seconds_since(t0);
    decoded += run;
    pos += run;
    for (int i = 0; i < run; ++i) {
      out.push_back(buf[i]);
      if (buf[i] == eos)
        break;
    }
  }
  buddy_hip_sampler_destroy(sampler);
  buddy_hip_session_destroy(s);

  printf("[Prefilling] %.1f tokens/s\n", (double)prompt.size() / prefill_s);
  printf("[Decoding] %.1f tokens/s\n", decoded ? decoded / decode_s : 0.0);
  printf("[Input ids]");
  for (int t : prompt)
    printf(" %d", t);
  printf("\n[Output ids]");
  for (int t : out)
    printf(" %d", t);
  printf("\n");
  return 0;
}
