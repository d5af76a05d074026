// Rates through the drop-in boundary: InferenceEngine::batch_generate_stream over a ModelBackend with synthetic
// weights, as GenerationStats reports them (prompt_tokens / prefill_seconds, generated_tokens / decode_seconds -
// the counters behind the reference server's prefill_speed / decode_speed, src/rwkv_api_service.cpp:294-338).
// Every decode step goes through forward_decode, the device sampler and the host round trip of the picked ids;
// every request creates its own GenerationState and logits.  Prints one JSON object per line:
//   {"request": i, "batch": B, "sampled": 0|1, "prefill_tok_s": .., "decode_tok_s": .., "decode_ms_per_step": ..,
//    "graph_captures": decode graphs captured during this request}
// Usage: engine_rate_bench <repo root> <model spec> <batch> <max tokens> <requests> <sampled 0|1> [wkv32 0|1]
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <string>
#include <vector>

#include "rwkv_hip.h"
#include "rwkv_inference_engine.hpp"

using namespace rwkv7_server;

int main(int argc, char** argv) {
  if (argc < 7) {
    std::fprintf(stderr, "usage: %s <repo root> <model spec> <batch> <max tokens> <requests> <sampled 0|1> [wkv32 0|1]\n", argv[0]);
    return 2;
  }
  const std::string root = argv[1];
  const std::string spec = argv[2];
  const int batch = std::atoi(argv[3]);
  const int max_tokens = std::atoi(argv[4]);
  const int requests = std::atoi(argv[5]);
  const bool sampled = std::atoi(argv[6]) != 0;
  const bool wkv32 = argc > 7 ? std::atoi(argv[7]) != 0 : true;
  try {
    auto tok = std::make_shared<TrieTokenizer>();
    if (tok->load(root + "/tests/golden/synthetic_vocab.txt") != kTokenizerSuccess) {
      std::fprintf(stderr, "vocabulary load failed\n");
      return 1;
    }
    auto backend = std::make_shared<ModelBackend>(spec, wkv32);
    InferenceEngine engine(backend, tok, "bench", 128);
    std::string prompt = "System: test\n\nUser: ";
    for (int i = 0; i < 24; ++i) prompt += "This is a test answer. ";
    prompt += "\n\nAssistant:";
    const std::vector<std::string> prompts(static_cast<std::size_t>(batch), prompt);
    GenerateOptions o;
    o.max_tokens = max_tokens;
    o.stop_tokens = {};  // random-init weights: run to max_tokens
    if (sampled) {
      o.top_k = 50; o.top_p = 0.6; o.temperature = 1.0;
      o.alpha_presence = 0.5; o.alpha_frequency = 0.1; o.alpha_decay = 0.99;
    } else {
      o.top_k = 0; o.top_p = 0.0; o.temperature = 1.0;
      o.alpha_presence = 0.0; o.alpha_frequency = 0.0; o.alpha_decay = 1.0;
    }
    for (int r = 0; r < requests; ++r) {
      int64_t before = 0, after = 0;
      rwkv_hip_graph_capture_count(&before);
      const auto stats = engine.batch_generate_stream(prompts, o, 8, [](int, const std::string&) { return true; });
      rwkv_hip_graph_capture_count(&after);
      const double steps = static_cast<double>(stats.generated_tokens) / batch;
      std::printf("{\"request\": %d, \"batch\": %d, \"sampled\": %d, \"prompt_tokens\": %d, \"generated_tokens\": %d, "
                  "\"prefill_tok_s\": %.1f, \"decode_tok_s\": %.1f, \"decode_ms_per_step\": %.4f, \"graph_captures\": %lld}\n",
                  r, batch, sampled ? 1 : 0, stats.prompt_tokens, stats.generated_tokens,
                  stats.prefill_seconds > 0 ? stats.prompt_tokens / stats.prefill_seconds : 0.0,
                  stats.decode_seconds > 0 ? stats.generated_tokens / stats.decode_seconds : 0.0,
                  steps > 0 ? stats.decode_seconds * 1e3 / steps : 0.0, static_cast<long long>(after - before));
      std::fflush(stdout);
    }
  } catch (const std::exception& e) {
    std::fprintf(stderr, "engine_rate_bench: %s\n", e.what());
    return 1;
  }
  return 0;
}
