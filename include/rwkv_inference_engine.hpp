// Inference engine host API, signature-compatible with the reference's include/rwkv_inference_engine.hpp.
#pragma once

#include <functional>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "rwkv_sampler.hpp"
#include "rwkv_server_backend.hpp"
#include "rwkv_tokenizer.hpp"

namespace rwkv7_server {

class InferenceEngine {
 public:
  using StreamCallback = std::function<bool(int, const std::string&)>;
  using ControlCallback = std::function<bool()>;

  struct GenerationStats {
    int prompt_tokens = 0;
    int generated_tokens = 0;
    double prefill_seconds = 0.0;
    double decode_seconds = 0.0;
    bool stopped = false;
    bool stop_token = false;
  };
  using StatsCallback = std::function<void(const GenerationStats&)>;

  InferenceEngine(std::shared_ptr<IModelBackend> model, std::shared_ptr<TrieTokenizer> tokenizer,
                  std::string model_name, int prefill_chunk_size = 128);

  std::vector<std::string> batch_generate(const std::vector<std::string>& prompts,
                                          const GenerateOptions& options) const;
  std::vector<std::string> batch_generate_state(const std::vector<std::string>& prompts, GenerationState& state,
                                                const GenerateOptions& options) const;
  GenerationStats batch_generate_stream(const std::vector<std::string>& prompts, const GenerateOptions& options,
                                        int chunk_size, const StreamCallback& emit,
                                        const ControlCallback& should_stop = {},
                                        const StatsCallback& on_prefill_complete = {}) const;
  void batch_generate_state_stream(const std::vector<std::string>& prompts, GenerationState& state,
                                   const GenerateOptions& options, int chunk_size, const StreamCallback& emit,
                                   const ControlCallback& should_stop = {}) const;
  int prefill_prompt(const std::string& prompt, GenerationState& state, DeviceLogits& logits) const;
  GenerationStats generate_from_logits_stream(GenerationState& state, DeviceLogits& logits,
                                              const GenerateOptions& options, int chunk_size,
                                              const StreamCallback& emit,
                                              const ControlCallback& should_stop = {}) const;

  std::string format_openai_prompt(const std::string& system,
                                   const std::vector<std::pair<std::string, std::string>>& messages,
                                   ThinkType think_type) const;
  std::string format_openai_prompt(const std::string& system,
                                   const std::vector<std::pair<std::string, std::string>>& messages,
                                   bool enable_think) const;
  int count_tokens(const std::string& text) const;

  std::shared_ptr<IModelBackend> model() const { return model_; }
  std::shared_ptr<TrieTokenizer> tokenizer() const { return tokenizer_; }
  const std::string& model_name() const { return model_name_; }
  int prefill_chunk_size() const { return prefill_chunk_size_; }

  // Continuous batching that shrinks (no counterpart in the reference, which keeps every finished row in the
  // batch and feeds it a stop token until the last row ends, src/rwkv_inference_engine.cpp:497-499).  When on,
  // batch_generate and batch_generate_stream gather the rows that are still generating into a narrower state
  // once at most half of the current width is left, so a batch with one long answer does not pay for the
  // finished ones.  Off by default: the reference's behaviour.  A row's greedy output is the same either way up
  // to the rounding differences between the kernels of different batch widths; stochastic draws are keyed by
  // the row's position in the batch, so they change when rows move.
  void set_shrink_batch(bool on) { shrink_batch_ = on; }
  bool shrink_batch() const { return shrink_batch_; }

 private:
  std::vector<int64_t> encode_prompt(const std::string& prompt) const;
  std::vector<std::vector<int64_t>> encode_prompts_sorted(const std::vector<std::string>& prompts,
                                                          std::vector<size_t>& sorted_to_original) const;
  void prefill_batch_chunked(const std::vector<std::vector<int64_t>>& sorted_prompt_ids, GenerationState& state,
                             DeviceLogits& logits) const;
  std::string generate_one(const std::string& prompt, GenerationState& state, const GenerateOptions& options,
                           const StreamCallback* emit, int stream_index, int chunk_size,
                           const ControlCallback& should_stop) const;

  std::shared_ptr<IModelBackend> model_;
  std::shared_ptr<TrieTokenizer> tokenizer_;
  std::string model_name_;
  int prefill_chunk_size_ = 128;
  bool shrink_batch_ = false;
};

}  // namespace rwkv7_server
