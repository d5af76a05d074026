// Sampler host wrapper (reference: src/rwkv_sampler.cpp:22-121): same argument checks and messages;
// the kernel launch goes through rwkv_hip_sample and the token ids come back with one blocking copy.
#include "rwkv_sampler.hpp"

#include <chrono>
#include <random>
#include <stdexcept>

namespace rwkv7_server {
namespace {

std::uint64_t fresh_seed() {
  std::random_device rd;
  const auto now = static_cast<std::uint64_t>(std::chrono::high_resolution_clock::now().time_since_epoch().count());
  std::uint64_t s = (static_cast<std::uint64_t>(rd()) << 32) ^ static_cast<std::uint64_t>(rd()) ^ now;
  return s ? s : 1;
}

}  // namespace

SamplerPenaltyState make_sampler_penalties(int vocab_size, int batch_size, std::uint64_t seed) {
  if (vocab_size <= 0) throw std::runtime_error("invalid sampler vocab size");
  if (batch_size <= 0) throw std::runtime_error("invalid sampler batch size");
  SamplerPenaltyState state;
  state.batch_size = batch_size;
  state.vocab_size = vocab_size;
  const std::size_t n = static_cast<std::size_t>(batch_size) * vocab_size;
  state.penalties.resize(n, "alloc sampler penalties");
  state.probs.resize(n, "alloc sampler probs");
  state.outputs.resize(batch_size, "alloc sampler outputs");
  state.penalties.zero("zero sampler penalties");
  state.seed = seed ? seed : fresh_seed();
  state.step = 0;
  return state;
}

std::vector<int> sample_batch_repetition_temperature_topk_topp(const DeviceLogits& logits,
                                                               SamplerPenaltyState& penalties,
                                                               const GenerateOptions& options) {
  if (logits.rows <= 0) throw std::runtime_error("sampler expects at least one logits row");
  if (logits.vocab_size <= 0 || logits.values.p == nullptr) throw std::runtime_error("empty device logits");
  if (penalties.vocab_size != logits.vocab_size)
    throw std::runtime_error("sampler logits size does not match sampler state");
  if (penalties.batch_size != logits.rows)
    throw std::runtime_error("sampler batch size does not match logits rows");

  const bool use_penalty = options.alpha_presence != 0.0 || options.alpha_frequency != 0.0;
  const int rc = rwkv_hip_sample(nullptr, logits.rows, logits.vocab_size, logits.values.p,
                                 use_penalty ? penalties.penalties.p : nullptr, penalties.probs.p, penalties.outputs.p,
                                 options.alpha_presence, options.alpha_frequency, options.alpha_decay,
                                 options.temperature, options.top_k, options.top_p, penalties.seed, penalties.step++);
  if (rc != RWKV_OK) throw std::invalid_argument(rwkv_hip_last_error());
  std::vector<int> tokens(static_cast<std::size_t>(logits.rows));
  rwkv7_fast_v4::check_hip(rwkv_hip_memcpy_d2h(tokens.data(), penalties.outputs.p, tokens.size() * sizeof(int)),
                           "copy sampled tokens to host");
  return tokens;
}

int sample_repetition_temperature_topk_topp(const DeviceLogits& logits, SamplerPenaltyState& penalties,
                                            const GenerateOptions& options) {
  if (logits.rows != 1) throw std::runtime_error("sampler currently expects a single logits row");
  return sample_batch_repetition_temperature_topk_topp(logits, penalties, options).front();
}

}  // namespace rwkv7_server
