// Sampler host API, signature-compatible with the reference's include/rwkv_sampler.hpp.
#pragma once

#include <cstdint>
#include <vector>

#include "rwkv_server_backend.hpp"

namespace rwkv7_server {

struct SamplerPenaltyState {
  int batch_size = 0;
  int vocab_size = 0;
  rwkv7_fast_v4::DeviceBuffer<float> penalties;
  rwkv7_fast_v4::DeviceBuffer<float> probs;
  rwkv7_fast_v4::DeviceBuffer<int> outputs;
  rwkv7_fast_v4::DeviceBuffer<std::uint8_t> rand_states;  // unused: the generator is counter-based
  std::uint64_t seed = 0;   // Philox key
  std::uint64_t step = 0;   // Philox counter, advanced by every sampling call
};

// seed == 0 draws a seed from std::random_device and the clock as the reference does
// (src/rwkv_sampler.cpp:14-19); any other value makes the token stream reproducible.
SamplerPenaltyState make_sampler_penalties(int vocab_size, int batch_size = 1, std::uint64_t seed = 0);

int sample_repetition_temperature_topk_topp(const DeviceLogits& logits, SamplerPenaltyState& penalties,
                                            const GenerateOptions& options);

std::vector<int> sample_batch_repetition_temperature_topk_topp(const DeviceLogits& logits,
                                                               SamplerPenaltyState& penalties,
                                                               const GenerateOptions& options);

}  // namespace rwkv7_server
