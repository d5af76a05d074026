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

// Streams: the sampling kernels run on the device's NULL stream and the token ids come back with a blocking copy,
// so the call returns with the ids on the host.  ModelBackend's forward calls run on per-session non-blocking
// streams and return only after their stream has drained, so logits handed from a forward call to the sampler on the
// same thread are complete, and the NULL stream never waits for another thread's forward.  Sampling calls of several
// threads queue behind one another on the NULL stream (each works on its own SamplerPenaltyState, so the results do
// not depend on the order); logits written by work still in flight on a stream of the caller's own must be
// synchronised by the caller first.
int sample_repetition_temperature_topk_topp(const DeviceLogits& logits, SamplerPenaltyState& penalties,
                                            const GenerateOptions& options);

std::vector<int> sample_batch_repetition_temperature_topk_topp(const DeviceLogits& logits,
                                                               SamplerPenaltyState& penalties,
                                                               const GenerateOptions& options);

}  // namespace rwkv7_server
