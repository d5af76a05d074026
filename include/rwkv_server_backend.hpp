// Host-side backend API, signature-compatible with the reference's include/rwkv_server_backend.hpp:15-147,
// implemented over librwkv_hip.so.  Both WKV state precisions are provided: fp16 (the default, use_wkv32 = false) and fp32.
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "rwkv7_fast_v4_common.hpp"

namespace rwkv7_server {

struct PrefillCapacity {
  std::size_t free_vram_bytes = 0;
  std::size_t total_vram_bytes = 0;
  std::size_t reserve_vram_bytes = 0;
  std::size_t bytes_per_batch = 0;
  int max_batch_size = 0;
};

enum class ThinkType { Fast, Free, PreferChinese, En, EnShort, EnLong };

struct GenerateOptions {
  int max_tokens = 8192;
  std::vector<int64_t> stop_tokens{0, 261, 24281};
  double temperature = 1.0;
  int top_k = 20;
  double top_p = 0.3;
  double alpha_presence = 2.0;
  double alpha_frequency = 0.2;
  double alpha_decay = 0.996;
  bool force_reasoning = false;
  int force_reasoning_token_offset = 0;
};

// shift f16 [L,2,B,C]; the WKV state [L,B,H,64,64] in wkv_state32 (f32, wkv32 == true) or wkv_state (f16,
// wkv32 == false): a backend allocates the one of its mode; elapsed i32 [B].
struct GenerationState {
  int batch_size = 0;
  bool wkv32 = false;
  rwkv7_fast_v4::DeviceBuffer<half> shift;
  rwkv7_fast_v4::DeviceBuffer<half> wkv_state;
  rwkv7_fast_v4::DeviceBuffer<float> wkv_state32;
  rwkv7_fast_v4::DeviceBuffer<int> elapsed;

  GenerationState() = default;
  GenerationState(const GenerationState&) = delete;
  GenerationState& operator=(const GenerationState&) = delete;
  GenerationState(GenerationState&&) noexcept = default;
  GenerationState& operator=(GenerationState&&) noexcept = default;
};

struct DeviceLogits {
  int rows = 0;
  int vocab_size = 0;
  rwkv7_fast_v4::DeviceBuffer<float> values;

  DeviceLogits() = default;
  DeviceLogits(const DeviceLogits&) = delete;
  DeviceLogits& operator=(const DeviceLogits&) = delete;
  DeviceLogits(DeviceLogits&&) noexcept = default;
  DeviceLogits& operator=(DeviceLogits&&) noexcept = default;
};

class IModelBackend {
 public:
  virtual ~IModelBackend() = default;

  virtual GenerationState create_state(int batch_size) const = 0;
  virtual void forward_prefill(const std::vector<std::vector<int64_t>>& token_batches, GenerationState& state,
                               DeviceLogits& logits) const = 0;
  virtual void forward_decode(const std::vector<int64_t>& token_batch, GenerationState& state,
                              DeviceLogits& logits) const = 0;
  virtual void copy_state_slice(const GenerationState& src, int src_offset, GenerationState& dst, int dst_offset,
                                int count) const = 0;
  virtual void copy_logits_slice(const DeviceLogits& src, int src_offset, DeviceLogits& dst, int dst_offset,
                                 int count) const = 0;
  virtual PrefillCapacity query_prefill_capacity(int prefill_chunk_size) const = 0;

  virtual int vocab_size() const = 0;
  virtual const std::string& model_path() const = 0;
  virtual const std::string& model_name() const = 0;
};

// model_path selects the weights: a .pth checkpoint, optionally followed by ":w8" or ":w4" (quantise on load), or
//   "synthetic:<0.1B|1.5B|7.2B|tiny>[:f16|w8|w4][:seed=<n>]"   a random-init model of that shape.
// use_wkv32 = false (the reference's default) keeps the WKV state in fp16 and runs the recurrence in fp16 as the
// reference's cuda/rwkv7_wkv_fp16_v2.cu does; true keeps it in fp32.  chunk_load reads the checkpoint on demand
// instead of through a whole-file copy.
class ModelBackend final : public IModelBackend {
 public:
  explicit ModelBackend(std::string model_path, bool use_wkv32 = false, bool chunk_load = false);
  ~ModelBackend() override;

  ModelBackend(const ModelBackend&) = delete;
  ModelBackend& operator=(const ModelBackend&) = delete;
  ModelBackend(ModelBackend&&) noexcept;
  ModelBackend& operator=(ModelBackend&&) noexcept;

  GenerationState create_state(int batch_size) const override;
  void forward_prefill(const std::vector<std::vector<int64_t>>& token_batches, GenerationState& state,
                       DeviceLogits& logits) const override;
  void forward_decode(const std::vector<int64_t>& token_batch, GenerationState& state,
                      DeviceLogits& logits) const override;
  void copy_state_slice(const GenerationState& src, int src_offset, GenerationState& dst, int dst_offset,
                        int count) const override;
  void copy_logits_slice(const DeviceLogits& src, int src_offset, DeviceLogits& dst, int dst_offset,
                         int count) const override;
  PrefillCapacity query_prefill_capacity(int prefill_chunk_size) const override;

  int vocab_size() const override;
  const std::string& model_path() const override;
  const std::string& model_name() const override;

  const rwkv7_fast_v4::ModelDims& dims() const;

 private:
  struct Impl;
  std::unique_ptr<Impl> impl_;
};

}  // namespace rwkv7_server
