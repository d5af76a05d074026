// IModelBackend double for engine control-flow tests: every forward call is recorded and answers with the next
// row of a scripted logits table (the same row for every batch element).  forward_prefill rewinds the script,
// so the logits after a prefill are always script row 0.  Same role as the reference's test/fake_backend.hpp.
#pragma once

#include <algorithm>

#include "test_common.hpp"

namespace host_test {

class ScriptedBackend final : public rwkv7_server::IModelBackend {
 public:
  using Tokens = std::vector<int64_t>;

  ScriptedBackend(std::vector<std::vector<float>> script, std::string name)
      : script_(std::move(script)), vocab_(script_.empty() ? 0 : int(script_[0].size())), name_(std::move(name)) {
    for (const auto& row : script_)
      if (int(row.size()) != vocab_) throw std::runtime_error("scripted rows differ in width");
  }

  // a script whose greedy decoding is `tokens` followed by token 0
  static std::vector<std::vector<float>> script_for(const std::vector<int>& tokens, int vocab) {
    std::vector<std::vector<float>> rows;
    for (int t : tokens) rows.push_back(one_hot(vocab, t));
    rows.push_back(one_hot(vocab, 0));
    return rows;
  }

  rwkv7_server::GenerationState create_state(int batch_size) const override {
    rwkv7_server::GenerationState s;
    s.batch_size = batch_size;
    return s;
  }
  void forward_prefill(const std::vector<Tokens>& batch, rwkv7_server::GenerationState& state,
                       rwkv7_server::DeviceLogits& logits) const override {
    prefills.push_back(batch);
    state.batch_size = int(batch.size());
    cursor_ = 0;
    answer(int(batch.size()), logits);
  }
  void forward_decode(const Tokens& batch, rwkv7_server::GenerationState&,
                      rwkv7_server::DeviceLogits& logits) const override {
    decodes.push_back(batch);
    ++cursor_;
    answer(int(batch.size()), logits);
  }
  void copy_state_slice(const rwkv7_server::GenerationState& src, int so, rwkv7_server::GenerationState& dst, int dof,
                        int count) const override {
    if (so < 0 || dof < 0 || count <= 0 || so + count > src.batch_size || dof + count > dst.batch_size)
      throw std::runtime_error("scripted backend: bad state slice");
    ++state_slice_copies;
  }
  void copy_logits_slice(const rwkv7_server::DeviceLogits& src, int so, rwkv7_server::DeviceLogits& dst, int dof,
                         int count) const override {
    if (so < 0 || dof < 0 || count <= 0 || so + count > src.rows || dof + count > dst.rows ||
        src.vocab_size != dst.vocab_size)
      throw std::runtime_error("scripted backend: bad logits slice");
    const std::size_t bytes = std::size_t(count) * src.vocab_size * sizeof(float);
    rwkv7_fast_v4::check_hip(rwkv_hip_memcpy_d2d(dst.values.p + std::size_t(dof) * dst.vocab_size,
                                                 src.values.p + std::size_t(so) * src.vocab_size, bytes),
                             "scripted logits slice");
  }
  rwkv7_server::PrefillCapacity query_prefill_capacity(int) const override {
    rwkv7_server::PrefillCapacity c;
    c.max_batch_size = 1024;
    return c;
  }
  int vocab_size() const override { return vocab_; }
  const std::string& model_path() const override { return path_; }
  const std::string& model_name() const override { return name_; }

  // Rows 1.. of every batch answer from this script instead (its last row repeats once it is used up), so that
  // batch rows can differ and finish at different steps.
  void set_script_for_other_rows(std::vector<std::vector<float>> script) { other_rows_ = std::move(script); }

  mutable std::vector<std::vector<Tokens>> prefills;  // one entry per forward_prefill call
  mutable std::vector<Tokens> decodes;                // one entry per forward_decode call
  mutable int state_slice_copies = 0;

 private:
  void answer(int rows, rwkv7_server::DeviceLogits& logits) const {
    if (cursor_ >= script_.size()) throw std::runtime_error("scripted backend ran out of rows");
    std::vector<float> host;
    for (int r = 0; r < rows; ++r) {
      const auto& row = (r == 0 || other_rows_.empty()) ? script_[cursor_]
                                                        : other_rows_[std::min(cursor_, other_rows_.size() - 1)];
      host.insert(host.end(), row.begin(), row.end());
    }
    logits.rows = rows;
    logits.vocab_size = vocab_;
    to_device(host, logits.values);
  }

  std::vector<std::vector<float>> script_;
  std::vector<std::vector<float>> other_rows_;
  int vocab_;
  std::string path_ = "scripted://backend";
  std::string name_;
  mutable std::size_t cursor_ = 0;
};

}  // namespace host_test
