// Generation control flow over IModelBackend: chunked batched prefill, sampling loops, force-reasoning logit
// mask, UTF-8-safe streaming, prompt templates.  Behaviour follows the reference's
// src/rwkv_inference_engine.cpp (prefill_batch_chunked :268-332, generate_one :334-385, batch_generate
// :387-440, batch_generate_stream :452-560, generate_from_logits_stream :585-642, templates :21-43,644-689).
#include "rwkv_inference_engine.hpp"

#include <algorithm>
#include <chrono>
#include <numeric>
#include <stdexcept>

namespace rwkv7_server {
namespace {

using Clock = std::chrono::steady_clock;

double seconds_since(Clock::time_point t0) { return std::chrono::duration<double>(Clock::now() - t0).count(); }

// ---- prompt templates -------------------------------------------------------------------------------------------

struct ThinkStyle {
  std::string assistant_header;  // appended after "Assistant: "
  std::string user_footer;       // appended to the last User message
};

ThinkStyle think_style(ThinkType type) {
  switch (type) {
    case ThinkType::Free: return {"<think", ""};
    case ThinkType::PreferChinese: return {"<think>\xE5\x97\xAF", ""};
    case ThinkType::En: return {"<think", " (think)"};
    case ThinkType::EnShort: return {"<think", " (think a bit)"};
    case ThinkType::EnLong: return {"<think", " (think a lot)"};
    case ThinkType::Fast: break;
  }
  return {"<think>\n</think", ""};
}

// ---- force-reasoning mask ---------------------------------------------------------------------------------------

// With force_reasoning on, generated tokens number 1 and 2 (counted from force_reasoning_token_offset) may not
// be 111 or 754: their logits are set to -1e30 for that one sampling call and restored afterwards.
constexpr int kDeniedTokens[] = {111, 754};
constexpr int kMaskFirstStep = 1;
constexpr int kMaskLastStep = 2;
constexpr float kMaskedLogit = -1.0e30f;

bool mask_applies(const GenerateOptions& options, int step) {
  const int total = options.force_reasoning_token_offset + step;
  return options.force_reasoning && total >= kMaskFirstStep && total <= kMaskLastStep;
}

class LogitMask {
 public:
  explicit LogitMask(DeviceLogits& logits) : logits_(logits) {
    if (logits.rows <= 0 || logits.vocab_size <= 0 || logits.values.p == nullptr) return;
    for (int row = 0; row < logits.rows; ++row) {
      for (int token : kDeniedTokens) {
        if (token >= logits.vocab_size) continue;
        float* slot = logits.values.p + static_cast<std::size_t>(row) * logits.vocab_size + token;
        float saved = 0.0f;
        rwkv7_fast_v4::check_hip(rwkv_hip_memcpy_d2h(&saved, slot, sizeof(float)), "read logit to mask");
        rwkv7_fast_v4::check_hip(rwkv_hip_memcpy_h2d(slot, &kMaskedLogit, sizeof(float)), "write masked logit");
        saved_.push_back({slot, saved});
      }
    }
  }
  ~LogitMask() {
    for (const auto& s : saved_) rwkv_hip_memcpy_h2d(s.first, &s.second, sizeof(float));
  }
  LogitMask(const LogitMask&) = delete;
  LogitMask& operator=(const LogitMask&) = delete;

 private:
  DeviceLogits& logits_;
  std::vector<std::pair<float*, float>> saved_;
};

std::vector<int> sample_rows(DeviceLogits& logits, SamplerPenaltyState& penalties, const GenerateOptions& options,
                             int step) {
  if (!mask_applies(options, step)) return sample_batch_repetition_temperature_topk_topp(logits, penalties, options);
  LogitMask mask(logits);
  return sample_batch_repetition_temperature_topk_topp(logits, penalties, options);
}

int sample_row(DeviceLogits& logits, SamplerPenaltyState& penalties, const GenerateOptions& options, int step) {
  if (logits.rows != 1) throw std::runtime_error("sampler currently expects a single logits row");
  return sample_rows(logits, penalties, options, step).front();
}

bool is_stop_token(const GenerateOptions& options, int token) {
  return std::find(options.stop_tokens.begin(), options.stop_tokens.end(), token) != options.stop_tokens.end();
}

// ---- UTF-8-safe text assembly -----------------------------------------------------------------------------------

// Well-formed UTF-8 (Unicode table 3-7): sequence length by lead byte and the allowed range of the second
// byte; further bytes are always 80..BF.  Length 0 marks a byte that cannot start a sequence.
struct Utf8Lead {
  int length;
  unsigned char second_lo, second_hi;
};

Utf8Lead utf8_lead(unsigned char b) {
  if (b <= 0x7F) return {1, 0, 0};
  if (b >= 0xC2 && b <= 0xDF) return {2, 0x80, 0xBF};
  if (b == 0xE0) return {3, 0xA0, 0xBF};
  if (b == 0xED) return {3, 0x80, 0x9F};
  if (b >= 0xE1 && b <= 0xEF) return {3, 0x80, 0xBF};
  if (b == 0xF0) return {4, 0x90, 0xBF};
  if (b == 0xF4) return {4, 0x80, 0x8F};
  if (b >= 0xF1 && b <= 0xF3) return {4, 0x80, 0xBF};
  return {0, 0, 0};
}

// Byte stream -> text that always ends on a character boundary.  A byte that cannot be part of a well-formed
// sequence becomes U+FFFD; an incomplete sequence at the end waits for more bytes, or is dropped on flush.
class Utf8Assembler {
 public:
  void push(const std::string& bytes) { pending_ += bytes; }

  std::string take(bool flush) {
    static const char kReplacement[] = "\xEF\xBF\xBD";
    std::string out;
    std::size_t i = 0;
    while (i < pending_.size()) {
      const Utf8Lead lead = utf8_lead(static_cast<unsigned char>(pending_[i]));
      if (lead.length == 0) {
        out += kReplacement;
        ++i;
        continue;
      }
      if (i + lead.length > pending_.size()) break;  // sequence still incomplete
      bool good = true;
      for (int k = 1; k < lead.length && good; ++k) {
        const auto c = static_cast<unsigned char>(pending_[i + k]);
        good = k == 1 ? (c >= lead.second_lo && c <= lead.second_hi) : (c >= 0x80 && c <= 0xBF);
      }
      if (!good) {
        out += kReplacement;
        ++i;
        continue;
      }
      out.append(pending_, i, lead.length);
      i += lead.length;
    }
    pending_.erase(0, i);
    if (flush) pending_.clear();
    return out;
  }

 private:
  std::string pending_;
};

// Per-stream text channel: tokens collect until `chunk_size` of them are waiting, then decode into the assembler.
class TokenStream {
 public:
  TokenStream(const TrieTokenizer& tokenizer, int chunk_size) : tokenizer_(tokenizer), chunk_size_(chunk_size) {}

  // Returns the text that became ready with this token (possibly empty).
  std::string add(int token) {
    waiting_.push_back(token);
    if (chunk_size_ <= 0 || static_cast<int>(waiting_.size()) < chunk_size_) return {};
    text_.push(tokenizer_.decode(waiting_));
    waiting_.clear();
    return text_.take(false);
  }

  std::string finish() {
    if (!waiting_.empty()) {
      text_.push(tokenizer_.decode(waiting_));
      waiting_.clear();
    }
    return text_.take(true);
  }

 private:
  const TrieTokenizer& tokenizer_;
  int chunk_size_;
  std::vector<int> waiting_;
  Utf8Assembler text_;
};

}  // namespace

InferenceEngine::InferenceEngine(std::shared_ptr<IModelBackend> model, std::shared_ptr<TrieTokenizer> tokenizer,
                                 std::string model_name, int prefill_chunk_size)
    : model_(std::move(model)),
      tokenizer_(std::move(tokenizer)),
      model_name_(std::move(model_name)),
      prefill_chunk_size_(prefill_chunk_size) {
  if (prefill_chunk_size_ <= 0) throw std::runtime_error("prefill chunk size must be positive");
}

std::vector<int64_t> InferenceEngine::encode_prompt(const std::string& prompt) const {
  const std::vector<int> ids = tokenizer_->encode(prompt);
  if (ids.empty()) throw std::runtime_error("prompt is empty after tokenization");
  return std::vector<int64_t>(ids.begin(), ids.end());
}

// Longest prompt first (stable), so that at any time the still-unfinished prompts are a prefix of the batch.
std::vector<std::vector<int64_t>> InferenceEngine::encode_prompts_sorted(const std::vector<std::string>& prompts,
                                                                         std::vector<size_t>& sorted_to_original) const {
  std::vector<std::vector<int64_t>> encoded;
  encoded.reserve(prompts.size());
  for (const std::string& p : prompts) encoded.push_back(encode_prompt(p));

  sorted_to_original.resize(prompts.size());
  std::iota(sorted_to_original.begin(), sorted_to_original.end(), size_t{0});
  std::stable_sort(sorted_to_original.begin(), sorted_to_original.end(),
                   [&](size_t a, size_t b) { return encoded[a].size() > encoded[b].size(); });

  std::vector<std::vector<int64_t>> sorted;
  sorted.reserve(prompts.size());
  for (size_t idx : sorted_to_original) sorted.push_back(std::move(encoded[idx]));
  return sorted;
}

// Every call to forward_prefill is rectangular: the rows that still have tokens left (a prefix, given the
// sort order) advance by min(shortest remainder among them, prefill_chunk_size).  Once some rows are done
// the rest run on a narrower state that is copied out of and back into the full one; the logits rows of
// finished prompts stay as their last chunk left them.
void InferenceEngine::prefill_batch_chunked(const std::vector<std::vector<int64_t>>& sorted_prompt_ids,
                                            GenerationState& state, DeviceLogits& logits) const {
  const int batch = static_cast<int>(sorted_prompt_ids.size());
  if (batch <= 0) throw std::runtime_error("prefill batch must not be empty");
  if (state.batch_size != batch) throw std::runtime_error("prefill state batch size mismatch");

  std::vector<int> done(batch, 0);
  auto remaining = [&](int i) { return static_cast<int>(sorted_prompt_ids[i].size()) - done[i]; };
  bool have_full_logits = false;

  for (;;) {
    int active = 0;
    while (active < batch && remaining(active) > 0) ++active;
    if (active == 0) return;

    int step = prefill_chunk_size_;
    for (int i = 0; i < active; ++i) step = std::min(step, remaining(i));

    std::vector<std::vector<int64_t>> chunk;
    chunk.reserve(active);
    for (int i = 0; i < active; ++i) {
      const auto first = sorted_prompt_ids[i].begin() + done[i];
      chunk.emplace_back(first, first + step);
      done[i] += step;
    }

    if (active == batch) {
      model_->forward_prefill(chunk, state, logits);
      have_full_logits = true;
      continue;
    }
    GenerationState narrow = model_->create_state(active);
    model_->copy_state_slice(state, 0, narrow, 0, active);
    DeviceLogits narrow_logits;
    model_->forward_prefill(chunk, narrow, narrow_logits);
    model_->copy_state_slice(narrow, 0, state, 0, active);
    if (!have_full_logits) throw std::runtime_error("batched prefill logits were not initialized");
    model_->copy_logits_slice(narrow_logits, 0, logits, 0, active);
  }
}

int InferenceEngine::prefill_prompt(const std::string& prompt, GenerationState& state, DeviceLogits& logits) const {
  std::vector<std::vector<int64_t>> one{encode_prompt(prompt)};
  prefill_batch_chunked(one, state, logits);
  return static_cast<int>(one.front().size());
}

// Single-row loop with an optional emitter.  The returned text is the concatenation of every generated
// token's bytes (no UTF-8 repair); a refusing emitter ends the call at once, without the final flush.
std::string InferenceEngine::generate_one(const std::string& prompt, GenerationState& state,
                                          const GenerateOptions& options, const StreamCallback* emit,
                                          int stream_index, int chunk_size, const ControlCallback& should_stop) const {
  DeviceLogits logits;
  prefill_prompt(prompt, state, logits);

  std::string text;
  TokenStream stream(*tokenizer_, emit ? chunk_size : 0);
  SamplerPenaltyState penalties = make_sampler_penalties(model_->vocab_size());
  for (int step = 0; step < options.max_tokens; ++step) {
    if (should_stop && should_stop()) break;
    const int token = sample_row(logits, penalties, options, step);
    if (is_stop_token(options, token)) break;
    text += tokenizer_->decode(token);
    const std::string ready = stream.add(token);
    if (emit && !ready.empty() && !(*emit)(stream_index, ready)) return text;
    model_->forward_decode({static_cast<int64_t>(token)}, state, logits);
  }
  if (emit) {
    const std::string tail = stream.finish();
    if (!tail.empty()) (*emit)(stream_index, tail);
  }
  return text;
}

namespace {

// Gathers the slots listed in `keep` (ascending) to the front of a state, a sampler state and a feed vector of
// width keep.size(); `rows` maps a slot to its prompt.  Runs of neighbouring slots move with one slice copy.
void gather_live_slots(const IModelBackend& model, const std::vector<int>& keep, GenerationState& state,
                       SamplerPenaltyState& penalties, std::vector<size_t>& rows, std::vector<int64_t>& feed) {
  const int width = static_cast<int>(keep.size());
  GenerationState narrow = model.create_state(width);
  SamplerPenaltyState narrow_penalties = make_sampler_penalties(penalties.vocab_size, width, penalties.seed);
  narrow_penalties.step = penalties.step;
  const std::size_t row_bytes = static_cast<std::size_t>(penalties.vocab_size) * sizeof(float);
  for (int to = 0; to < width;) {
    int run = 1;
    while (to + run < width && keep[to + run] == keep[to] + run) ++run;
    model.copy_state_slice(state, keep[to], narrow, to, run);
    rwkv7_fast_v4::check_hip(
        rwkv_hip_memcpy_d2d(narrow_penalties.penalties.p + static_cast<std::size_t>(to) * penalties.vocab_size,
                            penalties.penalties.p + static_cast<std::size_t>(keep[to]) * penalties.vocab_size,
                            run * row_bytes),
        "gather sampler penalties");
    to += run;
  }
  std::vector<size_t> new_rows(width);
  std::vector<int64_t> new_feed(width);
  for (int to = 0; to < width; ++to) {
    new_rows[to] = rows[keep[to]];
    new_feed[to] = feed[keep[to]];
  }
  state = std::move(narrow);
  penalties = std::move(narrow_penalties);
  rows.swap(new_rows);
  feed.swap(new_feed);
}

// slots of the current width whose prompt has not finished
std::vector<int> live_slots(const std::vector<size_t>& rows, const std::vector<char>& finished) {
  std::vector<int> keep;
  for (size_t slot = 0; slot < rows.size(); ++slot)
    if (!finished[rows[slot]]) keep.push_back(static_cast<int>(slot));
  return keep;
}

}  // namespace

std::vector<std::string> InferenceEngine::batch_generate(const std::vector<std::string>& prompts,
                                                         const GenerateOptions& options) const {
  if (prompts.empty()) return {};
  std::vector<size_t> order;
  const auto sorted_ids = encode_prompts_sorted(prompts, order);
  const int batch = static_cast<int>(prompts.size());

  GenerationState state = model_->create_state(batch);
  DeviceLogits logits;
  prefill_batch_chunked(sorted_ids, state, logits);

  // finished rows keep being fed a stop token so the batch stays rectangular
  const int64_t filler = options.stop_tokens.empty() ? 0 : options.stop_tokens.front();
  SamplerPenaltyState penalties = make_sampler_penalties(model_->vocab_size(), batch);
  std::vector<std::string> text(prompts.size());
  std::vector<char> finished(prompts.size(), 0);  // by prompt (sorted order)
  std::vector<int64_t> feed(prompts.size(), filler);
  std::vector<size_t> rows(prompts.size());       // slot of the current batch -> prompt
  std::iota(rows.begin(), rows.end(), size_t(0));
  int active = batch;

  for (int step = 0; step < options.max_tokens && active > 0; ++step) {
    const std::vector<int> sampled = sample_rows(logits, penalties, options, step);
    for (size_t slot = 0; slot < sampled.size(); ++slot) {
      const size_t i = rows[slot];
      feed[slot] = filler;
      if (finished[i]) continue;
      if (is_stop_token(options, sampled[slot])) {
        finished[i] = 1;
        --active;
        continue;
      }
      feed[slot] = sampled[slot];
      text[i] += tokenizer_->decode(sampled[slot]);
    }
    if (active == 0) break;
    if (shrink_batch_ && 2 * active <= static_cast<int>(rows.size()))
      gather_live_slots(*model_, live_slots(rows, finished), state, penalties, rows, feed);
    model_->forward_decode(feed, state, logits);
  }

  std::vector<std::string> outputs(prompts.size());
  for (size_t i = 0; i < text.size(); ++i) outputs[order[i]] = std::move(text[i]);
  return outputs;
}

std::vector<std::string> InferenceEngine::batch_generate_state(const std::vector<std::string>& prompts,
                                                               GenerationState& state,
                                                               const GenerateOptions& options) const {
  if (prompts.size() != 1 || state.batch_size != 1) {
    throw std::runtime_error("stateful generation only supports single prompt batch");
  }
  return {generate_one(prompts.front(), state, options, nullptr, 0, 0, {})};
}

void InferenceEngine::batch_generate_state_stream(const std::vector<std::string>& prompts, GenerationState& state,
                                                  const GenerateOptions& options, int chunk_size,
                                                  const StreamCallback& emit,
                                                  const ControlCallback& should_stop) const {
  if (prompts.size() != 1 || state.batch_size != 1) {
    throw std::runtime_error("stateful generation only supports single prompt batch");
  }
  generate_one(prompts.front(), state, options, &emit, 0, chunk_size, should_stop);
}

InferenceEngine::GenerationStats InferenceEngine::batch_generate_stream(
    const std::vector<std::string>& prompts, const GenerateOptions& options, int chunk_size,
    const StreamCallback& emit, const ControlCallback& should_stop, const StatsCallback& on_prefill_complete) const {
  GenerationStats stats;
  if (prompts.empty()) return stats;

  std::vector<size_t> order;
  const auto sorted_ids = encode_prompts_sorted(prompts, order);
  for (const auto& ids : sorted_ids) stats.prompt_tokens += static_cast<int>(ids.size());
  const int batch = static_cast<int>(prompts.size());

  GenerationState state = model_->create_state(batch);
  DeviceLogits logits;
  const auto prefill_t0 = Clock::now();
  prefill_batch_chunked(sorted_ids, state, logits);
  stats.prefill_seconds = seconds_since(prefill_t0);
  if (on_prefill_complete) on_prefill_complete(stats);

  const int64_t filler = options.stop_tokens.empty() ? 0 : options.stop_tokens.front();
  SamplerPenaltyState penalties = make_sampler_penalties(model_->vocab_size(), batch);
  std::vector<char> finished(prompts.size(), 0);  // by prompt (sorted order), as are the streams
  std::vector<int64_t> feed(prompts.size(), filler);
  std::vector<size_t> rows(prompts.size());       // slot of the current batch -> prompt
  std::iota(rows.begin(), rows.end(), size_t(0));
  std::vector<TokenStream> streams(prompts.size(), TokenStream(*tokenizer_, chunk_size));
  int active = batch;
  const auto decode_t0 = Clock::now();

  // emits to the caller's (unsorted) prompt index; false once the emitter refuses
  auto deliver = [&](size_t row, const std::string& piece) {
    if (piece.empty() || emit(static_cast<int>(order[row]), piece)) return true;
    stats.stopped = true;
    stats.decode_seconds = seconds_since(decode_t0);
    return false;
  };

  for (int step = 0; step < options.max_tokens && active > 0; ++step) {
    if (should_stop && should_stop()) {
      stats.stopped = true;
      break;
    }
    const std::vector<int> sampled = sample_rows(logits, penalties, options, step);
    for (size_t slot = 0; slot < sampled.size(); ++slot) {
      const size_t i = rows[slot];
      feed[slot] = filler;
      if (finished[i]) continue;
      if (is_stop_token(options, sampled[slot])) {
        finished[i] = 1;
        stats.stop_token = true;
        --active;
        if (!deliver(i, streams[i].finish())) return stats;
        continue;
      }
      ++stats.generated_tokens;
      feed[slot] = sampled[slot];
      if (!deliver(i, streams[i].add(sampled[slot]))) return stats;
    }
    if (active == 0) break;
    if (shrink_batch_ && 2 * active <= static_cast<int>(rows.size()))
      gather_live_slots(*model_, live_slots(rows, finished), state, penalties, rows, feed);
    model_->forward_decode(feed, state, logits);
  }

  for (size_t i = 0; i < prompts.size(); ++i) {
    if (!deliver(i, streams[i].finish())) return stats;
  }
  stats.decode_seconds = seconds_since(decode_t0);
  return stats;
}

InferenceEngine::GenerationStats InferenceEngine::generate_from_logits_stream(
    GenerationState& state, DeviceLogits& logits, const GenerateOptions& options, int chunk_size,
    const StreamCallback& emit, const ControlCallback& should_stop) const {
  if (state.batch_size != 1 || logits.rows != 1) {
    throw std::runtime_error("logit continuation only supports single prompt batch");
  }
  GenerationStats stats;
  TokenStream stream(*tokenizer_, chunk_size);
  SamplerPenaltyState penalties = make_sampler_penalties(model_->vocab_size());
  const auto decode_t0 = Clock::now();

  for (int step = 0; step < options.max_tokens; ++step) {
    if (should_stop && should_stop()) {
      stats.stopped = true;
      break;
    }
    const int token = sample_row(logits, penalties, options, step);
    if (is_stop_token(options, token)) {
      stats.stop_token = true;
      break;
    }
    ++stats.generated_tokens;
    const std::string ready = stream.add(token);
    if (!ready.empty() && !emit(0, ready)) {
      stats.stopped = true;
      break;
    }
    model_->forward_decode({static_cast<int64_t>(token)}, state, logits);
  }
  const std::string tail = stream.finish();
  if (!tail.empty() && !emit(0, tail)) stats.stopped = true;
  stats.decode_seconds = seconds_since(decode_t0);
  return stats;
}

std::string InferenceEngine::format_openai_prompt(const std::string& system,
                                                  const std::vector<std::pair<std::string, std::string>>& messages,
                                                  ThinkType think_type) const {
  const ThinkStyle style = think_style(think_type);
  // the footer goes on the last message whose role is "User"
  size_t footer_at = messages.size();
  if (!style.user_footer.empty()) {
    for (size_t i = messages.size(); i-- > 0;) {
      if (messages[i].first == "User") {
        footer_at = i;
        break;
      }
    }
  }
  std::string out;
  if (!system.empty()) out = "System: " + system + "\n\n";
  for (size_t i = 0; i < messages.size(); ++i) {
    out += messages[i].first + ": " + messages[i].second;
    if (i == footer_at) out += style.user_footer;
    out += "\n\n";
  }
  return out + "Assistant: " + style.assistant_header;
}

std::string InferenceEngine::format_openai_prompt(const std::string& system,
                                                  const std::vector<std::pair<std::string, std::string>>& messages,
                                                  bool enable_think) const {
  return format_openai_prompt(system, messages, enable_think ? ThinkType::Free : ThinkType::Fast);
}

int InferenceEngine::count_tokens(const std::string& text) const {
  return static_cast<int>(tokenizer_->encode(text).size());
}

}  // namespace rwkv7_server
