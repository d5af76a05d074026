// Engine control flow against a scripted backend (logits in device memory, sampled by the GPU sampler):
// the expectations of the reference's test/inference_engine_test.cpp:88-198 plus streaming/UTF-8/stop cases.
#include "rwkv_inference_engine.hpp"
#include "scripted_backend.hpp"

using namespace rwkv7_server;
using host_test::ScriptedBackend;

namespace {

const std::string kPrompt = "System: test\n\nUser: hi\n\nAssistant:";
const std::string kAnswer = "This is a test answer.";

std::shared_ptr<TrieTokenizer> tokenizer() {
  static std::shared_ptr<TrieTokenizer> tok = [] {
    auto t = std::make_shared<TrieTokenizer>();
    if (t->load(host_test::vocab_path()) != kTokenizerSuccess) throw std::runtime_error("vocab load failed");
    return t;
  }();
  return tok;
}

constexpr int kVocab = 400;

GenerateOptions greedy_options(int max_tokens) {
  GenerateOptions o;
  o.max_tokens = max_tokens;
  o.stop_tokens = {0};
  o.top_k = 0;
  o.top_p = 0.0;
  o.temperature = 1.0;
  o.alpha_presence = 0.0;
  o.alpha_frequency = 0.0;
  o.alpha_decay = 1.0;
  return o;
}

std::shared_ptr<ScriptedBackend> answer_backend(const std::vector<int>& ids, const char* name) {
  return std::make_shared<ScriptedBackend>(ScriptedBackend::script_for(ids, kVocab), name);
}

}  // namespace

HOST_TEST(prefill_chunks_hold_at_most_n_tokens) {
  auto tok = tokenizer();
  auto backend = answer_backend(tok->encode(kAnswer), "chunked");
  InferenceEngine engine(backend, tok, "chunked", 3);
  GenerationState state = backend->create_state(1);
  DeviceLogits logits;
  const std::string prompt = kPrompt + kPrompt + kPrompt;
  const int n = engine.prefill_prompt(prompt, state, logits);
  CHECK_EQ(n, int(tok->encode(prompt).size()));
  CHECK(n > 3);
  CHECK_EQ(backend->prefills.size(), std::size_t((n + 2) / 3));
  std::vector<int64_t> seen;
  for (const auto& call : backend->prefills) {
    CHECK_EQ(call.size(), std::size_t(1));
    CHECK(call[0].size() <= 3 && !call[0].empty());
    seen.insert(seen.end(), call[0].begin(), call[0].end());
  }
  const auto ids = tok->encode(prompt);
  CHECK(seen == std::vector<int64_t>(ids.begin(), ids.end()));  // every token once, in order
}

HOST_TEST(greedy_generation_reproduces_scripted_answer) {
  auto tok = tokenizer();
  const auto answer_ids = tok->encode(kAnswer);
  auto backend = answer_backend(answer_ids, "single");
  InferenceEngine engine(backend, tok, "single");
  const auto out = engine.batch_generate({kPrompt}, greedy_options(int(answer_ids.size()) + 1));
  CHECK_EQ(out.size(), std::size_t(1));
  CHECK_EQ(out[0], kAnswer);
  CHECK_EQ(backend->prefills.size(), std::size_t(1));
  CHECK_EQ(backend->prefills[0].size(), std::size_t(1));
  const auto prompt_ids = tok->encode(kPrompt);
  CHECK(backend->prefills[0][0] == std::vector<int64_t>(prompt_ids.begin(), prompt_ids.end()));
  // one decode per generated token, fed with that token; none after the stop token
  CHECK_EQ(backend->decodes.size(), answer_ids.size());
  for (std::size_t i = 0; i < answer_ids.size(); ++i) CHECK_EQ(backend->decodes[i], ScriptedBackend::Tokens{answer_ids[i]});
}

HOST_TEST(max_tokens_limits_generation) {
  auto tok = tokenizer();
  const auto answer_ids = tok->encode(kAnswer);
  auto backend = answer_backend(answer_ids, "limit");
  InferenceEngine engine(backend, tok, "limit");
  const auto out = engine.batch_generate({kPrompt}, greedy_options(3));
  CHECK_EQ(out[0], tok->decode(std::vector<int>(answer_ids.begin(), answer_ids.begin() + 3)));
  CHECK_EQ(backend->decodes.size(), std::size_t(3));  // the state also advances over the last kept token
}

namespace {
// Script of 3 steps preferring 'o','p','q' (112..114) at 90, with token 111 at 100 in step 1 and token 754 at
// 100 in step 2: unmasked greedy gives 112,111,754; with those two denied at steps 1 and 2 it gives "opq".
// (The reference's test uses a vocabulary of 755, which its own sampler refuses - sizes must be multiples of
// 4, src/utils/sampling.cu:492 - so 756 here.)
constexpr int kForceVocab = 756;
std::vector<std::vector<float>> force_script() {
  std::vector<std::vector<float>> rows;
  for (int i = 0; i < 3; ++i) {
    std::vector<float> row(kForceVocab, -100.0f);
    row[112 + i] = 90.0f;
    if (i == 1) row[111] = 100.0f;
    if (i == 2) row[754] = 100.0f;
    rows.push_back(row);
  }
  rows.push_back(host_test::one_hot(kForceVocab, 0));
  return rows;
}
}  // namespace

HOST_TEST(force_reasoning_masks_tokens_111_and_754_at_steps_1_and_2) {
  auto tok = tokenizer();
  GenerateOptions o = greedy_options(4);
  {
    auto backend = std::make_shared<ScriptedBackend>(force_script(), "force");
    InferenceEngine engine(backend, tok, "force");
    o.force_reasoning = true;
    CHECK_EQ(engine.batch_generate({kPrompt}, o)[0], std::string("opq"));
    CHECK_EQ(backend->decodes.size(), std::size_t(3));
  }
  {  // without the flag the denied tokens win: 'o', then 111 ('n'), then 754 (not in the vocabulary: no text)
    auto backend = std::make_shared<ScriptedBackend>(force_script(), "noforce");
    InferenceEngine engine(backend, tok, "noforce");
    o.force_reasoning = false;
    CHECK_EQ(engine.batch_generate({kPrompt}, o)[0], std::string("on"));
    CHECK_EQ(backend->decodes[1], ScriptedBackend::Tokens{111});
    CHECK_EQ(backend->decodes[2], ScriptedBackend::Tokens{754});
  }
  {  // an offset of 1 shifts the window to local steps 0 and 1: step 2 is no longer masked
    auto backend = std::make_shared<ScriptedBackend>(force_script(), "offset");
    InferenceEngine engine(backend, tok, "offset");
    o.force_reasoning = true;
    o.force_reasoning_token_offset = 1;
    engine.batch_generate({kPrompt}, o);
    CHECK_EQ(backend->decodes[0], ScriptedBackend::Tokens{112});
    CHECK_EQ(backend->decodes[1], ScriptedBackend::Tokens{113});
    CHECK_EQ(backend->decodes[2], ScriptedBackend::Tokens{754});
  }
  {  // the mask is undone after sampling: the logits buffer holds the scripted values again
    auto backend = std::make_shared<ScriptedBackend>(force_script(), "restore");
    InferenceEngine engine(backend, tok, "restore");
    GenerationState state = backend->create_state(1);
    DeviceLogits logits;
    engine.prefill_prompt(kPrompt, state, logits);
    o.force_reasoning_token_offset = 1;  // step 0 is masked
    o.max_tokens = 1;
    int calls = 0;
    engine.generate_from_logits_stream(state, logits, o, 1, [&](int, const std::string&) { ++calls; return false; });
    CHECK_EQ(calls, 1);
    // emit refused after the first token: no decode ran, logits are still script row 0
    CHECK(backend->decodes.empty());
    const auto host = host_test::to_host<float>(logits.values);
    CHECK_EQ(host[111], -100.0f);
    CHECK_EQ(host[754], -100.0f);
    CHECK_EQ(host[112], 90.0f);
  }
}

HOST_TEST(two_prompt_batch_prefills_width_2_then_1) {
  auto tok = tokenizer();
  const auto answer_ids = tok->encode(kAnswer);
  auto backend = answer_backend(answer_ids, "batch");
  InferenceEngine engine(backend, tok, "batch");
  const std::string longer = kPrompt + "\nextra";
  const auto out = engine.batch_generate({kPrompt, longer}, greedy_options(int(answer_ids.size()) + 1));
  CHECK_EQ(out.size(), std::size_t(2));
  CHECK_EQ(out[0], kAnswer);
  CHECK_EQ(out[1], kAnswer);
  CHECK_EQ(backend->prefills.size(), std::size_t(2));
  CHECK_EQ(backend->prefills[0].size(), std::size_t(2));
  CHECK_EQ(backend->prefills[1].size(), std::size_t(1));
  // rows are sorted longest first: row 0 of the first call starts the longer prompt, and both rows of a call
  // have the same length (the shorter prompt's)
  const auto short_ids = tok->encode(kPrompt);
  const auto long_ids = tok->encode(longer);
  CHECK_EQ(backend->prefills[0][0].size(), short_ids.size());
  CHECK_EQ(backend->prefills[0][1].size(), short_ids.size());
  CHECK_EQ(backend->prefills[1][0].size(), long_ids.size() - short_ids.size());
  CHECK_EQ(backend->state_slice_copies, 2);  // narrow state out and back
  CHECK_EQ(backend->decodes.size(), answer_ids.size());
  for (const auto& step : backend->decodes) CHECK_EQ(step.size(), std::size_t(2));
}

// With set_shrink_batch(true) the rows that are still generating are gathered into a narrower batch once at most
// half are left; the texts are those of the batch that never shrinks (the reference's behaviour, the default).
HOST_TEST(batch_shrinks_when_half_of_the_rows_have_finished) {
  auto tok = tokenizer();
  const auto answer_ids = tok->encode(kAnswer);
  const std::vector<int> short_ids(answer_ids.begin(), answer_ids.begin() + 2);
  const std::string short_text = tok->decode(short_ids);
  const auto options = greedy_options(int(answer_ids.size()) + 1);
  // row 0 (the longest prompt) answers kAnswer, every other row stops after two tokens
  const std::vector<std::string> prompts{kPrompt, kPrompt + "\nlonger than the others", kPrompt + " b", kPrompt + " c"};
  for (const bool streaming : {false, true}) {
    for (const bool shrink : {false, true}) {
      auto backend = answer_backend(answer_ids, "shrink");
      backend->set_script_for_other_rows(ScriptedBackend::script_for(short_ids, kVocab));
      InferenceEngine engine(backend, tok, "shrink");
      CHECK(!engine.shrink_batch());
      engine.set_shrink_batch(shrink);
      std::vector<std::string> out(prompts.size());
      if (streaming) {
        const auto stats = engine.batch_generate_stream(
            prompts, options, 1, [&](int i, const std::string& piece) { out[std::size_t(i)] += piece; return true; });
        CHECK_EQ(stats.generated_tokens, int(answer_ids.size()) + 3 * 2);
      } else {
        out = engine.batch_generate(prompts, options);
      }
      CHECK_EQ(out[1], kAnswer);  // the caller's index of the longest prompt
      CHECK_EQ(out[0], short_text);
      CHECK_EQ(out[2], short_text);
      CHECK_EQ(out[3], short_text);
      CHECK_EQ(backend->decodes.size(), answer_ids.size());
      // steps 0 and 1 feed all four rows; at step 2 three rows stop, and from then on the batch is one row wide
      // (or stays at four rows fed the stop token)
      for (std::size_t step = 0; step < backend->decodes.size(); ++step) {
        const std::size_t expect = (shrink && step >= 2) ? 1 : 4;
        CHECK_EQ(backend->decodes[step].size(), expect);
      }
      if (shrink) CHECK_EQ(backend->decodes.back()[0], int64_t(answer_ids.back()));
    }
  }
}

HOST_TEST(streaming_routes_chunks_to_the_callers_prompt_index) {
  auto tok = tokenizer();
  const auto answer_ids = tok->encode(kAnswer);
  const auto options = greedy_options(int(answer_ids.size()) + 1);
  {
    auto backend = answer_backend(answer_ids, "stream");
    InferenceEngine engine(backend, tok, "stream");
    std::string text;
    std::vector<int> indices;
    int prefill_reports = 0;
    const auto stats = engine.batch_generate_stream(
        {kPrompt}, options, 1,
        [&](int i, const std::string& s) { indices.push_back(i); text += s; return true; }, {},
        [&](const InferenceEngine::GenerationStats& s) {
          ++prefill_reports;
          CHECK_EQ(s.prompt_tokens, int(tok->encode(kPrompt).size()));
          CHECK_EQ(s.generated_tokens, 0);
        });
    CHECK_EQ(text, kAnswer);
    CHECK_EQ(indices.size(), answer_ids.size());  // chunk size 1: one emit per token
    for (int i : indices) CHECK_EQ(i, 0);
    CHECK_EQ(prefill_reports, 1);
    CHECK_EQ(stats.generated_tokens, int(answer_ids.size()));
    CHECK(stats.stop_token);
    CHECK(!stats.stopped);
  }
  {
    auto backend = answer_backend(answer_ids, "stream-batch");
    InferenceEngine engine(backend, tok, "stream-batch");
    std::vector<std::string> text(2);
    // the longer prompt is given FIRST here, the shorter second: indices must follow the caller's order
    const auto stats = engine.batch_generate_stream({kPrompt + "\nextra", kPrompt}, options, 4,
                                                    [&](int i, const std::string& s) { text.at(i) += s; return true; });
    CHECK_EQ(text[0], kAnswer);
    CHECK_EQ(text[1], kAnswer);
    CHECK_EQ(backend->prefills.size(), std::size_t(2));
    CHECK_EQ(backend->prefills[0].size(), std::size_t(2));
    CHECK_EQ(backend->prefills[1].size(), std::size_t(1));
    CHECK_EQ(stats.generated_tokens, 2 * int(answer_ids.size()));
  }
  {
    // Rows that differ: sorted row 0 (the longer prompt, given SECOND by the caller) answers kAnswer, sorted
    // row 1 (the shorter prompt, caller index 0) answers " hi" and stops after one token.
    auto backend = answer_backend(answer_ids, "stream-routing");
    const int hi = tok->encode(" hi").front();
    backend->set_script_for_other_rows(ScriptedBackend::script_for({hi}, kVocab));
    InferenceEngine engine(backend, tok, "stream-routing");
    std::vector<std::string> text(2);
    const auto stats = engine.batch_generate_stream({kPrompt, kPrompt + "\nextra"}, options, 2,
                                                    [&](int i, const std::string& s) { text.at(i) += s; return true; });
    CHECK_EQ(text[0], std::string(" hi"));
    CHECK_EQ(text[1], kAnswer);
    CHECK_EQ(stats.generated_tokens, int(answer_ids.size()) + 1);
    // the finished row keeps being fed the first stop token
    CHECK_EQ(backend->decodes.size(), answer_ids.size());
    CHECK_EQ(backend->decodes[0], (ScriptedBackend::Tokens{answer_ids[0], hi}));
    for (std::size_t i = 1; i < backend->decodes.size(); ++i)
      CHECK_EQ(backend->decodes[i], (ScriptedBackend::Tokens{answer_ids[i], 0}));
    // same routing without streaming
    auto backend2 = answer_backend(answer_ids, "batch-routing");
    backend2->set_script_for_other_rows(ScriptedBackend::script_for({hi}, kVocab));
    InferenceEngine engine2(backend2, tok, "batch-routing");
    const auto out = engine2.batch_generate({kPrompt, kPrompt + "\nextra"}, options);
    CHECK_EQ(out[0], std::string(" hi"));
    CHECK_EQ(out[1], kAnswer);
  }
}

HOST_TEST(streaming_stops_on_control_callback_and_on_refusing_emitter) {
  auto tok = tokenizer();
  const auto answer_ids = tok->encode(kAnswer);
  const auto options = greedy_options(int(answer_ids.size()) + 1);
  {
    auto backend = answer_backend(answer_ids, "ctl");
    InferenceEngine engine(backend, tok, "ctl");
    int polls = 0;
    std::string text;
    const auto stats = engine.batch_generate_stream(
        {kPrompt}, options, 1, [&](int, const std::string& s) { text += s; return true; },
        [&] { return ++polls > 2; });
    CHECK(stats.stopped);
    CHECK(!stats.stop_token);
    CHECK_EQ(stats.generated_tokens, 2);
    CHECK_EQ(text, tok->decode(std::vector<int>(answer_ids.begin(), answer_ids.begin() + 2)));
  }
  {
    auto backend = answer_backend(answer_ids, "refuse");
    InferenceEngine engine(backend, tok, "refuse");
    int emits = 0;
    const auto stats =
        engine.batch_generate_stream({kPrompt}, options, 1, [&](int, const std::string&) { return ++emits < 3; });
    CHECK(stats.stopped);
    CHECK_EQ(emits, 3);
    CHECK_EQ(stats.generated_tokens, 3);
    CHECK_EQ(backend->decodes.size(), std::size_t(2));  // no forward after the refusal
  }
  {  // stateful single-prompt stream: state and penalties are the caller's, same text
    auto backend = answer_backend(answer_ids, "stateful");
    InferenceEngine engine(backend, tok, "stateful");
    GenerationState state = backend->create_state(1);
    std::string text;
    engine.batch_generate_state_stream({kPrompt}, state, options, 5,
                                       [&](int i, const std::string& s) { CHECK_EQ(i, 0); text += s; return true; });
    CHECK_EQ(text, kAnswer);
    auto backend2 = answer_backend(answer_ids, "stateful2");
    InferenceEngine engine2(backend2, tok, "stateful2");
    GenerationState state2 = backend2->create_state(1);
    CHECK_EQ(engine2.batch_generate_state({kPrompt}, state2, options), std::vector<std::string>{kAnswer});
  }
}

HOST_TEST(stream_text_never_splits_a_character) {
  auto tok = tokenizer();
  // bytes of "中" (E4 B8 AD) arrive as token b'\xe4\xb8' + byte token AD; then a lone continuation byte (invalid),
  // then "é" split over two byte tokens, then an unfinished 4-byte lead at the very end (dropped on flush).
  const int t_e4b8 = tok->encode("\xE4\xB8").front();
  const std::vector<int> ids{t_e4b8, 0xAD + 1, 0x80 + 1, 0xC3 + 1, 0xA9 + 1, int('!') + 1, 0xF0 + 1};
  auto backend = answer_backend(ids, "utf8");
  InferenceEngine engine(backend, tok, "utf8");
  std::vector<std::string> pieces;
  const auto stats = engine.batch_generate_stream({kPrompt}, greedy_options(int(ids.size()) + 1), 1,
                                                  [&](int, const std::string& s) { pieces.push_back(s); return true; });
  CHECK_EQ(stats.generated_tokens, int(ids.size()));
  const std::vector<std::string> want{"\xE4\xB8\xAD", "\xEF\xBF\xBD", "\xC3\xA9", "!"};
  CHECK(pieces == want);
  // the non-streaming call returns the raw bytes of every token, unrepaired
  auto backend2 = answer_backend(ids, "utf8-raw");
  InferenceEngine engine2(backend2, tok, "utf8-raw");
  CHECK_EQ(engine2.batch_generate({kPrompt}, greedy_options(int(ids.size()) + 1))[0],
           std::string("\xE4\xB8\xAD\x80\xC3\xA9!\xF0"));
}

HOST_TEST(continuation_from_logits) {
  auto tok = tokenizer();
  const auto answer_ids = tok->encode(kAnswer);
  auto backend = answer_backend(answer_ids, "cont");
  InferenceEngine engine(backend, tok, "cont");
  GenerationState state = backend->create_state(1);
  DeviceLogits logits;
  engine.prefill_prompt(kPrompt, state, logits);
  std::string text;
  const auto stats = engine.generate_from_logits_stream(state, logits, greedy_options(100), 3,
                                                        [&](int, const std::string& s) { text += s; return true; });
  CHECK_EQ(text, kAnswer);
  CHECK(stats.stop_token);
  CHECK_EQ(stats.generated_tokens, int(answer_ids.size()));
}

int main(int argc, char** argv) { return host_test::run_all(argc, argv, true); }
