// Host API checks that need no GPU: tokenizer (cases of the reference's test/tokenizer_test.cpp plus the
// vocabulary-literal forms), prompt templates and argument errors of the engine
// (test/inference_engine_test.cpp:53-86 in the reference).
#include <fstream>

#include "rwkv_inference_engine.hpp"
#include "scripted_backend.hpp"

using namespace rwkv7_server;

namespace {

std::shared_ptr<TrieTokenizer> load_tokenizer() {
  auto tok = std::make_shared<TrieTokenizer>();
  CHECK_EQ(tok->load(host_test::vocab_path()), kTokenizerSuccess);
  return tok;
}

std::string temp_file(const std::string& name, const std::string& content) {
  const std::string path = "/tmp/rwkv_host_cpu_test_" + name;
  std::ofstream(path, std::ios::binary) << content;
  return path;
}

}  // namespace

HOST_TEST(tokenizer_load_errors_and_reload) {
  TrieTokenizer tok;
  CHECK_EQ(tok.load("/definitely/missing_vocab.txt"), kTokenizerError);
  CHECK_EQ(tok.load(host_test::vocab_path()), kTokenizerSuccess);
  CHECK_EQ(tok.load(host_test::vocab_path()), kTokenizerSuccess);  // loading twice is fine
  CHECK_EQ(tok.load(temp_file("bad_len", "1 'ab' 3\n")), kTokenizerError);     // declared length is wrong
  CHECK_EQ(tok.load(temp_file("bad_lit", "1 ab 2\n")), kTokenizerError);       // not a Python literal
  CHECK_EQ(tok.load(temp_file("bad_esc", "1 '\\q' 1\n")), kTokenizerError);    // unknown escape
  CHECK_EQ(tok.load(temp_file("empty", "")), kTokenizerError);
}

HOST_TEST(tokenizer_round_trips) {
  auto tok = load_tokenizer();
  const std::vector<std::string> samples{
      "hello world", "System: test\n\nUser: hi\n\nAssistant:", "\xE4\xB8\xAD\xE6\x96\x87\xE6\xB5\x8B\xE8\xAF\x95"
      "\xEF\xBC\x9A\xE4\xBD\xA0\xE5\xA5\xBD\xEF\xBC\x8C\xE4\xB8\x96\xE7\x95\x8C\xEF\xBC\x81",
      "line1\nline2\n\nline3", std::string("nul\0byte", 8), "\xF0\x9F\x98\x80 ok \xFF\xFE raw"};
  for (const std::string& s : samples) {
    const auto ids = tok->encode(s);
    CHECK(!ids.empty());
    CHECK_EQ(tok->decode(ids), s);
    CHECK_EQ(tok->decode(ids.front()), tok->decode(std::vector<int>{ids.front()}));
  }
  CHECK(tok->encode("").empty());
  CHECK_EQ(tok->decode(99999), std::string());  // unknown id decodes to nothing
}

HOST_TEST(tokenizer_is_greedy_longest_match) {
  auto tok = load_tokenizer();
  // single bytes are id = byte + 1
  CHECK_EQ(tok->encode("o"), std::vector<int>{112});
  CHECK_EQ(tok->encode("opq"), (std::vector<int>{112, 113, 114}));
  // " the" is one token although " t", " th", "th", "the", "he" all exist
  const auto the = tok->encode(" the");
  CHECK_EQ(the.size(), std::size_t(1));
  CHECK_EQ(tok->decode(the.front()), std::string(" the"));
  // "theX": longest prefix "the", then the byte
  const auto thex = tok->encode("theX");
  CHECK_EQ(thex.size(), std::size_t(2));
  CHECK_EQ(tok->decode(thex[0]), std::string("the"));
  CHECK_EQ(thex[1], int('X') + 1);
  // 中文 exists as one 6-byte token and wins over 中 + 文
  CHECK_EQ(tok->encode("\xE4\xB8\xAD\xE6\x96\x87").size(), std::size_t(1));
  // a dangling partial sequence falls back on the 2-byte bytes token b'\xe4\xb8'
  const auto part = tok->encode("\xE4\xB8");
  CHECK_EQ(part.size(), std::size_t(1));
  CHECK_EQ(tok->decode(part), std::string("\xE4\xB8"));
}

HOST_TEST(tokenizer_literal_forms) {
  // the escape forms that Python's repr() produces for str and bytes
  TrieTokenizer tok;
  const std::string vocab =
      "1 'a' 1\n"
      "2 '\\n' 1\n"
      "3 '\\t\\\\' 2\n"
      "4 \"'\" 1\n"
      "5 '\\'\"' 2\n"
      "6 b'\\xe4\\xb8' 2\n"
      "7 '\\x7f' 1\n"
      "8 '\\xe9' 2\n"          // str: U+00E9 -> 2 UTF-8 bytes
      "9 b'\\xe9' 1\n"         // bytes: the byte itself
      "10 '\\u4e2d' 3\n"
      "11 '\\U0001f600' 4\n"
      "12 'x y' 3\n"           // spaces inside the literal
      "13 b'\\\\' 1\r\n";      // CRLF line ending
  CHECK_EQ(tok.load(temp_file("forms", vocab)), kTokenizerSuccess);
  CHECK_EQ(tok.decode(2), std::string("\n"));
  CHECK_EQ(tok.decode(3), std::string("\t\\"));
  CHECK_EQ(tok.decode(4), std::string("'"));
  CHECK_EQ(tok.decode(5), std::string("'\""));
  CHECK_EQ(tok.decode(6), std::string("\xE4\xB8"));
  CHECK_EQ(tok.decode(7), std::string("\x7F"));
  CHECK_EQ(tok.decode(8), std::string("\xC3\xA9"));
  CHECK_EQ(tok.decode(9), std::string("\xE9"));
  CHECK_EQ(tok.decode(10), std::string("\xE4\xB8\xAD"));
  CHECK_EQ(tok.decode(11), std::string("\xF0\x9F\x98\x80"));
  CHECK_EQ(tok.decode(12), std::string("x y"));
  CHECK_EQ(tok.decode(13), std::string("\\"));
  CHECK_EQ(tok.encode("x y"), std::vector<int>{12});
  // bytes with no token at all are skipped
  CHECK_EQ(tok.encode("aZa"), (std::vector<int>{1, 1}));
}

HOST_TEST(prompt_templates) {
  auto tok = load_tokenizer();
  auto backend = std::make_shared<host_test::ScriptedBackend>(std::vector<std::vector<float>>{{0.f, 1.f}}, "fake");
  InferenceEngine engine(backend, tok, backend->model_name());
  CHECK_EQ(engine.prefill_chunk_size(), 128);
  CHECK_EQ(engine.model_name(), std::string("fake"));
  using Msgs = std::vector<std::pair<std::string, std::string>>;
  // The reference's source gives the Fast header as "<think>\n</think" (src/rwkv_inference_engine.cpp:30);
  // its test file expects "<think></think" (test/inference_engine_test.cpp:73), which that source cannot
  // produce.  The source is followed here.
  CHECK_EQ(engine.format_openai_prompt("SYS", Msgs{{"User", "Q1"}, {"Assistant", "A1"}, {"User", "Q2"}}, false),
           std::string("System: SYS\n\nUser: Q1\n\nAssistant: A1\n\nUser: Q2\n\nAssistant: <think>\n</think"));
  CHECK_EQ(engine.format_openai_prompt("SYS", Msgs{{"User", "Q"}}, true),
           std::string("System: SYS\n\nUser: Q\n\nAssistant: <think"));
  CHECK_EQ(engine.format_openai_prompt("SYS", Msgs{{"User", "Q"}}, ThinkType::EnShort),
           std::string("System: SYS\n\nUser: Q (think a bit)\n\nAssistant: <think"));
  CHECK_EQ(engine.format_openai_prompt("", Msgs{{"User", "Q"}}, ThinkType::En),
           std::string("User: Q (think)\n\nAssistant: <think"));
  // the footer goes on the LAST User message only, also when an Assistant message follows it
  CHECK_EQ(engine.format_openai_prompt("", Msgs{{"User", "A"}, {"User", "B"}, {"Assistant", "C"}}, ThinkType::EnLong),
           std::string("User: A\n\nUser: B (think a lot)\n\nAssistant: C\n\nAssistant: <think"));
  CHECK_EQ(engine.format_openai_prompt("", Msgs{}, ThinkType::PreferChinese),
           std::string("Assistant: <think>\xE5\x97\xAF"));
  CHECK_EQ(engine.format_openai_prompt("S", Msgs{}, ThinkType::Free), std::string("System: S\n\nAssistant: <think"));
}

HOST_TEST(engine_argument_errors) {
  auto tok = load_tokenizer();
  auto backend = std::make_shared<host_test::ScriptedBackend>(std::vector<std::vector<float>>{{0.f, 1.f}}, "fake");
  CHECK_THROWS(InferenceEngine(backend, tok, "bad", 0), "prefill chunk size must be positive");
  CHECK_THROWS(InferenceEngine(backend, tok, "bad", -4), "prefill chunk size must be positive");
  InferenceEngine engine(backend, tok, "fake");
  const std::string answer = "This is a test answer.";
  CHECK_EQ(engine.count_tokens(answer), int(tok->encode(answer).size()));
  CHECK_EQ(engine.count_tokens(""), 0);

  GenerationState two;
  two.batch_size = 2;
  auto emit = [](int, const std::string&) { return true; };
  CHECK_THROWS(engine.batch_generate_state({"prompt"}, two, GenerateOptions{}), "single prompt batch");
  CHECK_THROWS(engine.batch_generate_state_stream({"prompt", "prompt"}, two, GenerateOptions{}, 1, emit),
               "single prompt batch");
  DeviceLogits logits;
  logits.rows = 1;
  CHECK_THROWS(engine.generate_from_logits_stream(two, logits, GenerateOptions{}, 1, emit), "single prompt batch");
  CHECK(engine.batch_generate({}, GenerateOptions{}).empty());
  CHECK_EQ(engine.batch_generate_stream({}, GenerateOptions{}, 1, emit).prompt_tokens, 0);
  // a prompt with no encodable byte is refused before the backend is touched
  CHECK_THROWS(engine.batch_generate({""}, GenerateOptions{}), "prompt is empty after tokenization");
  CHECK(backend->prefills.empty());
}

int main(int argc, char** argv) { return host_test::run_all(argc, argv, false); }

// ---- prefill admission (scenario of the reference's test/prefill_admission_test.cpp, plus ordering and ownership) ----
#include <atomic>
#include <chrono>
#include <future>
#include <thread>

#include "rwkv_prefill_admission.hpp"

namespace {

struct FakeCapacity {
  std::atomic<int> lanes{4};
  std::atomic<int> asked{0};
  PrefillAdmissionController::CapacityProvider provider() {
    return [this] {
      ++asked;
      PrefillCapacity c;
      c.max_batch_size = lanes.load();
      c.bytes_per_batch = 1024;
      c.free_vram_bytes = 4096;
      c.total_vram_bytes = 8192;
      return c;
    };
  }
};

template <class F>
bool still_waiting(std::future<F>& f, int ms = 250) {
  return f.wait_for(std::chrono::milliseconds(ms)) == std::future_status::timeout;
}

}  // namespace

HOST_TEST(admission_waits_for_lanes_and_follows_the_capacity) {
  FakeCapacity cap;
  PrefillAdmissionController ctl(cap.provider());
  auto first = ctl.acquire(3, "first");
  CHECK(first.has_value() && bool(*first));
  CHECK_EQ(first->batch_size(), 3);
  cap.lanes = 3;  // memory got tighter: 3 of 3 lanes are now taken
  auto waiter = std::async(std::launch::async, [&] { return ctl.acquire(1, "second"); });
  CHECK(still_waiting(waiter));
  auto snap = ctl.snapshot(true);
  CHECK_EQ(snap.hard_max_batch_size, 4);
  CHECK_EQ(snap.dynamic_max_batch_size, 3);
  CHECK_EQ(snap.reserved_batch_size, 3);
  CHECK_EQ(snap.queued_requests, std::size_t(1));
  CHECK_EQ(snap.capacity.bytes_per_batch, std::size_t(1024));
  first->release();
  CHECK(!bool(*first));
  auto second = waiter.get();
  CHECK(second.has_value());
  CHECK_EQ(second->batch_size(), 1);
  CHECK_EQ(ctl.snapshot(false).reserved_batch_size, 1);
  second->release();
  second->release();  // releasing twice gives nothing back twice
  CHECK_EQ(ctl.snapshot(false).reserved_batch_size, 0);
  CHECK(cap.asked.load() >= 4);  // constructor, head-of-queue checks, release
}

HOST_TEST(admission_rejects_what_can_never_fit) {
  FakeCapacity cap;
  PrefillAdmissionController ctl(cap.provider());
  cap.lanes = 16;  // more memory later does not raise the limit fixed at start-up
  bool threw = false;
  try {
    (void)ctl.acquire(5, "wide");
  } catch (const PrefillBatchLimitExceeded& e) {
    threw = true;
    CHECK_EQ(e.request_batch_size(), 5);
    CHECK_EQ(e.max_batch_size(), 4);
    CHECK_EQ(std::string(e.what()), std::string("bsz overflow, Max bsz=4"));
  }
  CHECK(threw);
  CHECK_EQ(ctl.snapshot(true).dynamic_max_batch_size, 4);
  CHECK_EQ(ctl.snapshot(false).queued_requests, std::size_t(0));
  auto one = ctl.acquire(0, "zero counts as one");
  CHECK(one.has_value());
  CHECK_EQ(one->batch_size(), 1);
  CHECK_THROWS(PrefillAdmissionController(PrefillAdmissionController::CapacityProvider{}), "capacity provider");
}

HOST_TEST(admission_cancelled_waiter_leaves_the_queue) {
  FakeCapacity cap;
  PrefillAdmissionController ctl(cap.provider());
  auto all = ctl.acquire(4, "all");
  CHECK(all.has_value());
  std::atomic<bool> cancel{false};
  auto waiter = std::async(std::launch::async, [&] { return ctl.acquire(1, "gives up", [&] { return cancel.load(); }); });
  CHECK(still_waiting(waiter));
  CHECK_EQ(ctl.snapshot(false).queued_requests, std::size_t(1));
  cancel = true;
  auto none = waiter.get();
  CHECK(!none.has_value());
  CHECK_EQ(ctl.snapshot(false).queued_requests, std::size_t(0));
  CHECK_EQ(ctl.snapshot(false).reserved_batch_size, 4);
}

HOST_TEST(admission_is_first_come_first_served) {
  FakeCapacity cap;
  PrefillAdmissionController ctl(cap.provider());
  auto held = ctl.acquire(2, "held");
  CHECK(held.has_value());
  // a 3-lane request queues first; the 1-lane request behind it would fit at once but must not overtake
  auto wide = std::async(std::launch::async, [&] { return ctl.acquire(3, "wide"); });
  while (ctl.snapshot(false).queued_requests < 1) std::this_thread::yield();
  auto narrow = std::async(std::launch::async, [&] { return ctl.acquire(1, "narrow"); });
  while (ctl.snapshot(false).queued_requests < 2) std::this_thread::yield();
  CHECK(still_waiting(wide));
  CHECK(still_waiting(narrow, 50));
  held->release();
  auto w = wide.get();
  CHECK(w.has_value());
  auto n = narrow.get();  // 3 + 1 fit together once the wide one is in
  CHECK(n.has_value());
  CHECK(w->ticket() < n->ticket());
  CHECK_EQ(ctl.snapshot(false).reserved_batch_size, 4);
}

HOST_TEST(admission_permit_owns_its_lanes) {
  FakeCapacity cap;
  PrefillAdmissionController ctl(cap.provider());
  {
    auto p = ctl.acquire(2, "scoped");
    CHECK(p.has_value());
    PrefillAdmissionController::Permit moved(std::move(*p));
    CHECK(!bool(*p) && bool(moved));
    CHECK_EQ(ctl.snapshot(false).reserved_batch_size, 2);
    auto q = ctl.acquire(1, "other");
    CHECK(q.has_value());
    moved = std::move(*q);  // assignment gives the 2 lanes back and takes over the 1
    CHECK_EQ(ctl.snapshot(false).reserved_batch_size, 1);
    CHECK_EQ(moved.batch_size(), 1);
  }
  CHECK_EQ(ctl.snapshot(false).reserved_batch_size, 0);  // destructors released the rest
}
