// ModelBackend over the kernel library (synthetic tiny model): state and logits shapes, argument errors with
// the reference's messages (src/rwkv_server_backend.cpp:1399-1580), slice copies, and the engine end to end.
#include <algorithm>
#include <cstring>
#include <thread>

#include "rwkv_hip.h"
#include "rwkv_inference_engine.hpp"
#include "rwkv_prefill_admission.hpp"
#include "test_common.hpp"

using namespace rwkv7_server;

namespace {

std::shared_ptr<ModelBackend> tiny() {
  static auto backend = std::make_shared<ModelBackend>("synthetic:tiny:w8:seed=3", true);
  return backend;
}

std::vector<int64_t> ramp(int n, int start) {
  std::vector<int64_t> v;
  for (int i = 0; i < n; ++i) v.push_back((start + 37 * i) % 2048);
  return v;
}

double cosine(const std::vector<float>& a, const std::vector<float>& b, std::size_t off_a, std::size_t off_b,
              std::size_t n) {
  double ab = 0, aa = 0, bb = 0;
  for (std::size_t i = 0; i < n; ++i) {
    ab += double(a[off_a + i]) * b[off_b + i];
    aa += double(a[off_a + i]) * a[off_a + i];
    bb += double(b[off_b + i]) * b[off_b + i];
  }
  return ab / std::sqrt(aa * bb);
}

}  // namespace

HOST_TEST(construction_and_spec_errors) {
  CHECK_THROWS(ModelBackend("/some/model.pth", true), "load model: failed to open file");
  CHECK_THROWS(ModelBackend("synthetic:13B", true), "unknown synthetic model preset");
  CHECK_THROWS(ModelBackend("synthetic:tiny:w9", true), "bad synthetic model option");
  auto b = tiny();
  CHECK_EQ(b->vocab_size(), 2048);
  CHECK_EQ(b->dims().layers, 2);
  CHECK_EQ(b->model_path(), std::string("synthetic:tiny:w8:seed=3"));
  CHECK(!b->model_name().empty());
}

HOST_TEST(state_shapes_and_forward_errors) {
  auto b = tiny();
  const auto& d = b->dims();
  GenerationState s = b->create_state(3);
  CHECK_EQ(s.batch_size, 3);
  CHECK(s.wkv32);
  CHECK_EQ(s.shift.n, std::size_t(d.layers) * 2 * 3 * d.channels);
  CHECK_EQ(s.wkv_state32.n, std::size_t(d.layers) * 3 * d.heads * 64 * 64);
  CHECK_EQ(s.elapsed.n, std::size_t(3));
  for (float f : host_test::to_host<float>(s.wkv_state32)) CHECK_EQ(f, 0.0f);
  CHECK_THROWS(b->create_state(0), "batch_size must be positive");

  DeviceLogits logits;
  CHECK_THROWS(b->forward_prefill({}, s, logits), "token_batches must not be empty");
  CHECK_THROWS(b->forward_prefill({ramp(4, 1)}, s, logits), "state batch size mismatch");
  CHECK_THROWS(b->forward_prefill({ramp(4, 1), ramp(3, 2), ramp(4, 3)}, s, logits), "share the same length");
  CHECK_THROWS(b->forward_prefill({{}, {}, {}}, s, logits), "length must be positive");
  CHECK_THROWS(b->forward_decode({1, 2}, s, logits), "state batch size mismatch");
  CHECK_THROWS(b->forward_decode({1, 2, 99999}, s, logits), "token id out of range");
  // failed calls leave the state untouched
  CHECK(host_test::to_host<int>(s.elapsed) == (std::vector<int>{0, 0, 0}));

  b->forward_prefill({ramp(5, 1), ramp(5, 2), ramp(5, 3)}, s, logits);
  CHECK_EQ(logits.rows, 3);
  CHECK_EQ(logits.vocab_size, 2048);
  CHECK(host_test::to_host<int>(s.elapsed) == (std::vector<int>{5, 5, 5}));
  b->forward_decode({7, 8, 9}, s, logits);
  CHECK(host_test::to_host<int>(s.elapsed) == (std::vector<int>{6, 6, 6}));
  for (float f : host_test::to_host<float>(logits.values)) CHECK(std::isfinite(f));
}

HOST_TEST(slices_move_whole_sessions_between_batches) {
  auto b = tiny();
  const auto& d = b->dims();
  // three sessions prefilled together ...
  GenerationState s3 = b->create_state(3);
  DeviceLogits l3;
  b->forward_prefill({ramp(6, 1), ramp(6, 2), ramp(6, 3)}, s3, l3);
  // ... session 1 and 2 copied into a width-2 state equal the same two prompts prefilled at width 2
  GenerationState s2 = b->create_state(2);
  b->copy_state_slice(s3, 1, s2, 0, 2);
  GenerationState ref = b->create_state(2);
  DeviceLogits lref;
  b->forward_prefill({ramp(6, 2), ramp(6, 3)}, ref, lref);
  const auto got_wkv = host_test::to_host<float>(s2.wkv_state32), want_wkv = host_test::to_host<float>(ref.wkv_state32);
  CHECK_EQ(got_wkv.size(), want_wkv.size());
  double worst = 0, scale = 0;
  for (std::size_t i = 0; i < got_wkv.size(); ++i) {
    worst = std::max(worst, std::fabs(double(got_wkv[i]) - want_wkv[i]));
    scale = std::max(scale, std::fabs(double(want_wkv[i])));
  }
  CHECK(worst <= 1e-3 * scale);  // batch width changes GEMV summation order by an fp16 ulp at most
  CHECK(host_test::to_host<int>(s2.elapsed) == (std::vector<int>{6, 6}));
  // layout: the slice of layer l, slot j, batch b1 sits at ((l*2+j)*B + b1)*C; check one element each way
  const auto shift3 = host_test::to_host<uint16_t>(s3.shift), shift2 = host_test::to_host<uint16_t>(s2.shift);
  for (int l = 0; l < d.layers; ++l)
    for (int j = 0; j < 2; ++j)
      for (int c : {0, d.channels - 1}) {
        CHECK_EQ(shift2[(std::size_t(l * 2 + j) * 2 + 0) * d.channels + c],
                 shift3[(std::size_t(l * 2 + j) * 3 + 1) * d.channels + c]);
        CHECK_EQ(shift2[(std::size_t(l * 2 + j) * 2 + 1) * d.channels + c],
                 shift3[(std::size_t(l * 2 + j) * 3 + 2) * d.channels + c]);
      }
  // logits rows
  DeviceLogits l2;
  l2.rows = 2;
  l2.vocab_size = 2048;
  l2.values.resize(2 * 2048, "test logits");
  b->copy_logits_slice(l3, 2, l2, 0, 1);
  b->copy_logits_slice(l3, 0, l2, 1, 1);
  const auto h3 = host_test::to_host<float>(l3.values), h2 = host_test::to_host<float>(l2.values);
  for (int v : {0, 1, 2047}) {
    CHECK_EQ(h2[v], h3[2 * 2048 + v]);
    CHECK_EQ(h2[2048 + v], h3[v]);
  }
  CHECK(cosine(h3, host_test::to_host<float>(lref.values), 2048, 0, 2048) > 0.9995);

  CHECK_THROWS(b->copy_state_slice(s3, 2, s2, 0, 2), "exceeds batch size");
  CHECK_THROWS(b->copy_state_slice(s3, 0, s2, 0, 0), "invalid backend state slice range");
  CHECK_THROWS(b->copy_logits_slice(l3, 2, l2, 0, 2), "exceeds row count");
  CHECK_THROWS(b->copy_logits_slice(l3, -1, l2, 0, 1), "invalid backend logits slice range");
}

HOST_TEST(prefill_capacity_is_consistent) {
  auto b = tiny();
  const auto cap = b->query_prefill_capacity(128);
  CHECK(cap.total_vram_bytes >= cap.free_vram_bytes);
  CHECK(cap.free_vram_bytes > 0);
  CHECK(cap.bytes_per_batch > 0);
  CHECK(cap.max_batch_size >= 1);
  const auto cap2 = b->query_prefill_capacity(256);
  CHECK(cap2.bytes_per_batch > cap.bytes_per_batch);
  CHECK_THROWS(b->query_prefill_capacity(0), "prefill chunk size must be positive");
}

// The admission queue over the real backend, bound as the reference's API layer binds it
// (src/rwkv_api_service.cpp:808-811: the provider asks the backend for the capacity at the engine's chunk size).
// A permit sized to the batch brackets a prefill; the hard limit is the start-up capacity.
HOST_TEST(prefill_admission_over_the_backend_capacity) {
  auto b = tiny();
  const int chunk = 128;
  PrefillAdmissionController ctl([b, chunk] { return b->query_prefill_capacity(chunk); });
  const auto start = ctl.snapshot(false);
  CHECK(start.hard_max_batch_size >= 64);  // a tiny model on an empty 288 GB device
  CHECK_EQ(start.hard_max_batch_size, start.dynamic_max_batch_size);
  CHECK_EQ(start.capacity.bytes_per_batch, b->query_prefill_capacity(chunk).bytes_per_batch);
  {
    auto permit = ctl.acquire(8, "/v1/chat/completions");
    CHECK(permit.has_value());
    GenerationState s = b->create_state(8);
    DeviceLogits l;
    std::vector<std::vector<int64_t>> ids;
    for (int i = 0; i < 8; ++i) ids.push_back(ramp(16, 5 + i));
    b->forward_prefill(ids, s, l);
    CHECK_EQ(l.rows, 8);
    CHECK_EQ(ctl.snapshot(true).reserved_batch_size, 8);
  }
  CHECK_EQ(ctl.snapshot(true).reserved_batch_size, 0);
  bool threw = false;
  try {
    (void)ctl.acquire(start.hard_max_batch_size + 1, "too wide");
  } catch (const PrefillBatchLimitExceeded& e) {
    threw = true;
    CHECK_EQ(e.max_batch_size(), start.hard_max_batch_size);
  }
  CHECK(threw);
}

HOST_TEST(engine_end_to_end_on_the_real_backend) {
  auto b = tiny();
  auto tok = std::make_shared<TrieTokenizer>();
  CHECK_EQ(tok->load(host_test::vocab_path()), kTokenizerSuccess);
  GenerateOptions o;
  o.max_tokens = 12;
  o.stop_tokens = {};  // never stop early: token ids of a random model are arbitrary
  o.top_k = 0;
  o.top_p = 0.0;
  o.alpha_presence = 0.0;
  o.alpha_frequency = 0.0;
  const std::string p1 = "User: hi\n\nAssistant:", p2 = "System: test\n\nUser: This is a test\n\nAssistant: the";
  InferenceEngine chunk4(b, tok, "tiny", 4), chunk128(b, tok, "tiny", 128);
  // greedy decoding is a pure function of the prompt: two runs agree exactly
  const auto a = chunk128.batch_generate({p1, p2}, o);
  const auto a_again = chunk128.batch_generate({p1, p2}, o);
  CHECK(a == a_again);
  CHECK_EQ(a.size(), std::size_t(2));
  // chunked prefill (4 tokens a call, widths 2 then 1) carries the state exactly as one long call does, up to
  // fp16 rounding: the logits after the prompt agree
  GenerationState s_small = b->create_state(1), s_big = b->create_state(1);
  DeviceLogits l_small, l_big;
  const int n_small = chunk4.prefill_prompt(p2, s_small, l_small);
  const int n_big = chunk128.prefill_prompt(p2, s_big, l_big);
  CHECK_EQ(n_small, n_big);
  CHECK(host_test::to_host<int>(s_small.elapsed) == std::vector<int>{n_big});
  CHECK(cosine(host_test::to_host<float>(l_small.values), host_test::to_host<float>(l_big.values), 0, 0, 2048) > 0.9995);
  // streaming and non-streaming produce the same bytes when every token is valid UTF-8 on its own; here they
  // need not be, so compare token counts instead
  int emitted = 0;
  const auto stats = chunk128.batch_generate_stream({p1, p2}, o, 1, [&](int, const std::string&) { ++emitted; return true; });
  CHECK_EQ(stats.generated_tokens, 24);
  CHECK_EQ(stats.prompt_tokens, int(tok->encode(p1).size() + tok->encode(p2).size()));
  CHECK(stats.prefill_seconds > 0 && stats.decode_seconds > 0);
}

// The shrinking batch on the real backend: two of four prompts stop at their first token, so the engine gathers the
// other two (not neighbours in the sorted batch) into a batch of two; their greedy texts are those of the run that
// keeps all four rows.
HOST_TEST(shrinking_batch_continues_the_gathered_rows) {
  auto b = tiny();
  auto tok = std::make_shared<TrieTokenizer>();
  CHECK_EQ(tok->load(host_test::vocab_path()), kTokenizerSuccess);
  InferenceEngine engine(b, tok, "tiny", 128);
  const std::string first = "System: the longest prompt of the four, so it is row 0\n\nUser: hi\n\nAssistant:";
  const std::string third = "User: hello there\n\nAssistant: the";
  // greedy token ids of one prompt, decoded alone
  auto greedy_ids = [&](const std::string& prompt, int steps) {
    GenerationState s = b->create_state(1);
    DeviceLogits l;
    engine.prefill_prompt(prompt, s, l);
    std::vector<int> ids;
    for (int i = 0; i < steps; ++i) {
      const auto row = host_test::to_host<float>(l.values);
      ids.push_back(int(std::max_element(row.begin(), row.end()) - row.begin()));
      b->forward_decode({int64_t(ids.back())}, s, l);
    }
    return ids;
  };
  // a prompt whose first greedy token - the stop token of this test - the two long-running rows never produce
  std::vector<int> seen = greedy_ids(first, 24);
  const auto more = greedy_ids(third, 24);
  seen.insert(seen.end(), more.begin(), more.end());
  std::string stopper;
  int stop = -1;
  for (const char* candidate : {"User: a question that ends at once\n\nAssistant:", "User: 12345\n\nAssistant:", "zzz",
                                "User: \xE4\xBD\xA0\xE5\xA5\xBD\n\nAssistant:", "Q", "System: stop here"}) {
    const int t = greedy_ids(candidate, 1).front();
    if (std::find(seen.begin(), seen.end(), t) == seen.end()) {
      stopper = candidate;
      stop = t;
      break;
    }
  }
  CHECK(stop >= 0);
  GenerateOptions o;
  o.max_tokens = 24;
  o.stop_tokens = {stop};
  o.top_k = 0;
  o.top_p = 0.0;
  o.alpha_presence = 0.0;
  o.alpha_frequency = 0.0;
  const std::vector<std::string> prompts{first, stopper, third, stopper};
  const auto keep = engine.batch_generate(prompts, o);
  engine.set_shrink_batch(true);
  const auto shrunk = engine.batch_generate(prompts, o);
  CHECK_EQ(keep.size(), std::size_t(4));
  CHECK(keep[1].empty() && keep[3].empty());
  CHECK(!keep[0].empty() && !keep[2].empty());
  CHECK(shrunk == keep);
  std::vector<std::string> streamed(4);
  const auto stats = engine.batch_generate_stream(prompts, o, 1, [&](int i, const std::string& piece) {
    streamed[std::size_t(i)] += piece;
    return true;
  });
  CHECK(stats.stop_token);
  CHECK(streamed[1].empty() && streamed[3].empty());
}

// The reference's default constructor arguments (use_wkv32 = false): the WKV state lives in fp16 and the recurrence
// runs in fp16.  Same graph, so the logits follow the fp32-state backend's to fp16 accuracy; states of the two
// modes are not interchangeable; slices and the engine work as in the other mode.
HOST_TEST(default_arguments_give_the_fp16_state_mode) {
  ModelBackend b16("synthetic:tiny:w8:seed=3");
  auto b32 = tiny();
  const auto& d = b16.dims();
  GenerationState s16 = b16.create_state(2);
  CHECK(!s16.wkv32);
  CHECK_EQ(s16.wkv_state.n, std::size_t(d.layers) * 2 * d.heads * 64 * 64);
  CHECK_EQ(s16.wkv_state32.n, std::size_t(0));
  for (uint16_t h : host_test::to_host<uint16_t>(s16.wkv_state)) CHECK_EQ(h, uint16_t(0));
  GenerationState s32 = b32->create_state(2);
  DeviceLogits l16, l32;
  CHECK_THROWS(b16.forward_prefill({ramp(4, 1), ramp(4, 2)}, s32, l16), "state wkv precision mismatch");
  CHECK_THROWS(b32->forward_decode({1, 2}, s16, l32), "state wkv precision mismatch");
  // 20 tokens in one call (the w12 + w0 sum is rounded to fp16 first) ...
  b16.forward_prefill({ramp(20, 1), ramp(20, 2)}, s16, l16);
  b32->forward_prefill({ramp(20, 1), ramp(20, 2)}, s32, l32);
  CHECK(host_test::to_host<int>(s16.elapsed) == (std::vector<int>{20, 20}));
  for (int row = 0; row < 2; ++row)
    CHECK(cosine(host_test::to_host<float>(l16.values), host_test::to_host<float>(l32.values), row * 2048, row * 2048, 2048) > 0.999);
  // ... then decode steps (w0 added inside the recurrence)
  for (int step = 0; step < 6; ++step) {
    b16.forward_decode({int64_t(5 + step), int64_t(900 + step)}, s16, l16);
    b32->forward_decode({int64_t(5 + step), int64_t(900 + step)}, s32, l32);
  }
  CHECK(host_test::to_host<int>(s16.elapsed) == (std::vector<int>{26, 26}));
  for (int row = 0; row < 2; ++row)
    CHECK(cosine(host_test::to_host<float>(l16.values), host_test::to_host<float>(l32.values), row * 2048, row * 2048, 2048) > 0.999);
  bool nonzero = false;
  for (uint16_t h : host_test::to_host<uint16_t>(s16.wkv_state)) nonzero = nonzero || (h & 0x7fff) != 0;
  CHECK(nonzero);
  // slices between fp16 states; refused across modes
  GenerationState one = b16.create_state(1);
  b16.copy_state_slice(s16, 1, one, 0, 1);
  const auto all = host_test::to_host<uint16_t>(s16.wkv_state), part = host_test::to_host<uint16_t>(one.wkv_state);
  const std::size_t lane = std::size_t(d.heads) * 64 * 64;
  for (int l = 0; l < d.layers; ++l)
    for (std::size_t i : {std::size_t(0), lane / 2, lane - 1}) CHECK_EQ(part[l * lane + i], all[(std::size_t(l) * 2 + 1) * lane + i]);
  GenerationState one32 = b32->create_state(1);
  CHECK_THROWS(b16.copy_state_slice(s16, 0, one32, 0, 1), "state slice wkv precision mismatch");
  CHECK(b16.query_prefill_capacity(128).bytes_per_batch < b32->query_prefill_capacity(128).bytes_per_batch);
}

// Several host threads call forward_* on one backend, each with its own state (the server's request threads do):
// every thread's logits equal those of the same calls made from one thread, bit for bit.
HOST_TEST(concurrent_forward_calls_on_distinct_states_match_the_serial_run) {
  auto b = tiny();
  constexpr int kThreads = 2, kSteps = 200;
  auto run = [&](int who, std::vector<float>* last_logits, std::vector<float>* wkv) {
    GenerationState s = b->create_state(1);
    DeviceLogits l;
    b->forward_prefill({ramp(9, 10 + who)}, s, l);
    int64_t tok = 3 + who;
    for (int i = 0; i < kSteps; ++i) {
      b->forward_decode({tok}, s, l);
      tok = (tok * 31 + 7 + who) % 2048;
    }
    *last_logits = host_test::to_host<float>(l.values);
    *wkv = host_test::to_host<float>(s.wkv_state32);
  };
  std::vector<float> serial_l[kThreads], serial_s[kThreads], par_l[kThreads], par_s[kThreads];
  for (int t = 0; t < kThreads; ++t) run(t, &serial_l[t], &serial_s[t]);
  std::vector<std::thread> pool;
  std::vector<std::string> errors(kThreads);
  for (int t = 0; t < kThreads; ++t)
    pool.emplace_back([&, t] {
      try {
        run(t, &par_l[t], &par_s[t]);
      } catch (const std::exception& e) {
        errors[t] = e.what();
      }
    });
  for (auto& th : pool) th.join();
  for (int t = 0; t < kThreads; ++t) {
    CHECK(errors[t].empty());
    CHECK_EQ(par_l[t].size(), serial_l[t].size());
    CHECK(std::memcmp(par_l[t].data(), serial_l[t].data(), serial_l[t].size() * sizeof(float)) == 0);
    CHECK(std::memcmp(par_s[t].data(), serial_s[t].data(), serial_s[t].size() * sizeof(float)) == 0);
  }
  CHECK(std::memcmp(serial_l[0].data(), serial_l[1].data(), serial_l[0].size() * sizeof(float)) != 0);  // (the two differ)
}

// One pooled session serves states that alternate (the captured decode graph is keyed by the state's addresses): graph
// replays agree with themselves run after run and follow each state independently.
HOST_TEST(alternating_states_on_one_session_keep_apart) {
  auto b = tiny();
  GenerationState a = b->create_state(1), c = b->create_state(1), a2 = b->create_state(1), c2 = b->create_state(1);
  DeviceLogits la, lc, la2, lc2;
  b->forward_prefill({ramp(5, 1)}, a, la);
  b->forward_prefill({ramp(5, 2)}, c, lc);
  b->forward_prefill({ramp(5, 1)}, a2, la2);
  b->forward_prefill({ramp(5, 2)}, c2, lc2);
  for (int i = 0; i < 12; ++i) {   // interleaved on the shared session pool ...
    b->forward_decode({int64_t(40 + i)}, a, la);
    b->forward_decode({int64_t(80 + i)}, c, lc);
  }
  for (int i = 0; i < 12; ++i) b->forward_decode({int64_t(40 + i)}, a2, la2);   // ... equals one after the other
  for (int i = 0; i < 12; ++i) b->forward_decode({int64_t(80 + i)}, c2, lc2);
  const auto ha = host_test::to_host<float>(la.values), ha2 = host_test::to_host<float>(la2.values);
  const auto hc = host_test::to_host<float>(lc.values), hc2 = host_test::to_host<float>(lc2.values);
  CHECK(std::memcmp(ha.data(), ha2.data(), ha.size() * sizeof(float)) == 0);
  CHECK(std::memcmp(hc.data(), hc2.data(), hc.size() * sizeof(float)) == 0);
}

// Recycled blocks: the state and logits of a request come back at the addresses the last request of that shape had,
// so its decode steps replay the graph captured then (none is captured again); a recycled state is cleared like a
// new one; the blocks held count as free memory and can be given back.
HOST_TEST(consecutive_requests_reuse_buffers_and_the_captured_graph) {
  auto b = tiny();
  std::vector<float> first;
  const void* shift_at = nullptr;
  const void* logits_at = nullptr;
  int64_t after_first = 0;
  for (int request = 0; request < 3; ++request) {
    GenerationState st = b->create_state(3);
    for (uint16_t h : host_test::to_host<uint16_t>(st.shift)) CHECK_EQ(h, uint16_t(0));
    for (float f : host_test::to_host<float>(st.wkv_state32)) CHECK_EQ(f, 0.0f);
    CHECK(host_test::to_host<int>(st.elapsed) == (std::vector<int>{0, 0, 0}));
    DeviceLogits lg;
    b->forward_prefill({ramp(6, 1), ramp(6, 2), ramp(6, 3)}, st, lg);
    int64_t before = 0, after = 0;
    CHECK_EQ(rwkv_hip_graph_capture_count(&before), RWKV_OK);
    for (int i = 0; i < 5; ++i) b->forward_decode({int64_t(10 + i), int64_t(20 + i), int64_t(30 + i)}, st, lg);
    CHECK_EQ(rwkv_hip_graph_capture_count(&after), RWKV_OK);
    const auto host = host_test::to_host<float>(lg.values);
    if (request == 0) {
      first = host;
      shift_at = st.shift.p;
      logits_at = lg.values.p;
      after_first = after;
    } else {
      CHECK(st.shift.p == shift_at && lg.values.p == logits_at);      // the same blocks again
      CHECK_EQ(after, before);                                        // and no new capture
      CHECK_EQ(after, after_first);
      CHECK(std::memcmp(host.data(), first.data(), host.size() * sizeof(float)) == 0);
    }
  }
  // the blocks just given back are held: they count as free, and trimming returns them to the device
  std::size_t free0 = 0, free1 = 0, total = 0;
  CHECK_EQ(rwkv_hip_mem_info(&free0, &total), RWKV_OK);
  CHECK_EQ(rwkv_hip_recycle_trim(), RWKV_OK);
  CHECK_EQ(rwkv_hip_mem_info(&free1, &total), RWKV_OK);
  CHECK(free1 + (std::size_t(64) << 20) >= free0);   // nothing was double counted (other processes aside)
  void* p = nullptr;
  void* q = nullptr;
  CHECK_EQ(rwkv_hip_malloc_recycled(&p, 4096), RWKV_OK);
  CHECK_EQ(rwkv_hip_free_recycled(p, 4096), RWKV_OK);
  CHECK_EQ(rwkv_hip_malloc_recycled(&q, 4096), RWKV_OK);
  CHECK(p == q);
  CHECK_EQ(rwkv_hip_free_recycled(q, 4096), RWKV_OK);
  CHECK_EQ(rwkv_hip_recycle_trim(), RWKV_OK);
}

int main(int argc, char** argv) { return host_test::run_all(argc, argv, true); }
