// ModelBackend over the kernel library (synthetic tiny model): state and logits shapes, argument errors with
// the reference's messages (src/rwkv_server_backend.cpp:1399-1580), slice copies, and the engine end to end.
#include "rwkv_inference_engine.hpp"
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
  CHECK_THROWS(ModelBackend("synthetic:tiny", false), "fp32 WKV state only");
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

int main(int argc, char** argv) { return host_test::run_all(argc, argv, true); }
