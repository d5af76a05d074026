// Sampler known answers through the host API (reference: test/sampler_test.cpp:30-83) and seeded reproducibility.
#include "rwkv_sampler.hpp"
#include "test_common.hpp"

using namespace rwkv7_server;

namespace {
DeviceLogits make_logits(const std::vector<float>& host, int rows = 1) {
  DeviceLogits l;
  l.rows = rows;
  l.vocab_size = int(host.size()) / rows;
  host_test::to_device(host, l.values);
  return l;
}
GenerateOptions argmax_options() {
  GenerateOptions o;
  o.top_k = 0;
  o.top_p = 0.0;
  o.temperature = 1.0;
  return o;
}
}  // namespace

HOST_TEST(top_p_zero_is_argmax) {
  auto state = make_sampler_penalties(4);
  auto logits = make_logits({0.25f, 3.0f, 1.0f, -1.0f});
  CHECK_EQ(sample_repetition_temperature_topk_topp(logits, state, argmax_options()), 1);
}

HOST_TEST(zero_alphas_leave_penalties_at_zero) {
  auto state = make_sampler_penalties(4);
  auto logits = make_logits({0.25f, 3.0f, 1.0f, -1.0f});
  GenerateOptions o = argmax_options();
  o.alpha_presence = 0.0;
  o.alpha_frequency = 0.0;
  CHECK_EQ(sample_repetition_temperature_topk_topp(logits, state, o), 1);
  for (float p : host_test::to_host<float>(state.penalties)) CHECK_NEAR(p, 0.0, 1e-6);
}

HOST_TEST(penalty_recurrence_gives_2_then_6) {
  auto state = make_sampler_penalties(4);
  auto logits = make_logits({100.0f, 0.0f, 0.0f, 0.0f});
  GenerateOptions o = argmax_options();
  o.alpha_presence = 2.0;
  o.alpha_frequency = 5.0;
  o.alpha_decay = 0.5;
  CHECK_EQ(sample_repetition_temperature_topk_topp(logits, state, o), 0);
  auto p = host_test::to_host<float>(state.penalties);
  CHECK_NEAR(p.at(0), 2.0, 1e-4);
  CHECK_NEAR(p.at(1), 0.0, 1e-6);
  CHECK_EQ(sample_repetition_temperature_topk_topp(logits, state, o), 0);
  p = host_test::to_host<float>(state.penalties);
  CHECK_NEAR(p.at(0), 6.0, 1e-4);
}

HOST_TEST(penalties_change_the_choice) {
  // 5.0 vs 4.0: after token 0 is taken once with presence 2, token 1 (4.0) beats 5.0 - 2.0
  auto state = make_sampler_penalties(4);
  auto logits = make_logits({5.0f, 4.0f, 0.0f, 0.0f});
  GenerateOptions o = argmax_options();
  o.alpha_presence = 2.0;
  o.alpha_frequency = 0.5;
  o.alpha_decay = 1.0;
  CHECK_EQ(sample_repetition_temperature_topk_topp(logits, state, o), 0);
  CHECK_EQ(sample_repetition_temperature_topk_topp(logits, state, o), 1);
}

HOST_TEST(argument_errors) {
  auto state = make_sampler_penalties(4);
  auto logits = make_logits({1.0f, 2.0f, 3.0f, 4.0f});
  logits.rows = 2;
  CHECK_THROWS(sample_repetition_temperature_topk_topp(logits, state, GenerateOptions{}), "single logits row");
  CHECK_THROWS(sample_batch_repetition_temperature_topk_topp(logits, state, GenerateOptions{}),
               "batch size does not match");
  logits.rows = 1;
  auto wide = make_sampler_penalties(8);
  CHECK_THROWS(sample_repetition_temperature_topk_topp(logits, wide, GenerateOptions{}), "does not match sampler state");
  DeviceLogits empty;
  empty.rows = 1;
  CHECK_THROWS(sample_repetition_temperature_topk_topp(empty, state, GenerateOptions{}), "empty device logits");
  auto odd = make_sampler_penalties(6);
  auto odd_logits = make_logits({1.0f, 2.0f, 3.0f, 4.0f, 5.0f, 6.0f});
  CHECK_THROWS(sample_repetition_temperature_topk_topp(odd_logits, odd, GenerateOptions{}), "multiple of 4");
  GenerateOptions cold;
  cold.temperature = 0.0;
  CHECK_THROWS(sample_repetition_temperature_topk_topp(logits, state, cold), "Temperature outside range");
  CHECK_THROWS(make_sampler_penalties(0), "invalid sampler vocab size");
  CHECK_THROWS(make_sampler_penalties(4, 0), "invalid sampler batch size");
}

HOST_TEST(batch_rows_are_independent_and_seeded_streams_repeat) {
  const int V = 1000, B = 3;
  std::vector<float> host(std::size_t(B) * V);
  for (int b = 0; b < B; ++b)
    for (int v = 0; v < V; ++v) host[std::size_t(b) * V + v] = std::sin(0.37f * v + 1.3f * b) * 2.0f;
  auto logits = make_logits(host, B);
  GenerateOptions o;  // defaults: temperature 1, top_k 20, top_p 0.3, penalties on
  o.top_p = 0.9;
  auto run = [&](std::uint64_t seed) {
    auto state = make_sampler_penalties(V, B, seed);
    std::vector<std::vector<int>> draws;
    for (int i = 0; i < 16; ++i) draws.push_back(sample_batch_repetition_temperature_topk_topp(logits, state, o));
    return draws;
  };
  const auto a = run(1234), b = run(1234), c = run(99);
  CHECK(a == b);
  CHECK(a != c);
  for (const auto& step : a) {
    CHECK_EQ(step.size(), std::size_t(B));
    for (int t : step) CHECK(t >= 0 && t < V);
  }
}

int main(int argc, char** argv) { return host_test::run_all(argc, argv, true); }
