// ModelBackend built from a checkpoint file (the load pipeline of src/rwkv7_fast_v4.cu:110-701 in the reference):
// dimensions read from tensor shapes, whole-file and on-demand reading give the same model bit for bit, weight
// formats chosen by a suffix of the path, load errors.  Usage: <exe> <repo root> [<file.pth> [<logits out>]];
// default file: tests/golden/rwkv7_tiny.pth.  With <logits out> the fp32 logits of the fixed prompt below are
// written there (prefill of all tokens, then two decode steps: three rows of V floats) for a comparison against
// another route to the same weights.
#include <unistd.h>

#include <fstream>

#include "test_common.hpp"

using namespace rwkv7_server;

namespace {

std::string g_pth, g_out;

std::string checkpoint() { return g_pth.empty() ? host_test::repo_root() + "/tests/golden/rwkv7_tiny.pth" : g_pth; }

std::vector<int64_t> prompt(int vocab) {
  std::vector<int64_t> t;
  for (int i = 0; i < 11; ++i) t.push_back((3 + 7 * i) % vocab);
  return t;
}

// prefill + two decode steps; returns the three logit rows
std::vector<float> run(const ModelBackend& b) {
  const int V = b.vocab_size();
  GenerationState s = b.create_state(1);
  DeviceLogits logits;
  std::vector<float> rows;
  b.forward_prefill({prompt(V)}, s, logits);
  auto take = [&] {
    const std::vector<float> h = host_test::to_host<float>(logits.values);
    CHECK_EQ(h.size(), std::size_t(V));
    rows.insert(rows.end(), h.begin(), h.end());
  };
  take();
  b.forward_decode({5 % V}, s, logits);
  take();
  b.forward_decode({17 % V}, s, logits);
  take();
  for (float f : rows) CHECK(std::isfinite(f));
  return rows;
}

double cosine(const std::vector<float>& a, const std::vector<float>& b) {
  double ab = 0, aa = 0, bb = 0;
  for (std::size_t i = 0; i < a.size(); ++i) {
    ab += double(a[i]) * b[i];
    aa += double(a[i]) * a[i];
    bb += double(b[i]) * b[i];
  }
  return ab / std::sqrt(aa * bb);
}

}  // namespace

HOST_TEST(checkpoint_whole_and_on_demand_give_the_same_model) {
  ModelBackend whole(checkpoint(), true, false);
  ModelBackend lazy(checkpoint(), true, true);
  CHECK(whole.vocab_size() > 0);
  CHECK_EQ(whole.vocab_size(), lazy.vocab_size());
  CHECK_EQ(whole.dims().channels, whole.dims().heads * 64);
  CHECK(whole.dims().rank_w > 0 && whole.dims().rank_a > 0 && whole.dims().rank_g > 0 && whole.dims().rank_v > 0);
  if (g_pth.empty()) {  // the committed fixture
    CHECK_EQ(whole.dims().layers, 2);
    CHECK_EQ(whole.dims().channels, 64);
    CHECK_EQ(whole.dims().ffn, 128);
    CHECK_EQ(whole.vocab_size(), 32);
    CHECK_EQ(whole.dims().rank_g, 16);
    CHECK_EQ(whole.model_name(), std::string("rwkv7_tiny"));
  }
  CHECK_EQ(whole.model_path(), checkpoint());
  const std::vector<float> a = run(whole);
  const std::vector<float> b = run(lazy);
  CHECK(std::memcmp(a.data(), b.data(), a.size() * sizeof(float)) == 0);
  double spread = 0;
  for (float f : a) spread = std::max(spread, std::fabs(double(f)));
  CHECK(spread > 0);
  if (!g_out.empty()) {
    std::ofstream f(g_out, std::ios::binary);
    f.write(reinterpret_cast<const char*>(a.data()), static_cast<std::streamsize>(a.size() * sizeof(float)));
    CHECK(static_cast<bool>(f));
  }
}

HOST_TEST(weight_format_suffix_quantises_on_load) {
  ModelBackend f16(checkpoint() + ":f16", true);
  ModelBackend w8(checkpoint() + ":w8", true);
  CHECK_EQ(w8.model_path(), checkpoint() + ":w8");
  CHECK_EQ(w8.model_name(), f16.model_name());
  const std::vector<float> a = run(f16);
  const std::vector<float> b = run(w8);
  CHECK(cosine(a, b) > 0.995);  // int8 per-row quantisation of N(0, 0.02) matrices
  CHECK(std::memcmp(a.data(), b.data(), a.size() * sizeof(float)) != 0);
}

HOST_TEST(load_errors) {
  CHECK_THROWS(ModelBackend("/definitely/missing.pth", true), "load model: failed to open file");
  {
    ModelBackend fp16_state(checkpoint());   // the reference's default arguments: fp16 WKV state
    GenerationState st = fp16_state.create_state(1);
    CHECK(!st.wkv32);
    DeviceLogits lg;
    fp16_state.forward_prefill({{1, 2, 3, 4, 5}}, st, lg);
    for (float f : host_test::to_host<float>(lg.values)) CHECK(std::isfinite(f));
  }
  const std::string junk = "/tmp/rwkv_pth_backend_junk_" + std::to_string(::getpid()) + ".pth";
  {
    std::ofstream f(junk, std::ios::binary);
    f << std::string(300, 'x');
  }
  CHECK_THROWS(ModelBackend(junk, true), "end of central directory not found");
  std::remove(junk.c_str());
}

int main(int argc, char** argv) {
  if (argc > 2) g_pth = argv[2];
  if (argc > 3) g_out = argv[3];
  return host_test::run_all(argc, argv, true);
}
