// Three-level state cache with capacities (1, 1): put/get bit-exact, demotion order device -> host -> database,
// reload from the database, delete (reference: test/state_cache_test.cpp:67-99), for both state precisions,
// plus persistence across shutdown.  Usage: <exe> <repo root> [database path]
#include <cstdio>
#include <cstring>
#include <unistd.h>

#include "rwkv_server_backend.hpp"
#include "rwkv_state_cache.hpp"
#include "test_common.hpp"

using namespace rwkv7_server;

namespace {

std::string g_db_path;

template <typename T>
bool contains(const std::vector<T>& v, const T& x) {
  for (const T& e : v)
    if (e == x) return true;
  return false;
}

GenerationState make_state(bool wkv32, int batch, std::vector<uint16_t> shift, std::vector<float> wkv,
                           std::vector<int> elapsed) {
  GenerationState s;
  s.batch_size = batch;
  s.wkv32 = wkv32;
  host_test::to_device(shift, s.shift);
  if (wkv32) {
    host_test::to_device(wkv, s.wkv_state32);
  } else {
    std::vector<uint16_t> bits;
    for (float f : wkv) bits.push_back(uint16_t(0x3C00 + int(f)));  // any distinct 16-bit patterns do
    host_test::to_device(bits, s.wkv_state);
  }
  host_test::to_device(elapsed, s.elapsed);
  return s;
}

void expect_same(const GenerationState& got, const GenerationState& want) {
  CHECK_EQ(got.batch_size, want.batch_size);
  CHECK_EQ(got.wkv32, want.wkv32);
  CHECK(host_test::to_host<uint16_t>(got.shift) == host_test::to_host<uint16_t>(want.shift));
  CHECK(host_test::to_host<uint16_t>(got.wkv_state) == host_test::to_host<uint16_t>(want.wkv_state));
  // compare fp32 state by bit pattern (NaN payloads and -0 must survive too)
  CHECK(host_test::to_host<uint32_t>(got.wkv_state32) == host_test::to_host<uint32_t>(want.wkv_state32));
  CHECK(host_test::to_host<int>(got.elapsed) == host_test::to_host<int>(want.elapsed));
}

void demotion_scenario(bool wkv32) {
  auto& cache = StateCacheManager::instance();
  std::remove(g_db_path.c_str());
  cache.initialize(1, 1, g_db_path);
  CHECK(cache.database_available());

  const float nan = std::nanf("7"), neg0 = -0.0f;
  auto s1 = make_state(wkv32, 1, {0x3C00, 0x4000}, {3.0f, neg0, wkv32 ? nan : 5.0f}, {7});
  auto s2 = make_state(wkv32, 1, {0x4600}, {7.0f, 8.0f}, {9});
  auto s3 = make_state(wkv32, 2, {0x4900, 0x4980}, {12.0f}, {13, 14});

  cache.put_state("", s1);  // an empty id is ignored
  CHECK(!cache.get_state("").has_value());
  CHECK(!cache.get_state("missing").has_value());

  cache.put_state("session-1", s1);
  auto got = cache.get_state("session-1");
  CHECK(got.has_value());
  expect_same(*got, s1);
  // the cache holds its own copy: changing the caller's state afterwards does not reach it
  rwkv7_fast_v4::check_hip(rwkv_hip_memset(s1.shift.p, 0xFF, s1.shift.n * 2), "scribble");
  auto s1_original = make_state(wkv32, 1, {0x3C00, 0x4000}, {3.0f, neg0, wkv32 ? nan : 5.0f}, {7});
  expect_same(*cache.get_state("session-1"), s1_original);

  cache.put_state("session-2", s2);
  auto summary = cache.list_all_states();
  CHECK(contains(summary.l1_cache, std::string("session-2")));
  CHECK(contains(summary.l2_cache, std::string("session-1")));
  CHECK(summary.database.empty());

  cache.put_state("session-3", s3);
  summary = cache.list_all_states();
  CHECK(contains(summary.l1_cache, std::string("session-3")));
  CHECK(contains(summary.l2_cache, std::string("session-2")));
  CHECK(contains(summary.database, std::string("session-1")));
  CHECK_EQ(summary.l1_cache.size(), std::size_t(1));
  CHECK_EQ(summary.l2_cache.size(), std::size_t(1));

  // reload from the database: bit-exact, and the entry is now the device-level one (3 -> host, 2 -> database)
  auto from_db = cache.get_state("session-1");
  CHECK(from_db.has_value());
  expect_same(*from_db, s1_original);
  CHECK(cache.get_db_timestamp("session-1").has_value());
  CHECK(!cache.get_db_timestamp("never-stored").has_value());
  summary = cache.list_all_states();
  CHECK(contains(summary.l1_cache, std::string("session-1")));
  CHECK(contains(summary.l2_cache, std::string("session-3")));
  CHECK(contains(summary.database, std::string("session-2")));

  // a host-level hit moves the entry back to the device level
  auto from_host = cache.get_state("session-3");
  CHECK(from_host.has_value());
  expect_same(*from_host, s3);
  summary = cache.list_all_states();
  CHECK(contains(summary.l1_cache, std::string("session-3")));
  CHECK(contains(summary.l2_cache, std::string("session-1")));

  CHECK(cache.delete_state_from_any_level("session-2"));   // database only
  CHECK(!cache.get_state("session-2").has_value());
  CHECK(!cache.delete_state_from_any_level("session-2"));
  CHECK(cache.delete_state_from_any_level("session-3"));   // device level
  CHECK(!cache.get_state("session-3").has_value());

  // shutdown writes what is still cached to the database; a new instance lifetime reads it back
  cache.shutdown();
  CHECK(!cache.get_state("session-1").has_value());  // not initialised: nothing is served
  cache.initialize(4, 4, g_db_path);
  auto revived = cache.get_state("session-1");
  CHECK(revived.has_value());
  expect_same(*revived, s1_original);
  cache.shutdown();
  std::remove(g_db_path.c_str());
}

}  // namespace

HOST_TEST(demotion_reload_delete_fp32_state) { demotion_scenario(true); }
HOST_TEST(demotion_reload_delete_fp16_state) { demotion_scenario(false); }

HOST_TEST(overwriting_a_session_replaces_it_at_every_level) {
  auto& cache = StateCacheManager::instance();
  std::remove(g_db_path.c_str());
  cache.initialize(1, 1, g_db_path);
  auto a = make_state(true, 1, {1}, {1.0f}, {1});
  auto b = make_state(true, 1, {2}, {2.0f}, {2});
  auto a2 = make_state(true, 1, {3}, {3.0f}, {3});
  cache.put_state("a", a);
  cache.put_state("b", b);     // a -> host level
  cache.put_state("a", a2);    // a leaves the host level and re-enters at the device level; b -> host
  auto summary = cache.list_all_states();
  CHECK_EQ(summary.l1_cache, std::vector<std::string>{"a"});
  CHECK_EQ(summary.l2_cache, std::vector<std::string>{"b"});
  expect_same(*cache.get_state("a"), a2);
  cache.shutdown();
  std::remove(g_db_path.c_str());
}

// A real generation state of each precision (the fp16-state backend is the reference's default) goes through the
// device, host and database levels and resumes bit for bit: the restored copy continues exactly like the original.
HOST_TEST(real_backend_states_resume_bitwise_from_every_level) {
  for (bool wkv32 : {false, true}) {
    ModelBackend backend("synthetic:tiny:w8:seed=5", wkv32);
    auto& cache = StateCacheManager::instance();
    std::remove(g_db_path.c_str());
    cache.initialize(1, 1, g_db_path);
    GenerationState live = backend.create_state(1);
    DeviceLogits logits;
    backend.forward_prefill({{5, 6, 7, 8, 9, 10, 11}}, live, logits);
    cache.put_state("live", live);
    // push it down: one more session -> host level, another -> database
    auto filler1 = make_state(wkv32, 1, {1}, {1.0f}, {1});
    auto filler2 = make_state(wkv32, 1, {2}, {2.0f}, {2});
    auto filler3 = make_state(wkv32, 1, {3}, {3.0f}, {3});
    std::vector<std::vector<float>> want;
    for (int step = 0; step < 3; ++step) {
      backend.forward_decode({int64_t(100 + step)}, live, logits);
      want.push_back(host_test::to_host<float>(logits.values));
    }
    for (int level = 0; level < 3; ++level) {
      if (level == 1) cache.put_state("filler-1", filler1);
      if (level == 2) {   // (the host-level hit above brought it back to the device level: two more sessions push it out)
        cache.put_state("filler-2", filler2);
        cache.put_state("filler-3", filler3);
      }
      const auto summary = cache.list_all_states();
      if (level == 1) CHECK(contains(summary.l2_cache, std::string("live")));
      if (level == 2) CHECK(contains(summary.database, std::string("live")));
      auto restored = cache.get_state("live");
      CHECK(restored.has_value());
      CHECK_EQ(restored->wkv32, wkv32);
      CHECK(host_test::to_host<int>(restored->elapsed) == std::vector<int>{7});
      DeviceLogits again;
      for (int step = 0; step < 3; ++step) {
        backend.forward_decode({int64_t(100 + step)}, *restored, again);
        const auto got = host_test::to_host<float>(again.values);
        CHECK(std::memcmp(got.data(), want[step].data(), got.size() * sizeof(float)) == 0);
      }
      if (level == 0) {
        // get_state handed out a copy: the cached entry is still the state after the prompt
        CHECK(host_test::to_host<int>(cache.get_state("live")->elapsed) == std::vector<int>{7});
      }
    }
    cache.shutdown();
    std::remove(g_db_path.c_str());
  }
}

int main(int argc, char** argv) {
  g_db_path = argc > 2 ? argv[2] : "/tmp/rwkv_state_cache_test_" + std::to_string(getpid()) + ".db";
  return host_test::run_all(argc, argv, true);
}
