// Minimal harness for the host-API test executables: named cases, CHECK macros that throw, one line per case.
// Usage: <exe> <repo root>.  Exit status 0 only when every case passed.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <functional>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "rwkv_server_backend.hpp"

namespace host_test {

struct Failure : std::runtime_error {
  using std::runtime_error::runtime_error;
};

inline std::string& repo_root() {
  static std::string root = ".";
  return root;
}
inline std::string vocab_path() { return repo_root() + "/tests/golden/synthetic_vocab.txt"; }

struct Case {
  const char* name;
  std::function<void()> body;
};
inline std::vector<Case>& cases() {
  static std::vector<Case> all;
  return all;
}
struct Register {
  Register(const char* name, std::function<void()> body) { cases().push_back({name, std::move(body)}); }
};

#define HOST_TEST(name)                                            \
  static void name();                                              \
  static ::host_test::Register register_##name(#name, name);       \
  static void name()

#define FAIL_HERE(msg)                                                              \
  do {                                                                              \
    std::ostringstream os_;                                                         \
    os_ << __FILE__ << ":" << __LINE__ << ": " << msg;                              \
    throw ::host_test::Failure(os_.str());                                          \
  } while (0)

#define CHECK(cond)                                  \
  do {                                               \
    if (!(cond)) FAIL_HERE("CHECK(" #cond ")");      \
  } while (0)

#define CHECK_EQ(a, b)                                                      \
  do {                                                                      \
    if (!((a) == (b))) FAIL_HERE("CHECK_EQ(" #a ", " #b ")");               \
  } while (0)

#define CHECK_NEAR(a, b, tol)                                                                  \
  do {                                                                                         \
    if (!(std::fabs(double(a) - double(b)) <= (tol)))                                          \
      FAIL_HERE("CHECK_NEAR(" #a ", " #b "): " << double(a) << " vs " << double(b));           \
  } while (0)

// the expression must throw a std::exception whose what() contains `text`
#define CHECK_THROWS(expr, text)                                                         \
  do {                                                                                   \
    bool threw_ = false;                                                                 \
    try {                                                                                \
      (void)(expr);                                                                      \
    } catch (const ::host_test::Failure&) {                                              \
      throw;                                                                             \
    } catch (const std::exception& e_) {                                                 \
      threw_ = true;                                                                     \
      if (std::string(e_.what()).find(text) == std::string::npos)                        \
        FAIL_HERE("wrong message for " #expr ": " << e_.what());                         \
    }                                                                                    \
    if (!threw_) FAIL_HERE("no exception from " #expr);                                  \
  } while (0)

inline int run_all(int argc, char** argv, bool needs_gpu) {
  if (argc > 1) repo_root() = argv[1];
  if (needs_gpu) {
    int n = 0;
    if (rwkv_hip_device_count(&n) != RWKV_OK || n <= 0) {
      std::printf("no GPU visible: this executable needs one\n");
      return 2;
    }
  }
  int failed = 0;
  for (const Case& c : cases()) {
    try {
      c.body();
      std::printf("ok   %s\n", c.name);
    } catch (const std::exception& e) {
      ++failed;
      std::printf("FAIL %s: %s\n", c.name, e.what());
    }
    std::fflush(stdout);
  }
  std::printf("%zu cases, %d failed\n", cases().size(), failed);
  return failed ? 1 : 0;
}

// ---- device helpers ---------------------------------------------------------------------------------------------

template <typename T, typename H>
void to_device(const std::vector<H>& host, rwkv7_fast_v4::DeviceBuffer<T>& buf) {
  static_assert(sizeof(T) == sizeof(H), "element sizes must match");
  buf.resize(host.size(), "test alloc");
  if (!host.empty())
    rwkv7_fast_v4::check_hip(rwkv_hip_memcpy_h2d(buf.p, host.data(), host.size() * sizeof(T)), "test h2d");
}

template <typename H, typename T>
std::vector<H> to_host(const rwkv7_fast_v4::DeviceBuffer<T>& buf) {
  static_assert(sizeof(T) == sizeof(H), "element sizes must match");
  std::vector<H> host(buf.n);
  if (buf.n) rwkv7_fast_v4::check_hip(rwkv_hip_memcpy_d2h(host.data(), buf.p, buf.n * sizeof(T)), "test d2h");
  return host;
}

inline std::vector<float> one_hot(int vocab, int hot_token, float hot = 100.0f, float cold = -100.0f) {
  std::vector<float> v(static_cast<std::size_t>(vocab), cold);
  if (hot_token >= 0 && hot_token < vocab) v[hot_token] = hot;
  return v;
}

}  // namespace host_test
