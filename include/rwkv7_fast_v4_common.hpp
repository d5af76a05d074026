// CUDA-free rendition of the reference's common types that the host API exposes
// (include/rwkv7_fast_v4_common.hpp:21-27,64-110 in the reference): the owning device buffer and the
// handful of constants.  Device memory goes through the C ABI of librwkv_hip.so.
#pragma once

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

#include "rwkv_hip.h"

// fp16 storage type of the host API: a 16-bit POD (the reference uses cuda_fp16.h's `half` here).
using half = std::uint16_t;

namespace rwkv7_fast_v4 {

constexpr int kLowrankMax = 512;
constexpr float kLnEps = 1e-5f;

// Device errors surface as exceptions (the reference prints and calls std::exit, :57-62).
inline void check_hip(int rc, const char* what) {
  if (rc != RWKV_OK) throw std::runtime_error(std::string(what) + " failed: " + rwkv_hip_last_error());
}

// Move-only owner of `n` elements of device memory.  resize() only grows and does not keep the old
// contents; zero() clears the whole allocation.
template <typename T>
struct DeviceBuffer {
  T* p = nullptr;
  std::size_t n = 0;

  DeviceBuffer() = default;
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  DeviceBuffer(DeviceBuffer&& o) noexcept : p(o.p), n(o.n), recycled(o.recycled) { o.p = nullptr; o.n = 0; o.recycled = false; }
  DeviceBuffer& operator=(DeviceBuffer&& o) noexcept {
    if (this != &o) {
      release();
      p = o.p; n = o.n; recycled = o.recycled;
      o.p = nullptr; o.n = 0; o.recycled = false;
    }
    return *this;
  }
  ~DeviceBuffer() { release(); }

  void resize(std::size_t count, const char* what) {
    if (count <= n) return;
    release();
    void* q = nullptr;
    check_hip(rwkv_hip_malloc(&q, count * sizeof(T)), what);
    p = static_cast<T*>(q);
    n = count;
  }

  // The same from the recycled blocks (rwkv_hip_malloc_recycled): freed buffers of this size come back at their old
  // addresses.  For buffers that a serving loop allocates per request (generation state, logits).
  void resize_recycled(std::size_t count, const char* what) {
    if (count <= n) return;
    release();
    void* q = nullptr;
    check_hip(rwkv_hip_malloc_recycled(&q, count * sizeof(T)), what);
    p = static_cast<T*>(q);
    n = count;
    recycled = true;
  }

  void zero(const char* what) {
    if (p && n) check_hip(rwkv_hip_memset(p, 0, n * sizeof(T)), what);
  }

 private:
  void release() {
    if (p) {
      if (recycled) rwkv_hip_free_recycled(p, n * sizeof(T));
      else rwkv_hip_free(p);
    }
    p = nullptr;
    n = 0;
    recycled = false;
  }
  bool recycled = false;
};

struct ModelDims {
  int layers = 0, channels = 0, heads = 0, head_size = 64, vocab = 0, ffn = 0;
  int rank_w = 0, rank_a = 0, rank_g = 0, rank_v = 0;  // LoRA ranks (read from tensor shapes in the reference)
};

}  // namespace rwkv7_fast_v4
