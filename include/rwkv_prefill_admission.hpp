// Prefill admission: a first-come-first-served queue that lets a request start its prefill only while the batch
// lanes it needs fit into the device memory the backend reports free.  Same class, method and member names as the
// reference's include/rwkv_prefill_admission.hpp (used by its API layer, src/rwkv_api_service.cpp:808-811,1118),
// so that code written against it compiles unchanged.
#pragma once

#include <condition_variable>
#include <cstdint>
#include <deque>
#include <functional>
#include <mutex>
#include <optional>
#include <stdexcept>
#include <string>

#include "rwkv_server_backend.hpp"

namespace rwkv7_server {

// A request wider than the limit fixed at start-up can never be admitted.
class PrefillBatchLimitExceeded : public std::runtime_error {
 public:
  PrefillBatchLimitExceeded(int request_batch_size, int max_batch_size);
  int request_batch_size() const { return request_batch_size_; }
  int max_batch_size() const { return max_batch_size_; }

 private:
  int request_batch_size_ = 0;
  int max_batch_size_ = 0;
};

class PrefillAdmissionController {
 public:
  using CapacityProvider = std::function<PrefillCapacity()>;  // e.g. backend->query_prefill_capacity(chunk)
  using CancelCallback = std::function<bool()>;

  struct Snapshot {
    int hard_max_batch_size = 0;     // the capacity seen at construction: the widest request ever accepted
    int dynamic_max_batch_size = 0;  // the capacity at the last refresh, never above the hard limit
    int reserved_batch_size = 0;     // lanes held by live permits
    std::size_t queued_requests = 0;
    PrefillCapacity capacity;
  };

  // Lanes reserved for one request; gives them back when released or destroyed.  Move-only.
  class Permit {
   public:
    Permit() = default;
    Permit(const Permit&) = delete;
    Permit& operator=(const Permit&) = delete;
    Permit(Permit&& other) noexcept;
    Permit& operator=(Permit&& other) noexcept;
    ~Permit();

    explicit operator bool() const { return controller_ != nullptr; }
    int batch_size() const { return batch_size_; }
    std::uint64_t ticket() const { return ticket_; }
    void release();

   private:
    friend class PrefillAdmissionController;
    Permit(PrefillAdmissionController* controller, int batch_size, std::uint64_t ticket);

    PrefillAdmissionController* controller_ = nullptr;
    int batch_size_ = 0;
    std::uint64_t ticket_ = 0;
  };

  explicit PrefillAdmissionController(CapacityProvider capacity_provider);

  // Blocks until the request is at the head of the queue and its lanes fit, then returns the permit; returns
  // nothing if should_cancel() turns true while waiting (polled every 100 ms); throws PrefillBatchLimitExceeded
  // at once for a request wider than the hard limit.  request_batch_size below 1 counts as 1.
  std::optional<Permit> acquire(int request_batch_size, std::string request_label, const CancelCallback& should_cancel = {});
  Snapshot snapshot(bool refresh_capacity = true);

 private:
  struct QueueEntry {
    std::uint64_t ticket = 0;
    int batch_size = 0;
    std::string label;
  };

  void release(int batch_size, std::uint64_t ticket);
  void refresh_capacity_locked();
  void remove_ticket_locked(std::uint64_t ticket);

  CapacityProvider capacity_provider_;
  mutable std::mutex mutex_;
  std::condition_variable condition_;
  std::deque<QueueEntry> queue_;
  PrefillCapacity capacity_;
  int hard_max_batch_size_ = 0;
  bool hard_limit_initialized_ = false;
  int dynamic_max_batch_size_ = 0;
  int reserved_batch_size_ = 0;
  std::uint64_t next_ticket_ = 0;
};

}  // namespace rwkv7_server
