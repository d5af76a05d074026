// Prefill admission queue (interface: include/rwkv_prefill_admission.hpp).  Behaviour follows the reference's
// src/rwkv_prefill_admission.cpp:53-176: the capacity seen at construction is the hard limit, the capacity is asked
// again whenever the head of the queue is considered and whenever lanes come back, admission is strictly in ticket
// order (a narrow request never overtakes a wide one that is waiting for room), a waiter polls its cancel callback
// every 100 ms.  Log lines go to stdout with the reference's "[PrefillQueue]" prefix.
#include "rwkv_prefill_admission.hpp"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <utility>

namespace rwkv7_server {

PrefillBatchLimitExceeded::PrefillBatchLimitExceeded(int request_batch_size, int max_batch_size)
    : std::runtime_error("bsz overflow, Max bsz=" + std::to_string(max_batch_size)),  // the text the API returns
      request_batch_size_(request_batch_size),
      max_batch_size_(max_batch_size) {}

// ---- Permit ----------------------------------------------------------------------------------------------------------
PrefillAdmissionController::Permit::Permit(PrefillAdmissionController* controller, int batch_size, std::uint64_t ticket)
    : controller_(controller), batch_size_(batch_size), ticket_(ticket) {}

PrefillAdmissionController::Permit::Permit(Permit&& other) noexcept
    : controller_(std::exchange(other.controller_, nullptr)), batch_size_(other.batch_size_), ticket_(other.ticket_) {}

PrefillAdmissionController::Permit& PrefillAdmissionController::Permit::operator=(Permit&& other) noexcept {
  if (this == &other) return *this;
  release();
  controller_ = std::exchange(other.controller_, nullptr);
  batch_size_ = other.batch_size_;
  ticket_ = other.ticket_;
  return *this;
}

PrefillAdmissionController::Permit::~Permit() { release(); }

void PrefillAdmissionController::Permit::release() {
  if (PrefillAdmissionController* owner = std::exchange(controller_, nullptr)) owner->release(batch_size_, ticket_);
}

// ---- controller ------------------------------------------------------------------------------------------------------
PrefillAdmissionController::PrefillAdmissionController(CapacityProvider capacity_provider)
    : capacity_provider_(std::move(capacity_provider)) {
  if (!capacity_provider_) throw std::runtime_error("prefill capacity provider must not be empty");
  std::lock_guard<std::mutex> lock(mutex_);
  refresh_capacity_locked();
  hard_max_batch_size_ = dynamic_max_batch_size_;
  hard_limit_initialized_ = true;
  std::printf("[PrefillQueue] initialized max_prefill_bsz=%d bytes_per_bsz=%zu free_vram=%zu\n", hard_max_batch_size_,
              capacity_.bytes_per_batch, capacity_.free_vram_bytes);
}

void PrefillAdmissionController::refresh_capacity_locked() {
  capacity_ = capacity_provider_();
  dynamic_max_batch_size_ = std::max(capacity_.max_batch_size, 0);
  if (hard_limit_initialized_ && dynamic_max_batch_size_ > hard_max_batch_size_) dynamic_max_batch_size_ = hard_max_batch_size_;
}

void PrefillAdmissionController::remove_ticket_locked(std::uint64_t ticket) {
  for (auto it = queue_.begin(); it != queue_.end(); ++it) {
    if (it->ticket == ticket) {
      queue_.erase(it);
      return;
    }
  }
}

std::optional<PrefillAdmissionController::Permit> PrefillAdmissionController::acquire(int request_batch_size,
                                                                                      std::string request_label,
                                                                                      const CancelCallback& should_cancel) {
  const int lanes = request_batch_size < 1 ? 1 : request_batch_size;
  std::unique_lock<std::mutex> lock(mutex_);
  if (lanes > hard_max_batch_size_) throw PrefillBatchLimitExceeded(lanes, hard_max_batch_size_);

  const std::uint64_t ticket = next_ticket_++;
  queue_.push_back(QueueEntry{ticket, lanes, request_label});
  // whatever way the wait ends without a permit (cancelled, or the callbacks threw), the ticket leaves the queue and
  // the next one in line is woken
  struct Withdraw {
    PrefillAdmissionController* self;
    std::uint64_t ticket;
    bool armed = true;
    ~Withdraw() {
      if (!armed) return;
      self->remove_ticket_locked(ticket);
      self->condition_.notify_all();
    }
  } withdraw{this, ticket};

  bool announced = false;
  for (;;) {
    if (should_cancel && should_cancel()) return std::nullopt;
    if (!queue_.empty() && queue_.front().ticket == ticket) {
      refresh_capacity_locked();
      const int available = std::max(dynamic_max_batch_size_ - reserved_batch_size_, 0);
      if (lanes <= available) {
        reserved_batch_size_ += lanes;
        queue_.pop_front();
        withdraw.armed = false;
        condition_.notify_all();
        std::printf("[PrefillQueue] admitted ticket=%llu path=%s request_bsz=%d reserved_bsz=%d max_prefill_bsz=%d\n",
                    static_cast<unsigned long long>(ticket), request_label.c_str(), lanes, reserved_batch_size_,
                    dynamic_max_batch_size_);
        return Permit(this, lanes, ticket);
      }
    }
    if (!announced) {
      announced = true;
      std::printf("[PrefillQueue] queued ticket=%llu path=%s request_bsz=%d requests_ahead=%zu reserved_bsz=%d max_prefill_bsz=%d\n",
                  static_cast<unsigned long long>(ticket), request_label.c_str(), lanes,
                  queue_.empty() ? std::size_t(0) : queue_.size() - 1, reserved_batch_size_, dynamic_max_batch_size_);
    }
    condition_.wait_for(lock, std::chrono::milliseconds(100));
  }
}

void PrefillAdmissionController::release(int batch_size, std::uint64_t ticket) {
  std::lock_guard<std::mutex> lock(mutex_);
  reserved_batch_size_ = std::max(reserved_batch_size_ - batch_size, 0);
  refresh_capacity_locked();
  std::printf("[PrefillQueue] released ticket=%llu request_bsz=%d reserved_bsz=%d max_prefill_bsz=%d\n",
              static_cast<unsigned long long>(ticket), batch_size, reserved_batch_size_, dynamic_max_batch_size_);
  condition_.notify_all();
}

PrefillAdmissionController::Snapshot PrefillAdmissionController::snapshot(bool refresh_capacity) {
  std::lock_guard<std::mutex> lock(mutex_);
  if (refresh_capacity) refresh_capacity_locked();
  Snapshot out;
  out.hard_max_batch_size = hard_max_batch_size_;
  out.dynamic_max_batch_size = dynamic_max_batch_size_;
  out.reserved_batch_size = reserved_batch_size_;
  out.queued_requests = queue_.size();
  out.capacity = capacity_;
  return out;
}

}  // namespace rwkv7_server
