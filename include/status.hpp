// Error carrier of the checkpoint reader: the reference's `llm_infer::Status` / `Result<T>` (include/status.hpp:7-60),
// same names and members so that code written against the reference's reader compiles against this one.  Nothing
// here throws; a failed Result holds a default-constructed value and the message.
#pragma once

#include <string>
#include <utility>

namespace llm_infer {

class Status {
public:
  Status() = default;
  static Status ok() { return Status(); }
  static Status error(std::string message) {
    Status s;
    s.failed_ = true;
    s.text_ = std::move(message);
    return s;
  }
  bool ok_status() const { return !failed_; }
  const std::string& message() const { return text_; }

private:
  bool failed_ = false;
  std::string text_;
};

template <typename T>
class Result {
public:
  Result(T value) : payload_(std::move(value)) {}           // NOLINT: implicit, as in the reference
  Result(Status status) : state_(std::move(status)) {}      // NOLINT
  bool ok() const { return state_.ok_status(); }
  const Status& status() const { return state_; }
  const T& value() const { return payload_; }
  T& value() { return payload_; }

private:
  T payload_{};
  Status state_;
};

}  // namespace llm_infer
