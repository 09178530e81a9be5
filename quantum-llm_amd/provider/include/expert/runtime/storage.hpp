// Status and error codes of the common runtime and the digest type
// (runtime/include/expert/runtime/storage.hpp:17-47); the storage requests
// of that header belong to routed-expert paging and are not restated.
#pragma once

#include <array>
#include <cstddef>
#include <cstdint>
#include <string>
#include <string_view>
#include <utility>

namespace expert::runtime {

// storage.hpp:17-45
enum class ErrorCode : std::uint8_t {
  ok,
  cancelled,
  deadline_exceeded,
  backpressure,
  invalid_argument,
  open_failed,
  io_failed,
  short_read,
  checksum_mismatch,
  upload_failed,
  internal,
};

class Status final {
 public:
  Status() = default;
  Status(ErrorCode code, std::string message)
      : code_(code), message_(std::move(message)) {}
  [[nodiscard]] static Status success() { return {}; }
  [[nodiscard]] bool ok() const noexcept { return code_ == ErrorCode::ok; }
  [[nodiscard]] ErrorCode code() const noexcept { return code_; }
  [[nodiscard]] std::string_view message() const noexcept { return message_; }

 private:
  ErrorCode code_{ErrorCode::ok};
  std::string message_;
};

// storage.hpp:47
using Sha256Digest = std::array<std::byte, 32>;

}  // namespace expert::runtime
