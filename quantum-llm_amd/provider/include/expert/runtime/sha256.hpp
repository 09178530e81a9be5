// SHA-256 (FIPS 180-4) for authenticating artifact files: the program file
// against the manifest, packs against their index entries, record names
// against their headers.  sha256() and constant_time_equal() stand for the
// functions of the same names in the reference
// (runtime/include/expert/runtime/sha256.hpp:26-28).
#pragma once

#include "expert/runtime/storage.hpp"

#include <array>
#include <cstddef>
#include <cstdint>
#include <span>

namespace expert::runtime {

// Incremental form: feed() any number of times, then digest().
class Sha256Stream final {
 public:
  // `portable` keeps to plain integer code even where the CPU has SHA
  // instructions (both give the same digests; the flag exists for testing).
  explicit Sha256Stream(bool portable = false) noexcept;
  void feed(std::span<const std::byte> bytes) noexcept;
  [[nodiscard]] Sha256Digest digest() noexcept;

 private:
  void block(const std::byte* sixty_four_bytes) noexcept;
  std::uint32_t h_[8];
  std::byte partial_[64];
  std::size_t partial_size_{0};
  std::uint64_t total_size_{0};
  bool accelerated_{false};
};

[[nodiscard]] Sha256Digest sha256(std::span<const std::byte> input) noexcept;
[[nodiscard]] Sha256Digest sha256_portable(std::span<const std::byte> input) noexcept;
// Compares all 32 bytes whatever the first difference is.
[[nodiscard]] bool constant_time_equal(const Sha256Digest& left,
                                       const Sha256Digest& right) noexcept;

}  // namespace expert::runtime
