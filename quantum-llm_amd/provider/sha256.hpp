// SHA-256 (FIPS 180-4) for authenticating artifact files: the program file
// against the manifest, packs against their index entries, record payloads
// against their headers.  Same interface as the reference's
// runtime/include/expert/runtime/sha256.hpp:11-29.
#pragma once

#include <array>
#include <cstddef>
#include <cstdint>
#include <span>

namespace expert::runtime {

// storage.hpp:47
using Sha256Digest = std::array<std::byte, 32>;

class Sha256 final {
 public:
  Sha256() noexcept;
  void update(std::span<const std::byte> input) noexcept;
  // The digest of everything fed so far; further updates are ignored.
  [[nodiscard]] Sha256Digest finalize() noexcept;

 private:
  void compress(const std::byte* block) noexcept;
  std::array<std::uint32_t, 8> state_{};
  std::array<std::byte, 64> pending_{};
  std::size_t pending_bytes_{};
  std::uint64_t message_bytes_{};
  Sha256Digest digest_{};
  bool finalized_{};
};

[[nodiscard]] Sha256Digest sha256(std::span<const std::byte> input) noexcept;
[[nodiscard]] bool constant_time_equal(const Sha256Digest& left,
                                       const Sha256Digest& right) noexcept;

}  // namespace expert::runtime
