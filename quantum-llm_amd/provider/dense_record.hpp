// Header check of a dense record inside an Expert Pack v1 pack file; the
// record layout is docs/expert-pack-v1.md:20-36 with the header of
// compiler/expert_pack/constants.py:72-92.
#pragma once

#include "expert/runtime/model_artifact.hpp"

#include <cstddef>
#include <cstdint>

namespace expert::runtime {

// Checks the 256-byte header of a dense record against its index entry:
// magic, version, sizes, row-major flag, rank and shape, SHA-256 of the name,
// section ranges, and the byte counts the quantisation ABI implies
// (compiler/expert_pack/validate.py:148-325, without re-hashing the payload,
// which the pack's own checksum covers).  `record` points at the header.
[[nodiscard]] Status validate_dense_record(const ArtifactDenseTensor& entry,
                                           const std::byte* record,
                                           std::uint64_t available_bytes) noexcept;

}  // namespace expert::runtime
