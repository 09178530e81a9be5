// Header check of a dense record (docs/expert-pack-v1.md:20-36; header
// fields compiler/expert_pack/constants.py:72-92; the checks of
// compiler/expert_pack/validate.py:148-325 without re-hashing the payload).
#include "dense_record.hpp"

#include "expert/runtime/sha256.hpp"

#include <algorithm>
#include <cstring>
#include <span>
#include <stdexcept>
#include <string>

namespace expert::runtime {
namespace {

// ---- dense record header (little endian, 148 bytes used of 256) ------------

constexpr std::size_t kHeaderBytes = 256;
constexpr std::size_t kHeaderUsedBytes = 148;
constexpr std::uint32_t kFlagRowMajor = 1U << 0;
constexpr std::uint32_t kFlagSymmetric = 1U << 2;
constexpr std::uint32_t kFlagPerRowScales = 1U << 3;

struct DenseHeader final {
  std::uint16_t version{};
  std::uint16_t header_bytes{};
  std::uint32_t flags{};
  std::uint32_t quant_abi{};
  std::uint32_t rank{};
  std::uint32_t dimensions[5]{};
  std::uint64_t record_bytes{};
  std::uint64_t data_offset{};
  std::uint64_t data_bytes{};
  std::uint64_t scale_offset{};
  std::uint64_t scale_bytes{};
  Sha256Digest name_sha256{};
  Sha256Digest payload_sha256{};
};

template <typename Integer>
Integer little_endian(const std::byte* bytes) {
  Integer value{};
  for (std::size_t index = 0; index < sizeof(Integer); ++index)
    value |= static_cast<Integer>(
        static_cast<Integer>(std::to_integer<std::uint8_t>(bytes[index]))
        << (8U * index));
  return value;
}

DenseHeader decode_header(const std::byte* record) {
  DenseHeader header;
  const std::byte* cursor = record + 8;
  header.version = little_endian<std::uint16_t>(cursor);
  header.header_bytes = little_endian<std::uint16_t>(cursor + 2);
  cursor += 4;
  header.flags = little_endian<std::uint32_t>(cursor);
  header.quant_abi = little_endian<std::uint32_t>(cursor + 4);
  header.rank = little_endian<std::uint32_t>(cursor + 8);
  cursor += 12;
  for (auto& dimension : header.dimensions) {
    dimension = little_endian<std::uint32_t>(cursor);
    cursor += 4;
  }
  std::uint64_t* const wide[5] = {&header.record_bytes, &header.data_offset,
                                  &header.data_bytes, &header.scale_offset,
                                  &header.scale_bytes};
  for (auto* field : wide) {
    *field = little_endian<std::uint64_t>(cursor);
    cursor += 8;
  }
  std::memcpy(header.name_sha256.data(), cursor, 32);
  std::memcpy(header.payload_sha256.data(), cursor + 32, 32);
  return header;
}

}  // namespace

Status validate_dense_record(const ArtifactDenseTensor& entry,
                             const std::byte* record,
                             std::uint64_t available_bytes) noexcept {
  const auto wrong = [&](const char* what) {
    return Status{ErrorCode::invalid_argument,
                  std::string(what) + ": " + entry.name};
  };
  try {
    if (!record || available_bytes < kHeaderBytes ||
        entry.stored_bytes < kHeaderBytes || entry.stored_bytes > available_bytes)
      return wrong("invalid dense size");
    if (std::memcmp(record, "EPDENS01", 8) != 0)
      return wrong("unknown dense record ABI");
    for (std::size_t index = kHeaderUsedBytes; index < kHeaderBytes; ++index)
      if (record[index] != std::byte{0})
        return wrong("dense header padding is nonzero");
    const DenseHeader header = decode_header(record);
    if (header.version != 1U) return wrong("unknown dense record ABI");
    if (header.header_bytes != kHeaderBytes)
      return wrong("invalid dense header fields");
    if (header.record_bytes != entry.stored_bytes)
      return wrong("dense record/manifest size mismatch");
    if (!(header.flags & kFlagRowMajor)) return wrong("dense record is not row-major");
    if (header.rank < 1U || header.rank > 5U) return wrong("invalid dense rank");
    if (header.rank < 5U && header.dimensions[4] != 0U)
      return wrong("invalid dense rank padding");
    if (entry.shape.size() != header.rank ||
        !std::equal(entry.shape.begin(), entry.shape.end(), header.dimensions))
      return wrong("dense shape mismatch");
    if (header.quant_abi != entry.quant_abi)
      return wrong("dense quantisation ABI mismatch");
    const auto name_bytes =
        std::as_bytes(std::span(entry.name.data(), entry.name.size()));
    if (sha256(name_bytes) != header.name_sha256)
      return wrong("dense name hash mismatch");
    if (header.data_offset != entry.data_offset ||
        header.data_bytes != entry.data_bytes)
      return wrong("dense data section mismatch");
    if (header.scale_offset != entry.scale_offset ||
        header.scale_bytes != entry.scale_bytes)
      return wrong("dense scale section mismatch");
    if (header.data_offset < kHeaderBytes ||
        header.data_offset > header.record_bytes ||
        header.data_bytes > header.record_bytes - header.data_offset)
      return wrong("bad dense data span");
    if (header.payload_sha256 != entry.payload_sha256)
      return wrong("dense payload/manifest checksum mismatch");

    std::uint64_t elements = 1;
    for (std::uint32_t index = 0; index < header.rank; ++index)
      elements *= header.dimensions[index];
    const std::uint64_t columns = header.dimensions[header.rank - 1U];
    const std::uint64_t rows = columns ? elements / columns : 0U;
    constexpr std::uint32_t kScaled = kFlagSymmetric | kFlagPerRowScales;
    if (header.quant_abi == 0U) {
      if (header.scale_offset != 0U || header.scale_bytes != 0U)
        return wrong("unknown dense quant ABI");
      const std::uint64_t element_bytes =
          entry.encoding == "I64" ? 8U : entry.encoding == "BF16" ? 2U : 4U;
      if (entry.encoding != "F32" && entry.encoding != "I64" &&
          entry.encoding != "BF16")
        return wrong("unknown raw dense dtype");
      if (header.data_bytes != elements * element_bytes)
        return wrong("raw dense data byte count mismatch");
    } else if (header.quant_abi == 3U) {  // FP4 E2M1, UE8M0 per 32 columns
      if ((header.flags & kScaled) != kScaled)
        return wrong("FP4 dense flags are incomplete");
      const std::uint64_t padded = (columns + 31U) / 32U * 32U;
      if (header.scale_offset % 256U) return wrong("unaligned dense scales");
      if (header.data_bytes != rows * padded / 2U)
        return wrong("FP4 dense data byte count mismatch");
      if (header.scale_bytes != rows * padded / 32U)
        return wrong("FP4 dense scale count mismatch");
    } else if (header.quant_abi == 1U) {  // int8 with one f32 scale per row
      if ((header.flags & kScaled) != kScaled)
        return wrong("INT8 dense flags are incomplete");
      if (header.rank != 2U) return wrong("INT8 dense storage requires a matrix");
      if (header.scale_offset % 256U) return wrong("unaligned dense scales");
      if (header.scale_bytes != std::uint64_t{header.dimensions[0]} * 4U)
        return wrong("dense scale count mismatch");
      if (header.data_bytes != elements)
        return wrong("INT8 dense data byte count mismatch");
    }
    if (header.scale_bytes &&
        (header.scale_offset > header.record_bytes ||
         header.scale_bytes > header.record_bytes - header.scale_offset))
      return wrong("bad dense scale span");
    return Status::success();
  } catch (const std::exception& error) {
    return {ErrorCode::internal, error.what()};
  }
}

}  // namespace expert::runtime
