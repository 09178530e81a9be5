// Reader of a published Expert Pack v1 artifact directory: manifest.json names
// the model program (runtime-model.tsv, bound by size and SHA-256), the pack
// files and, per dense tensor, its record inside a pack.  Dense-only: an
// artifact whose program declares routed expert components is rejected, since
// this provider executes none.  Names and meanings follow
// runtime/include/expert/runtime/model_artifact.hpp:15-92.
#pragma once

#include "expert/runtime/model_descriptor.hpp"

#include <cstdint>
#include <filesystem>
#include <memory>
#include <string>
#include <string_view>
#include <vector>

namespace expert::runtime {

struct ArtifactPack final {
  std::string name;
  std::string kind;  // "dense" or "experts"
  std::filesystem::path path;
  std::uint64_t bytes{};
  Sha256Digest sha256{};
};

// Offsets of the sections are relative to the record, which starts
// `record_offset` bytes into the pack.
struct ArtifactDenseTensor final {
  std::string name;
  std::string pack;
  std::uint64_t record_offset{};
  std::uint64_t stored_bytes{};
  std::string encoding;
  std::uint32_t quant_abi{};
  std::vector<std::uint32_t> shape;
  std::uint64_t data_offset{};
  std::uint64_t data_bytes{};
  std::uint64_t scale_offset{};
  std::uint64_t scale_bytes{};
  Sha256Digest payload_sha256{};
};

class ModelArtifact final {
 public:
  ModelArtifact() = default;
  ModelArtifact(const ModelArtifact&) = delete;
  ModelArtifact& operator=(const ModelArtifact&) = delete;
  ModelArtifact(ModelArtifact&&) noexcept = default;
  ModelArtifact& operator=(ModelArtifact&&) noexcept = default;

  [[nodiscard]] static Status load_expert_pack_v1(
      const std::filesystem::path& root, ModelArtifact& destination) noexcept;
  // Picks the storage adapter from the manifest's format name and version.
  [[nodiscard]] static Status load(const std::filesystem::path& root,
                                   ModelArtifact& destination) noexcept;
  // Changes the draft depth of the in-memory program only (model_artifact.cpp:
  // 75-101): the artifact must declare an exact-decode ABI >= 2 whose
  // maximum_emitted_tokens equals its draft_depth + 1.
  [[nodiscard]] Status configure_mtp_draft_depth(std::uint32_t depth) noexcept;

  [[nodiscard]] const std::filesystem::path& root() const noexcept { return root_; }
  [[nodiscard]] const ModelDescriptor& model() const noexcept { return model_; }
  [[nodiscard]] const std::vector<ArtifactPack>& packs() const noexcept {
    return packs_;
  }
  [[nodiscard]] const std::vector<ArtifactDenseTensor>& dense_tensors()
      const noexcept {
    return dense_tensors_;
  }
  [[nodiscard]] const ArtifactPack* find_pack(std::string_view name) const noexcept;

 private:
  std::filesystem::path root_;
  ModelDescriptor model_;
  std::vector<ArtifactPack> packs_;
  std::vector<ArtifactDenseTensor> dense_tensors_;
};

}  // namespace expert::runtime
