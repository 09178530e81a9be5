// The dense packs of an artifact as immutable tensors
// (runtime/include/expert/runtime/model_tensor_store.hpp:15-34).
#pragma once

#include "expert/runtime/model_artifact.hpp"
#include "expert/runtime/program_executor.hpp"

#include <memory>
#include <string_view>

namespace expert::runtime {

// Read-only memory mapping of the dense packs, each checked against the
// manifest's SHA-256 when it is mapped.  resolve() hands out views into the
// mapping; they stay valid while the store or any resolved tensor lives.
class MappedModelTensorStore final : public IModelTensorStore {
 public:
  MappedModelTensorStore();
  MappedModelTensorStore(const MappedModelTensorStore&) = delete;
  MappedModelTensorStore& operator=(const MappedModelTensorStore&) = delete;
  MappedModelTensorStore(MappedModelTensorStore&&) noexcept;
  MappedModelTensorStore& operator=(MappedModelTensorStore&&) noexcept;
  ~MappedModelTensorStore() override;

  [[nodiscard]] static Status create(const ModelArtifact& artifact,
                                     MappedModelTensorStore& destination) noexcept;
  [[nodiscard]] ResolveModelTensorResult resolve(std::string_view name) override;
  [[nodiscard]] bool valid() const noexcept;

 private:
  struct Core;
  std::shared_ptr<Core> core_;
};

}  // namespace expert::runtime
