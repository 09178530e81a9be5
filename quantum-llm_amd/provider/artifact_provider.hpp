// The module factory: an artifact directory in, a prepared provider out.
// Loads and authenticates the artifact, derives the dense geometry from the
// model program, constructs the provider and binds every operation of the
// program to its tensors - what the reference does in
// make_sm86_dense_fp4_callable_provider (runtime/tools/dense_fp4_provider.cpp:
// 11402-11470) followed by the executor's start-up loop
// (runtime/src/program_executor.cpp:1725-1826).
#pragma once

#include "dense_fp4_provider.hpp"
#include "model_artifact.hpp"

#include <filesystem>
#include <memory>
#include <string>
#include <vector>

namespace qllm {

struct ArtifactProviderOptions final {
  std::uint32_t max_context{};      // 0 = the artifact's max_context_tokens
  std::uint32_t kv_page_tokens{256};
  // "q4-f16-per-head" (also chosen by "artifact") or "fp16"
  std::string kv_cache_dtype{"artifact"};
  std::uint32_t mtp_draft_depth{};  // 0 = the artifact's declared depth
};

struct ExecutionProviderModule final {
  er::WorkerProviderDefinition definition;
  std::shared_ptr<er::ModelArtifact> artifact;
  std::shared_ptr<er::IModelTensorStore> tensor_store;
  std::shared_ptr<Mi355DenseFp4Provider> implementation;
  // one prepared operation per program operation, then the exact decode
  std::vector<std::shared_ptr<const er::IPreparedOperation>> operations;
  std::shared_ptr<const er::IPreparedOperation> exact_decode;
  er::ServiceContract service;
};

struct CreateExecutionProviderModuleResult final {
  er::Status status;
  ExecutionProviderModule module;
};

// The descriptor check behind every capability of this provider: the slice of
// validate_dense_fp4_descriptor (dense_fp4_provider.cpp:804-994) that concerns
// a dense full-attention decoder.
[[nodiscard]] er::Status validate_dense_fp4_descriptor(
    const er::ModelDescriptor& model);

// Geometry from the program's attributes, capabilities and tensor shapes.
[[nodiscard]] er::Status dense_geometry_from_artifact(
    const er::ModelDescriptor& model, er::IModelTensorStore& tensors,
    const ArtifactProviderOptions& options, DenseGeometry& geometry);

[[nodiscard]] CreateExecutionProviderModuleResult
make_mi355_dense_fp4_callable_provider(const std::filesystem::path& artifact_root,
                                       const ArtifactProviderOptions& options);

}  // namespace qllm
