// The module factory: an artifact directory in, a provider module out - the
// artifact loaded and authenticated, the dense geometry derived from the model
// program, the provider constructed, the service contract filled in
// (make_sm86_dense_fp4_callable_provider, runtime/tools/dense_fp4_provider.cpp:
// 11402-11490) - and the start-up binding loop for hosts without the common
// VM.
#pragma once

#include "dense_fp4_provider.hpp"
#include "expert/runtime/model_artifact.hpp"
#include "expert/runtime/model_tensor_store.hpp"

#include <filesystem>
#include <memory>
#include <string>
#include <string_view>
#include <vector>

namespace qllm {

// Launch options of a worker as far as this provider reads them
// (WorkerLaunchOptions, runtime/include/expert/runtime/worker_contract.hpp:
// 15-58).
struct ArtifactProviderOptions final {
  std::uint32_t max_context{};      // 0 = the artifact's max_context_tokens
  std::uint32_t kv_page_tokens{256};
  // "q4-f16-per-head" (also chosen by "artifact") or "fp16"
  std::string kv_cache_dtype{"artifact"};
  std::uint32_t mtp_draft_depth{};  // 0 = the artifact's declared depth
  std::uint64_t vram_cache_bytes{1};  // echoed in the service contract
  std::string routed_vram_policy{"fixed"};
  std::uint32_t capacity{1};        // request slots
  bool profile_gpu_phases{};        // provider_gpu_*_ns telemetry, uncaptured passes
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

// The module factory with the signature the common runner calls
// (make_sm86_dense_fp4_callable_provider, dense_fp4_provider.cpp:11402-11412;
// forward declaration and call in runtime/tools/moe_vm_runner.cpp:50-54,
// 459-468).  Arguments that concern routed experts, RAM caches and secondary
// devices are accepted and not used: a dense resident decoder has none.
[[nodiscard]] er::CreateExecutionProviderModuleResult
make_mi355_dense_fp4_callable_provider(
    const std::filesystem::path& artifact_root, std::uint32_t max_context,
    std::uint32_t capacity, std::uint64_t ram_cache_bytes,
    std::uint64_t vram_cache_bytes, std::uint64_t kv_cache_bytes,
    std::uint32_t kv_page_tokens, std::string_view kv_cache_dtype,
    std::string_view placement_profile, std::string_view routed_vram_policy,
    bool profile_gpu_phases, bool discover_active_expert_devices,
    std::vector<int> active_expert_devices,
    std::uint64_t active_expert_device_cache_bytes,
    std::uint64_t active_expert_host_cache_bytes,
    std::uint32_t mtp_draft_depth);

// The same for a host that has loaded the artifact already (the artifact is
// read and hashed once).
[[nodiscard]] er::CreateExecutionProviderModuleResult
make_mi355_dense_fp4_module(std::shared_ptr<er::ModelArtifact> artifact,
                            const ArtifactProviderOptions& options);

// What the common VM's start-up does with a module
// (ExecutionProviderRegistry::add / bind, then the preparation loop of
// MoeProgramExecutor::create, runtime/src/program_executor.cpp:1725-1826), for
// hosts that drive the provider without that VM: every operation of the
// program bound to its tensors and prepared, in program order, then the exact
// decode program.
struct PreparedProgram final {
  er::BoundExecutionProvider bound;
  std::vector<std::shared_ptr<const er::IPreparedOperation>> operations;
  std::shared_ptr<const er::IPreparedOperation> exact_decode;
};
[[nodiscard]] er::Status prepare_program(const er::ModelDescriptor& model,
                                         const er::ExecutionProviderModule& module,
                                         PreparedProgram& prepared);

}  // namespace qllm
