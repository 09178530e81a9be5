// Capability negotiation between a model program and the registered providers
// (runtime/include/expert/runtime/execution_provider.hpp:13-77): a provider
// is a name, a priority and a capability table, optionally with the callable
// implementation behind it; bind() picks, per required kernel, the provider
// with the highest priority whose ABI range and validator accept the model.
#pragma once

#include "expert/runtime/model_descriptor.hpp"

#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <utility>
#include <vector>

namespace expert::runtime {

class IOperationProvider;

enum class ExecutionProviderBindingMode : std::uint8_t {
  metadata,
  executable,
};

// :23-39
struct ExecutionProviderDefinition final {
  std::string name;
  std::uint32_t priority{};
  std::vector<KernelCapability> capabilities;
  // absent for control-plane inspection; executable binding skips such entries
  std::shared_ptr<IOperationProvider> implementation;

  ExecutionProviderDefinition() = default;
  ExecutionProviderDefinition(
      std::string name_value, std::uint32_t priority_value,
      std::vector<KernelCapability> capabilities_value,
      std::shared_ptr<IOperationProvider> implementation_value = {})
      : name(std::move(name_value)), priority(priority_value),
        capabilities(std::move(capabilities_value)),
        implementation(std::move(implementation_value)) {}
};

// :41-60
struct BoundExecutionProviderReference final {
  std::string name;
  std::uint32_t registry_index{};
  std::shared_ptr<IOperationProvider> implementation;
};

struct BoundExecutionProvider final {
  std::vector<BoundExecutionProviderReference> providers;
  Sha256Digest model_content_hash{};
  std::uint32_t model_schema_version{};
  CompiledModelProgram program;
};

struct BindExecutionProviderResult final {
  Status status;
  BoundExecutionProvider provider;
};

// :66-77
class ExecutionProviderRegistry final {
 public:
  [[nodiscard]] Status add(ExecutionProviderDefinition provider) noexcept;
  [[nodiscard]] BindExecutionProviderResult bind(
      const ModelDescriptor& descriptor,
      ExecutionProviderBindingMode mode =
          ExecutionProviderBindingMode::metadata) const noexcept;
  [[nodiscard]] std::size_t size() const noexcept { return providers_.size(); }

 private:
  std::vector<ExecutionProviderDefinition> providers_;
};

}  // namespace expert::runtime
