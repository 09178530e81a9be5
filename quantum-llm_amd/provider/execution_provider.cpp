// Provider registry: registration checks and per-kernel selection
// (runtime/src/execution_provider.cpp:10-131).  For every kernel the model
// requires, the winner is the registered provider whose capability has that
// name, whose ABI range holds the required version and whose validator
// accepts the model; among several, the highest priority, then the smaller
// name.  The compiled program records the winner of every kernel.
#include "expert/runtime/execution_provider.hpp"

#include <algorithm>
#include <set>
#include <stdexcept>
#include <string>

namespace expert::runtime {
namespace {

struct Choice final {
  std::uint32_t provider{};
  std::uint32_t capability{};
};

bool serves(const KernelCapability& offered, const KernelRequirement& required) {
  return offered.capability == required.capability &&
         required.abi_version >= offered.minimum_abi &&
         required.abi_version <= offered.maximum_abi;
}

}  // namespace

Status ExecutionProviderRegistry::add(
    ExecutionProviderDefinition provider) noexcept {
  try {
    if (provider.name.empty() || provider.capabilities.empty())
      return {ErrorCode::invalid_argument,
              "execution provider definition is incomplete"};
    for (const auto& known : providers_)
      if (known.name == provider.name)
        return {ErrorCode::invalid_argument,
                "execution provider name is duplicated"};
    std::set<std::string_view> seen;
    for (const auto& offered : provider.capabilities) {
      const bool sound = !offered.capability.empty() &&
                         offered.minimum_abi != 0U &&
                         offered.maximum_abi >= offered.minimum_abi &&
                         seen.insert(offered.capability).second;
      if (!sound)
        return {ErrorCode::invalid_argument,
                "execution provider capability is invalid or duplicated"};
    }
    providers_.push_back(std::move(provider));
    return Status::success();
  } catch (const std::exception& error) {
    return {ErrorCode::internal,
            std::string("execution provider registration failed: ") +
                error.what()};
  }
}

BindExecutionProviderResult ExecutionProviderRegistry::bind(
    const ModelDescriptor& descriptor,
    ExecutionProviderBindingMode mode) const noexcept {
  try {
    if (const auto valid = validate_model_descriptor(descriptor); !valid.ok())
      return {{valid.code(), std::string(valid.message())}, {}};

    std::vector<Choice> chosen;
    std::vector<KernelCapability> chosen_capabilities;
    for (const auto& required : descriptor.required_kernels) {
      std::optional<Choice> best;
      for (std::uint32_t p = 0; p < providers_.size(); ++p) {
        const auto& candidate = providers_[p];
        if (mode == ExecutionProviderBindingMode::executable &&
            !candidate.implementation)
          continue;
        for (std::uint32_t c = 0; c < candidate.capabilities.size(); ++c) {
          const auto& offered = candidate.capabilities[c];
          if (!serves(offered, required)) continue;
          if (offered.validate && !offered.validate(descriptor).ok()) continue;
          const bool wins =
              !best || candidate.priority > providers_[best->provider].priority ||
              (candidate.priority == providers_[best->provider].priority &&
               candidate.name < providers_[best->provider].name);
          if (wins) best = Choice{p, c};
        }
      }
      if (!best)
        return {{ErrorCode::invalid_argument,
                 "no execution provider implements required kernel: " +
                     required.capability},
                {}};
      chosen.push_back(*best);
      chosen_capabilities.push_back(
          providers_[best->provider].capabilities[best->capability]);
    }

    auto compiled = compile_model_program(descriptor, chosen_capabilities);
    if (!compiled.status.ok())
      return {{compiled.status.code(), std::string(compiled.status.message())},
              {}};
    BoundExecutionProvider plan;
    plan.model_content_hash = descriptor.content_hash;
    plan.model_schema_version = descriptor.schema_version;
    plan.program = std::move(compiled.program);
    std::set<std::uint32_t> referenced;
    for (auto& kernel : plan.program.kernels) {
      const auto& choice = chosen.at(kernel.requirement_index);
      kernel.provider_registry_index = choice.provider;
      kernel.provider_capability_index = choice.capability;
      referenced.insert(choice.provider);
    }
    for (const auto index : referenced)
      plan.providers.push_back({providers_[index].name, index,
                                providers_[index].implementation});
    return {Status::success(), std::move(plan)};
  } catch (const std::exception& error) {
    return {{ErrorCode::internal,
             std::string("execution provider binding failed: ") + error.what()},
            {}};
  }
}

}  // namespace expert::runtime
