// The artifact-declared model program (`runtime-model.tsv`): what the model
// needs (kernel capabilities and ABIs), its operations in order with their
// integer parameters, tensor roles and SSA values, and the optional exact
// (speculative) decode service.  Types and functions carry the names and
// meanings of runtime/include/expert/runtime/model_descriptor.hpp:18-293,
// the compiled form (CompiledModelProgram, :195-262) included.
#pragma once

#include "expert/runtime/storage.hpp"

#include <cstdint>
#include <filesystem>
#include <functional>
#include <limits>
#include <map>
#include <optional>
#include <span>
#include <string>
#include <string_view>
#include <utility>
#include <vector>

namespace expert::runtime {

// Layer of an operation that belongs to the model, not to a layer (:20-21).
inline constexpr std::uint32_t kModelLevelOperationLayer =
    std::numeric_limits<std::uint32_t>::max();

struct ModelDescriptor;

using ParameterMap = std::map<std::string, std::uint64_t, std::less<>>;
using BindingMap = std::map<std::string, std::string, std::less<>>;

// :28-32
struct RouterProgramDescriptor final {
  std::string capability;
  std::uint32_t abi_version{1U};
  ParameterMap parameters;
};

// :37-55
struct RoutedExpertComponentDescriptor final {
  std::string name;
  std::uint64_t namespace_id{};
  std::uint32_t layer_count{};
  std::uint32_t experts_per_layer{};
  std::uint32_t route_width{};
  std::uint32_t shared_experts_per_layer{};
  std::uint32_t hidden_size{};
  std::uint32_t intermediate_size{};
  std::string execution_capability;
  std::uint32_t execution_abi{1U};
  std::uint32_t source_abi{};
  std::uint32_t encoding_abi{};
  std::string encoding;
  ParameterMap attributes;
  RouterProgramDescriptor router;
};

// :60-63
struct KernelRequirement final {
  std::string capability;
  std::uint32_t abi_version{1U};
};

// :65-82
struct KernelCapability final {
  std::string capability;
  std::uint32_t minimum_abi{1U};
  std::uint32_t maximum_abi{1U};
  std::function<Status(const ModelDescriptor&)> validate;

  KernelCapability(std::string capability_value,
                   std::uint32_t minimum_abi_value = 1U,
                   std::uint32_t maximum_abi_value = 1U,
                   std::function<Status(const ModelDescriptor&)> validator = {})
      : capability(std::move(capability_value)),
        minimum_abi(minimum_abi_value),
        maximum_abi(maximum_abi_value),
        validate(std::move(validator)) {}
};

// :87-96
struct LayerProgramDescriptor final {
  std::uint32_t logical_layer{};
  std::string block_capability;
  std::uint32_t block_abi_version{1U};
  std::string routed_component;
  std::uint32_t component_layer{};
  ParameterMap parameters;
};

// :102-122
struct OperationProgramDescriptor final {
  std::uint32_t logical_operation{};
  std::uint32_t logical_layer{};
  std::string capability;
  std::uint32_t abi_version{1U};
  std::string routed_component;
  std::uint32_t component_layer{};
  ParameterMap parameters;
  BindingMap tensor_bindings;  // provider role -> tensor name in the dense index
  struct ValueBinding final {
    std::string value;
    std::string abi;
  };
  // provider port -> artifact-declared SSA value and its ABI
  std::map<std::string, ValueBinding, std::less<>> input_bindings;
  std::map<std::string, ValueBinding, std::less<>> output_bindings;

  OperationProgramDescriptor() = default;
  OperationProgramDescriptor(
      std::uint32_t logical_operation_value, std::uint32_t logical_layer_value,
      std::string capability_value, std::uint32_t abi_version_value,
      std::string routed_component_value, std::uint32_t component_layer_value,
      ParameterMap parameters_value = {}, BindingMap tensor_bindings_value = {},
      std::map<std::string, ValueBinding, std::less<>> input_bindings_value = {},
      std::map<std::string, ValueBinding, std::less<>> output_bindings_value = {})
      : logical_operation(logical_operation_value),
        logical_layer(logical_layer_value),
        capability(std::move(capability_value)),
        abi_version(abi_version_value),
        routed_component(std::move(routed_component_value)),
        component_layer(component_layer_value),
        parameters(std::move(parameters_value)),
        tensor_bindings(std::move(tensor_bindings_value)),
        input_bindings(std::move(input_bindings_value)),
        output_bindings(std::move(output_bindings_value)) {}
};

// :149-152
struct ProgramEndpointDescriptor final {
  std::string value;
  std::string abi;
};

// :160-170
struct ExactDecodeProgramDescriptor final {
  std::string capability;
  std::uint32_t abi_version{1U};
  std::uint32_t maximum_emitted_tokens{};
  ParameterMap parameters;
  BindingMap tensor_bindings;
};

// :172-198
struct ModelDescriptor final {
  std::uint32_t schema_version{1U};
  std::string architecture_id;
  Sha256Digest content_hash{};
  std::uint32_t vocab_size{};
  std::uint32_t max_context_tokens{};
  std::uint32_t hidden_size{};
  ParameterMap attributes;
  BindingMap tensor_bindings;
  std::vector<RoutedExpertComponentDescriptor> routed_components;
  std::vector<KernelRequirement> required_kernels;
  std::vector<LayerProgramDescriptor> layer_program;
  std::vector<OperationProgramDescriptor> operation_program;
  std::map<std::string, ProgramEndpointDescriptor, std::less<>> program_inputs;
  std::map<std::string, ProgramEndpointDescriptor, std::less<>> program_outputs;
  std::optional<ExactDecodeProgramDescriptor> exact_decode_program;
};

// The program with every name resolved to an index, once, at start-up
// (:195-262): which capability of which provider serves a required kernel,
// which SSA value a port reads or writes.
struct CompiledKernelBinding final {
  std::uint32_t requirement_index{};
  // filled in by ExecutionProviderRegistry::bind; compile_model_program()
  // compiles against one capability table and leaves it zero
  std::uint32_t provider_registry_index{};
  std::uint32_t provider_capability_index{};
};

struct CompiledLayerProgram final {
  std::uint32_t logical_layer{};
  std::uint32_t block_kernel_binding{};
  std::optional<std::uint32_t> routed_component_index;
  std::uint32_t component_layer{};
  ParameterMap parameters;
};

struct CompiledOperationProgram final {
  std::uint32_t logical_operation{};
  std::uint32_t logical_layer{};
  std::uint32_t kernel_binding{};
  std::optional<std::uint32_t> routed_component_index;
  std::uint32_t component_layer{};
  ParameterMap parameters;
  BindingMap tensor_bindings;
  struct ValueBinding final {
    std::string port;
    std::uint32_t value_index{};
  };
  std::vector<ValueBinding> input_values;
  std::vector<ValueBinding> output_values;
};

struct CompiledProgramValue final {
  std::string name;
  std::string abi;
};

struct CompiledProgramEndpoint final {
  std::string role;
  std::uint32_t value_index{};
};

struct CompiledExactDecodeProgram final {
  std::uint32_t kernel_binding{};
  std::uint32_t maximum_emitted_tokens{};
  ParameterMap parameters;
  BindingMap tensor_bindings;
};

struct CompiledModelProgram final {
  std::vector<CompiledKernelBinding> kernels;
  std::vector<CompiledLayerProgram> layers;
  std::vector<CompiledOperationProgram> operations;
  std::vector<CompiledProgramValue> values;
  std::vector<CompiledProgramEndpoint> inputs;
  std::vector<CompiledProgramEndpoint> outputs;
  std::optional<CompiledExactDecodeProgram> exact_decode;
};

struct CompileModelProgramResult final {
  Status status;
  CompiledModelProgram program;
};

struct ParseModelDescriptorResult final {
  Status status;
  ModelDescriptor descriptor;
};

// :269-293
[[nodiscard]] Status validate_model_descriptor(
    const ModelDescriptor& descriptor) noexcept;
[[nodiscard]] Status validate_routed_component(
    const RoutedExpertComponentDescriptor& component,
    std::uint32_t model_hidden_size) noexcept;
[[nodiscard]] Status provider_supports_model(
    const ModelDescriptor& descriptor,
    std::span<const KernelCapability> capabilities) noexcept;
[[nodiscard]] CompileModelProgramResult compile_model_program(
    const ModelDescriptor& descriptor,
    std::span<const KernelCapability> capabilities) noexcept;
// Parses the line-oriented program text.  Component namespace offsets are
// added to `namespace_base` (never zero), which the loader derives from the
// artifact's content hash.
[[nodiscard]] ParseModelDescriptorResult parse_model_descriptor_artifact(
    std::string_view text, const Sha256Digest& content_hash,
    std::uint64_t namespace_base) noexcept;
// Reads the program file, which must have exactly `expected_bytes` bytes and
// the given SHA-256, then parses it.
[[nodiscard]] ParseModelDescriptorResult load_model_descriptor_artifact(
    const std::filesystem::path& path, std::uint64_t expected_bytes,
    const Sha256Digest& expected_sha256, const Sha256Digest& content_hash,
    std::uint64_t namespace_base) noexcept;
[[nodiscard]] std::uint64_t expert_table_entries(
    const RoutedExpertComponentDescriptor& component) noexcept;
[[nodiscard]] const RoutedExpertComponentDescriptor* find_routed_component(
    const ModelDescriptor& descriptor, std::string_view name) noexcept;
[[nodiscard]] std::uint64_t namespace_id_from_content_hash(
    const Sha256Digest& digest) noexcept;

}  // namespace expert::runtime
