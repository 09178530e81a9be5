// Binds a model program against a set of providers described in text and
// prints the outcome - status, the providers the plan refers to, the compiled
// program - in a canonical form, for comparing two implementations of the
// registry and of compile_model_program.  Written against the names of
// namespace expert::runtime only, so the same code runs over this library's
// headers and over any other implementation with the same declarations
// (runtime/include/expert/runtime/execution_provider.hpp, model_descriptor.hpp:
// 195-262).
//
// Provider description, one record per line, fields separated by tabs:
//   provider <name> <priority> <callable 0|1>
//   capability <name> <minimum_abi> <maximum_abi>      (of the provider above)
#pragma once

#include "expert/runtime/execution_provider.hpp"
#include "expert/runtime/program_executor.hpp"

#include "descriptor_dump.hpp"

#include <cstdint>
#include <memory>
#include <sstream>
#include <string>
#include <string_view>
#include <vector>

namespace qllm::dump {

// A callable provider that is never called: executable binding only asks
// whether an implementation exists.
class InertProvider final : public expert::runtime::IOperationProvider {
 public:
  expert::runtime::PrepareOperationResult prepare(
      const expert::runtime::OperationPreparationContext&) override {
    return {{expert::runtime::ErrorCode::internal, "inert"}, {}};
  }
  expert::runtime::CreateOperationRequestStateResult create_request_state(
      const expert::runtime::ProgramRequestContext&) override {
    return {{expert::runtime::ErrorCode::internal, "inert"}, {}};
  }
  expert::runtime::OperationExecutionHandle execute(
      const expert::runtime::IPreparedOperation&,
      const std::shared_ptr<expert::runtime::IOperationProviderRequestState>&,
      const expert::runtime::OperationInvocation&) override {
    return {};
  }
};

inline std::string compiled_program(
    const expert::runtime::CompiledModelProgram& program) {
  Lines out;
  for (const auto& kernel : program.kernels)
    out.add("kernel", kernel.requirement_index, kernel.provider_registry_index,
            kernel.provider_capability_index);
  for (const auto& layer : program.layers) {
    out.add("layer", layer.logical_layer, layer.block_kernel_binding,
            layer.routed_component_index
                ? std::to_string(*layer.routed_component_index)
                : std::string("-"),
            layer.component_layer);
    for (const auto& [key, value] : layer.parameters)
      out.add("layer_parameter", layer.logical_layer, key, value);
  }
  for (const auto& op : program.operations) {
    out.add("operation", op.logical_operation, op.logical_layer, op.kernel_binding,
            op.routed_component_index ? std::to_string(*op.routed_component_index)
                                      : std::string("-"),
            op.component_layer);
    for (const auto& [key, value] : op.parameters)
      out.add("operation_parameter", op.logical_operation, key, value);
    for (const auto& [role, tensor] : op.tensor_bindings)
      out.add("operation_tensor", op.logical_operation, role, tensor);
    for (const auto& value : op.input_values)
      out.add("operation_input", op.logical_operation, value.port,
              value.value_index);
    for (const auto& value : op.output_values)
      out.add("operation_output", op.logical_operation, value.port,
              value.value_index);
  }
  for (const auto& value : program.values) out.add("value", value.name, value.abi);
  for (const auto& endpoint : program.inputs)
    out.add("input", endpoint.role, endpoint.value_index);
  for (const auto& endpoint : program.outputs)
    out.add("output", endpoint.role, endpoint.value_index);
  if (program.exact_decode) {
    out.add("exact_decode", program.exact_decode->kernel_binding,
            program.exact_decode->maximum_emitted_tokens);
    for (const auto& [key, value] : program.exact_decode->parameters)
      out.add("exact_decode_parameter", key, value);
    for (const auto& [role, tensor] : program.exact_decode->tensor_bindings)
      out.add("exact_decode_tensor", role, tensor);
  }
  return out.take();
}

// Returns the report; the first line is "status <code> <message>".
inline std::string bind_report(std::string_view program_text,
                               const expert::runtime::Sha256Digest& content_hash,
                               std::uint64_t namespace_base,
                               std::string_view providers_text, bool executable) {
  namespace er = expert::runtime;
  Lines out;
  const auto status_line = [&](const char* stage, const er::Status& status) {
    out.add("status", stage, static_cast<std::uint32_t>(status.code()),
            std::string(status.message()));
  };
  auto parsed =
      er::parse_model_descriptor_artifact(program_text, content_hash, namespace_base);
  if (!parsed.status.ok()) {
    status_line("parse", parsed.status);
    return out.take();
  }
  er::ExecutionProviderRegistry registry;
  std::vector<er::ExecutionProviderDefinition> definitions;
  std::istringstream lines{std::string(providers_text)};
  std::string line;
  while (std::getline(lines, line)) {
    if (line.empty()) continue;
    std::vector<std::string> fields;
    std::istringstream split(line);
    std::string field;
    while (std::getline(split, field, '\t')) fields.push_back(field);
    if (fields[0] == "provider" && fields.size() == 4U) {
      er::ExecutionProviderDefinition definition;
      definition.name = fields[1];
      definition.priority = static_cast<std::uint32_t>(std::stoul(fields[2]));
      if (fields[3] == "1") definition.implementation = std::make_shared<InertProvider>();
      definitions.push_back(std::move(definition));
    } else if (fields[0] == "capability" && fields.size() == 4U &&
               !definitions.empty()) {
      definitions.back().capabilities.push_back(er::KernelCapability{
          fields[1], static_cast<std::uint32_t>(std::stoul(fields[2])),
          static_cast<std::uint32_t>(std::stoul(fields[3]))});
    } else {
      out.add("status", "providers", std::uint32_t{4}, "bad provider description");
      return out.take();
    }
  }
  for (auto& definition : definitions) {
    const auto name = definition.name;
    const auto added = registry.add(std::move(definition));
    out.add("add", name, static_cast<std::uint32_t>(added.code()),
            std::string(added.message()));
  }
  const auto bound = registry.bind(
      parsed.descriptor, executable ? er::ExecutionProviderBindingMode::executable
                                    : er::ExecutionProviderBindingMode::metadata);
  status_line("bind", bound.status);
  if (!bound.status.ok()) return out.take();
  out.add("plan", hex(bound.provider.model_content_hash),
          bound.provider.model_schema_version);
  for (const auto& reference : bound.provider.providers)
    out.add("plan_provider", reference.name, reference.registry_index,
            reference.implementation ? "callable" : "metadata");
  return out.take() + compiled_program(bound.provider.program);
}

}  // namespace qllm::dump
