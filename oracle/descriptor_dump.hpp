// Canonical text form of a parsed model descriptor and of an artifact's
// index, for comparing two loaders field by field.  The functions are
// templates over the descriptor / artifact types, so the same writer runs over
// this library's types and over any other implementation with the same member
// names (runtime/include/expert/runtime/model_descriptor.hpp:172-198,
// model_artifact.hpp:15-37).
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>

namespace qllm::dump {

template <typename Digest>
std::string hex(const Digest& digest) {
  static constexpr char kDigits[] = "0123456789abcdef";
  std::string text;
  for (const auto byte : digest) {
    const auto value = static_cast<unsigned>(byte);
    text.push_back(kDigits[value >> 4U]);
    text.push_back(kDigits[value & 15U]);
  }
  return text;
}

class Lines final {
 public:
  template <typename... Fields>
  void add(const Fields&... fields) {
    bool first = true;
    ((append(fields, first)), ...);
    text_.push_back('\n');
  }
  [[nodiscard]] std::string take() { return std::move(text_); }

 private:
  void separator(bool& first) {
    if (!first) text_.push_back('\t');
    first = false;
  }
  void append(const std::string& field, bool& first) {
    separator(first);
    text_ += field;
  }
  void append(const char* field, bool& first) {
    separator(first);
    text_ += field;
  }
  void append(std::uint64_t field, bool& first) {
    separator(first);
    text_ += std::to_string(field);
  }
  void append(std::uint32_t field, bool& first) {
    separator(first);
    text_ += std::to_string(field);
  }
  std::string text_;
};

template <typename Descriptor>
std::string model_descriptor(const Descriptor& d) {
  Lines out;
  out.add("model", d.schema_version, d.architecture_id, d.vocab_size,
          d.max_context_tokens, d.hidden_size);
  out.add("content_hash", hex(d.content_hash));
  for (const auto& [key, value] : d.attributes) out.add("attribute", key, value);
  for (const auto& [role, tensor] : d.tensor_bindings)
    out.add("model_tensor", role, tensor);
  for (const auto& [role, endpoint] : d.program_inputs)
    out.add("program_input", role, endpoint.value, endpoint.abi);
  for (const auto& [role, endpoint] : d.program_outputs)
    out.add("program_output", role, endpoint.value, endpoint.abi);
  for (const auto& kernel : d.required_kernels)
    out.add("kernel", kernel.capability, kernel.abi_version);
  if (d.exact_decode_program) {
    const auto& decode = *d.exact_decode_program;
    out.add("exact_decode", decode.capability, decode.abi_version,
            decode.maximum_emitted_tokens);
    for (const auto& [key, value] : decode.parameters)
      out.add("exact_decode_parameter", key, value);
    for (const auto& [role, tensor] : decode.tensor_bindings)
      out.add("exact_decode_tensor", role, tensor);
  }
  for (const auto& c : d.routed_components) {
    out.add("component", c.name, c.namespace_id, c.layer_count,
            c.experts_per_layer, c.route_width, c.shared_experts_per_layer,
            c.hidden_size, c.intermediate_size, c.execution_capability,
            c.execution_abi, c.source_abi, c.encoding_abi, c.encoding);
    for (const auto& [key, value] : c.attributes)
      out.add("component_attribute", c.name, key, value);
    out.add("router", c.name, c.router.capability, c.router.abi_version);
    for (const auto& [key, value] : c.router.parameters)
      out.add("router_parameter", c.name, key, value);
  }
  for (const auto& layer : d.layer_program) {
    out.add("layer", layer.logical_layer, layer.block_capability,
            layer.block_abi_version,
            layer.routed_component.empty() ? std::string("-")
                                           : layer.routed_component,
            layer.component_layer);
    for (const auto& [key, value] : layer.parameters)
      out.add("layer_parameter", layer.logical_layer, key, value);
  }
  for (const auto& op : d.operation_program) {
    out.add("operation", op.logical_operation, op.logical_layer, op.capability,
            op.abi_version,
            op.routed_component.empty() ? std::string("-") : op.routed_component,
            op.component_layer);
    for (const auto& [key, value] : op.parameters)
      out.add("operation_parameter", op.logical_operation, key, value);
    for (const auto& [role, tensor] : op.tensor_bindings)
      out.add("operation_tensor", op.logical_operation, role, tensor);
    for (const auto& [port, binding] : op.input_bindings)
      out.add("operation_input", op.logical_operation, port, binding.value,
              binding.abi);
    for (const auto& [port, binding] : op.output_bindings)
      out.add("operation_output", op.logical_operation, port, binding.value,
              binding.abi);
  }
  return out.take();
}

// Packs and dense tensors of a loaded artifact, then its model descriptor.
template <typename Artifact>
std::string model_artifact(const Artifact& artifact) {
  Lines out;
  for (const auto& pack : artifact.packs())
    out.add("pack", pack.name, pack.kind, pack.bytes, hex(pack.sha256));
  for (const auto& tensor : artifact.dense_tensors()) {
    std::string shape;
    for (const auto dimension : tensor.shape) {
      if (!shape.empty()) shape.push_back('x');
      shape += std::to_string(dimension);
    }
    out.add("tensor", tensor.name, tensor.pack, tensor.record_offset,
            tensor.stored_bytes, tensor.encoding, tensor.quant_abi, shape,
            tensor.data_offset, tensor.data_bytes, tensor.scale_offset,
            tensor.scale_bytes, hex(tensor.payload_sha256));
  }
  return out.take() + model_descriptor(artifact.model());
}

}  // namespace qllm::dump
