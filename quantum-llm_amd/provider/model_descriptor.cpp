// Parser and validator of the artifact's model program.  Behaviour (what is
// accepted, what is rejected and with which message) follows
// runtime/src/model_descriptor.cpp:107-723 of the reference.
#include "expert/runtime/model_descriptor.hpp"
#include "expert/runtime/sha256.hpp"

#include <algorithm>
#include <charconv>
#include <fstream>
#include <set>

namespace expert::runtime {
namespace {

Status rejected(std::string message) {
  return {ErrorCode::invalid_argument, std::move(message)};
}

// An identifier inside a record: non-empty, free of field and line separators.
bool is_atom(std::string_view text) noexcept {
  return !text.empty() && text.find_first_of("\t\r\n") == std::string_view::npos;
}

bool to_u64(std::string_view text, std::uint64_t& value) noexcept {
  if (text.empty()) return false;
  const char* const end = text.data() + text.size();
  const auto [stop, error] = std::from_chars(text.data(), end, value);
  return error == std::errc{} && stop == end;
}

bool to_u32(std::string_view text, std::uint32_t& value) noexcept {
  std::uint64_t wide{};
  if (!to_u64(text, wide) || wide > std::numeric_limits<std::uint32_t>::max())
    return false;
  value = static_cast<std::uint32_t>(wide);
  return true;
}

template <typename Range, typename Match>
auto* first_match(Range& range, Match match) noexcept {
  const auto found = std::find_if(range.begin(), range.end(), match);
  return found == range.end() ? nullptr : &*found;
}

template <typename Map>
bool all_atoms(const Map& bindings) {
  return std::all_of(bindings.begin(), bindings.end(), [](const auto& item) {
    return is_atom(item.first) && is_atom(item.second);
  });
}

template <typename Map>
bool all_value_bindings_atoms(const Map& bindings) {
  return std::all_of(bindings.begin(), bindings.end(), [](const auto& item) {
    return is_atom(item.first) && is_atom(item.second.value) &&
           is_atom(item.second.abi);
  });
}

using RequirementSet = std::set<std::pair<std::string, std::uint32_t>>;

bool required(const RequirementSet& requirements, const std::string& capability,
              std::uint32_t abi) {
  return requirements.contains({capability, abi});
}

// ---- the checks of validate_model_descriptor, in the reference's order -----

Status check_exact_decode(const ModelDescriptor& d,
                          const RequirementSet& requirements) {
  if (!d.exact_decode_program) return Status::success();
  const auto& decode = *d.exact_decode_program;
  if (d.schema_version < 3U || !is_atom(decode.capability) ||
      decode.abi_version == 0U || decode.maximum_emitted_tokens < 2U ||
      !required(requirements, decode.capability, decode.abi_version))
    return rejected("exact decode program is invalid or unsupported");
  for (const auto& item : decode.parameters)
    if (!is_atom(item.first))
      return rejected("exact decode program parameter is invalid");
  if (!all_atoms(decode.tensor_bindings))
    return rejected("exact decode tensor binding is invalid");
  return Status::success();
}

Status check_component_kernels(const ModelDescriptor& d,
                               const RequirementSet& requirements) {
  for (const auto& component : d.routed_components) {
    if (!required(requirements, component.execution_capability,
                  component.execution_abi))
      return rejected("routed component lacks its execution kernel requirement");
    const auto& router = component.router;
    const bool has_router = !router.capability.empty();
    if ((d.schema_version >= 2U && !has_router) ||
        (has_router &&
         (router.abi_version == 0U ||
          !required(requirements, router.capability, router.abi_version))))
      return rejected("routed component lacks its routing kernel requirement");
  }
  return Status::success();
}

Status check_layers(const ModelDescriptor& d, const RequirementSet& requirements,
                    std::set<std::uint32_t>& logical_layers) {
  for (const auto& layer : d.layer_program) {
    if (layer.block_capability.empty() || layer.block_abi_version == 0U ||
        layer.logical_layer != logical_layers.size() ||
        !logical_layers.insert(layer.logical_layer).second ||
        !required(requirements, layer.block_capability, layer.block_abi_version))
      return rejected("layer program is invalid or lacks a kernel requirement");
    if (!layer.routed_component.empty()) {
      const auto* component = find_routed_component(d, layer.routed_component);
      if (!component || layer.component_layer >= component->layer_count)
        return rejected("layer program references an unavailable expert component");
    } else if (layer.component_layer != 0U) {
      return rejected("dense layer program has a routed component index");
    }
  }
  if (*logical_layers.begin() != 0U ||
      *logical_layers.rbegin() + 1ULL != logical_layers.size())
    return rejected("layer program logical indices are not contiguous");
  return Status::success();
}

Status check_operations(const ModelDescriptor& d,
                        const RequirementSet& requirements,
                        const std::set<std::uint32_t>& logical_layers) {
  std::set<std::uint32_t> seen_operations;
  std::set<std::uint32_t> covered_layers;
  std::uint32_t previous_layer{};
  bool any_layer_operation = false;
  for (const auto& operation : d.operation_program) {
    const bool model_level = operation.logical_layer == kModelLevelOperationLayer;
    if (operation.capability.empty() || operation.abi_version == 0U ||
        operation.logical_operation != seen_operations.size() ||
        !seen_operations.insert(operation.logical_operation).second ||
        (!model_level && !logical_layers.contains(operation.logical_layer)) ||
        (model_level && d.schema_version < 3U) ||
        (!model_level && any_layer_operation &&
         operation.logical_layer < previous_layer) ||
        !required(requirements, operation.capability, operation.abi_version))
      return rejected("operation program is invalid or unsupported");
    if (!all_atoms(operation.tensor_bindings))
      return rejected("operation tensor binding is invalid");
    if (!all_value_bindings_atoms(operation.input_bindings))
      return rejected("operation input binding is invalid");
    if (!all_value_bindings_atoms(operation.output_bindings))
      return rejected("operation output binding is invalid");
    if (!model_level) {
      previous_layer = operation.logical_layer;
      any_layer_operation = true;
      covered_layers.insert(operation.logical_layer);
    }
    if (!operation.routed_component.empty()) {
      if (model_level)
        return rejected("model-level operation references an expert component");
      const auto* component =
          find_routed_component(d, operation.routed_component);
      if (!component || operation.component_layer >= component->layer_count)
        return rejected(
            "operation program references an unavailable expert component");
    } else if (operation.component_layer != 0U) {
      return rejected("model-level operation has a component-local index");
    }
  }
  if (*seen_operations.begin() != 0U ||
      *seen_operations.rbegin() + 1ULL != seen_operations.size() ||
      covered_layers != logical_layers)
    return rejected("operation program indices or layer coverage are invalid");

  if (d.schema_version < 2U) return Status::success();
  // every routed layer names its router and its expert operation explicitly
  for (const auto& layer : d.layer_program) {
    if (layer.routed_component.empty()) continue;
    const auto* component = find_routed_component(d, layer.routed_component);
    const auto has_operation = [&](const std::string& capability,
                                   std::uint32_t abi) {
      return std::any_of(
          d.operation_program.begin(), d.operation_program.end(),
          [&](const OperationProgramDescriptor& operation) {
            return operation.logical_layer == layer.logical_layer &&
                   operation.routed_component == layer.routed_component &&
                   operation.component_layer == layer.component_layer &&
                   operation.capability == capability &&
                   operation.abi_version == abi;
          });
    };
    if (!component ||
        !has_operation(component->router.capability,
                       component->router.abi_version) ||
        !has_operation(component->execution_capability,
                       component->execution_abi))
      return rejected("routed layer lacks explicit router or expert operations");
  }
  return Status::success();
}

// Schema 3: every value has one producer and is produced before it is used.
Status check_data_flow(const ModelDescriptor& d) {
  if (d.program_inputs.empty() || d.program_outputs.empty())
    return rejected("schema v3 model descriptor lacks program endpoints");
  BindingMap value_abi;
  for (const auto& [role, endpoint] : d.program_inputs)
    if (!is_atom(role) || !is_atom(endpoint.value) || !is_atom(endpoint.abi) ||
        !value_abi.emplace(endpoint.value, endpoint.abi).second)
      return rejected("schema v3 program input is invalid or duplicated");
  for (const auto& operation : d.operation_program) {
    if (operation.input_bindings.empty() && operation.output_bindings.empty())
      return rejected("schema v3 operation lacks explicit data flow");
    for (const auto& item : operation.input_bindings) {
      const auto known = value_abi.find(item.second.value);
      if (known == value_abi.end() || known->second != item.second.abi)
        return rejected(
            "schema v3 operation input is unavailable or has the wrong ABI");
    }
    for (const auto& item : operation.output_bindings)
      if (!value_abi.emplace(item.second.value, item.second.abi).second)
        return rejected("schema v3 operation output has multiple producers");
  }
  for (const auto& [role, endpoint] : d.program_outputs) {
    const auto known = value_abi.find(endpoint.value);
    if (!is_atom(role) || !is_atom(endpoint.value) || !is_atom(endpoint.abi) ||
        known == value_abi.end() || known->second != endpoint.abi)
      return rejected("schema v3 program output is unavailable or invalid");
  }
  return Status::success();
}

// ---- the line parser --------------------------------------------------------

struct Record {
  std::vector<std::string_view> fields;
  [[nodiscard]] std::size_t size() const noexcept { return fields.size(); }
  [[nodiscard]] std::string_view operator[](std::size_t index) const noexcept {
    return fields[index];
  }
  [[nodiscard]] std::string text(std::size_t index) const {
    return std::string(fields[index]);
  }
};

Record split_record(std::string_view line) {
  Record record;
  for (;;) {
    const auto tab = line.find('\t');
    record.fields.push_back(line.substr(0U, tab));
    if (tab == std::string_view::npos) return record;
    line.remove_prefix(tab + 1U);
  }
}

// Builds the descriptor one record at a time; every handler returns false for
// a record that the format does not allow at this point.
class ProgramReader final {
 public:
  ProgramReader(ModelDescriptor& descriptor, std::uint64_t namespace_base)
      : d_(descriptor), namespace_base_(namespace_base) {}

  [[nodiscard]] bool model_seen() const noexcept { return model_; }

  bool accept(const Record& r) {
    const std::string_view kind = r[0];
    if (kind == "model") return model(r);
    if (kind == "attribute")
      return model_ && r.size() == 3U && put_number(d_.attributes, r[1], r[2]);
    if (kind == "model_tensor")
      return model_ && r.size() == 3U && put_text(d_.tensor_bindings, r[1], r[2]);
    if (kind == "program_input" || kind == "program_output")
      return endpoint(r, kind == "program_input" ? d_.program_inputs
                                                 : d_.program_outputs);
    if (kind == "kernel") return kernel(r);
    if (kind == "exact_decode") return exact_decode(r);
    if (kind == "exact_decode_parameter")
      return d_.exact_decode_program && r.size() == 3U &&
             put_number(d_.exact_decode_program->parameters, r[1], r[2]);
    if (kind == "exact_decode_tensor")
      return d_.exact_decode_program && r.size() == 3U &&
             put_text(d_.exact_decode_program->tensor_bindings, r[1], r[2]);
    if (kind == "component") return component(r);
    if (kind == "component_attribute") {
      auto* item = component_of(r);
      return item && put_number(item->attributes, r[2], r[3]);
    }
    if (kind == "router") {
      auto* item = component_of(r);
      if (!item || !is_atom(r[2]) || !item->router.capability.empty() ||
          !to_u32(r[3], item->router.abi_version))
        return false;
      item->router.capability = r.text(2);
      return true;
    }
    if (kind == "router_parameter") {
      auto* item = component_of(r);
      return item && !item->router.capability.empty() &&
             put_number(item->router.parameters, r[2], r[3]);
    }
    if (kind == "layer") return layer(r);
    if (kind == "layer_parameter") {
      std::uint32_t index{};
      auto* item = r.size() == 4U && to_u32(r[1], index)
                       ? first_match(d_.layer_program,
                                     [index](const auto& layer) {
                                       return layer.logical_layer == index;
                                     })
                       : nullptr;
      return item && put_number(item->parameters, r[2], r[3]);
    }
    if (kind == "operation") return operation(r);
    if (kind == "operation_parameter") {
      auto* item = operation_of(r, 4U);
      return item && put_number(item->parameters, r[2], r[3]);
    }
    if (kind == "operation_tensor") {
      auto* item = operation_of(r, 4U);
      return item && put_text(item->tensor_bindings, r[2], r[3]);
    }
    if (kind == "operation_input" || kind == "operation_output") {
      auto* item = operation_of(r, 5U);
      if (!item || !is_atom(r[2]) || !is_atom(r[3]) || !is_atom(r[4]))
        return false;
      auto& bindings = kind == "operation_input" ? item->input_bindings
                                                 : item->output_bindings;
      return bindings.emplace(r.text(2), OperationProgramDescriptor::ValueBinding{
                                             r.text(3), r.text(4)})
          .second;
    }
    return false;
  }

 private:
  static bool put_number(ParameterMap& map, std::string_view key,
                         std::string_view number) {
    std::uint64_t value{};
    return is_atom(key) && to_u64(number, value) &&
           map.emplace(std::string(key), value).second;
  }
  static bool put_text(BindingMap& map, std::string_view key,
                       std::string_view value) {
    return is_atom(key) && is_atom(value) &&
           map.emplace(std::string(key), std::string(value)).second;
  }

  bool model(const Record& r) {
    if (model_ || r.size() != 6U || !is_atom(r[2]) ||
        !to_u32(r[1], d_.schema_version) || !to_u32(r[3], d_.vocab_size) ||
        !to_u32(r[4], d_.max_context_tokens) || !to_u32(r[5], d_.hidden_size))
      return false;
    d_.architecture_id = r.text(2);
    model_ = true;
    return true;
  }

  bool endpoint(const Record& r,
                std::map<std::string, ProgramEndpointDescriptor, std::less<>>&
                    endpoints) {
    return model_ && r.size() == 4U && is_atom(r[1]) && is_atom(r[2]) &&
           is_atom(r[3]) &&
           endpoints
               .emplace(r.text(1), ProgramEndpointDescriptor{r.text(2), r.text(3)})
               .second;
  }

  bool kernel(const Record& r) {
    KernelRequirement item;
    if (!model_ || r.size() != 3U || !is_atom(r[1]) ||
        !to_u32(r[2], item.abi_version))
      return false;
    item.capability = r.text(1);
    d_.required_kernels.push_back(std::move(item));
    return true;
  }

  bool exact_decode(const Record& r) {
    ExactDecodeProgramDescriptor item;
    if (!model_ || d_.exact_decode_program || r.size() != 4U || !is_atom(r[1]) ||
        !to_u32(r[2], item.abi_version) ||
        !to_u32(r[3], item.maximum_emitted_tokens))
      return false;
    item.capability = r.text(1);
    d_.exact_decode_program = std::move(item);
    return true;
  }

  bool component(const Record& r) {
    RoutedExpertComponentDescriptor item;
    std::uint64_t offset{};
    if (!model_ || r.size() != 14U || !is_atom(r[1]) || !is_atom(r[9]) ||
        !is_atom(r[13]) || !to_u64(r[2], offset) ||
        offset > std::numeric_limits<std::uint64_t>::max() - namespace_base_ ||
        !to_u32(r[3], item.layer_count) ||
        !to_u32(r[4], item.experts_per_layer) ||
        !to_u32(r[5], item.route_width) ||
        !to_u32(r[6], item.shared_experts_per_layer) ||
        !to_u32(r[7], item.hidden_size) ||
        !to_u32(r[8], item.intermediate_size) ||
        !to_u32(r[10], item.execution_abi) || !to_u32(r[11], item.source_abi) ||
        !to_u32(r[12], item.encoding_abi))
      return false;
    item.name = r.text(1);
    item.namespace_id = namespace_base_ + offset;
    item.execution_capability = r.text(9);
    item.encoding = r.text(13);
    d_.routed_components.push_back(std::move(item));
    return true;
  }

  RoutedExpertComponentDescriptor* component_of(const Record& r) {
    if (r.size() != 4U) return nullptr;
    return first_match(d_.routed_components, [&](const auto& item) {
      return item.name == r[1];
    });
  }

  bool layer(const Record& r) {
    LayerProgramDescriptor item;
    if (!model_ || r.size() != 6U || !is_atom(r[2]) ||
        !to_u32(r[1], item.logical_layer) ||
        !to_u32(r[3], item.block_abi_version) ||
        !to_u32(r[5], item.component_layer))
      return false;
    item.block_capability = r.text(2);
    if (r[4] != "-") {
      if (!is_atom(r[4])) return false;
      item.routed_component = r.text(4);
    }
    d_.layer_program.push_back(std::move(item));
    return true;
  }

  bool operation(const Record& r) {
    OperationProgramDescriptor item;
    if (!model_ || r.size() != 7U || !is_atom(r[3]) ||
        !to_u32(r[1], item.logical_operation) ||
        (r[2] != "-" && !to_u32(r[2], item.logical_layer)) ||
        !to_u32(r[4], item.abi_version) || !to_u32(r[6], item.component_layer))
      return false;
    if (r[2] == "-") item.logical_layer = kModelLevelOperationLayer;
    item.capability = r.text(3);
    if (r[5] != "-") {
      if (!is_atom(r[5])) return false;
      item.routed_component = r.text(5);
    }
    d_.operation_program.push_back(std::move(item));
    return true;
  }

  OperationProgramDescriptor* operation_of(const Record& r, std::size_t fields) {
    std::uint32_t index{};
    if (r.size() != fields || !to_u32(r[1], index)) return nullptr;
    return first_match(d_.operation_program, [index](const auto& item) {
      return item.logical_operation == index;
    });
  }

  ModelDescriptor& d_;
  std::uint64_t namespace_base_;
  bool model_{false};
};

}  // namespace

std::uint64_t expert_table_entries(
    const RoutedExpertComponentDescriptor& component) noexcept {
  return std::uint64_t{component.layer_count} * component.experts_per_layer;
}

const RoutedExpertComponentDescriptor* find_routed_component(
    const ModelDescriptor& descriptor, std::string_view name) noexcept {
  return first_match(descriptor.routed_components,
                     [name](const auto& item) { return item.name == name; });
}

// The first eight digest bytes, little endian; never zero (:98-107).
std::uint64_t namespace_id_from_content_hash(const Sha256Digest& digest) noexcept {
  std::uint64_t value{};
  for (std::size_t index = 0; index < 8U; ++index)
    value |= std::uint64_t{std::to_integer<std::uint8_t>(digest[index])}
             << (8U * index);
  return value ? value : 1U;
}

Status validate_routed_component(const RoutedExpertComponentDescriptor& item,
                                 std::uint32_t model_hidden_size) noexcept {
  if (item.name.empty() || item.namespace_id == 0U || item.layer_count == 0U ||
      item.experts_per_layer == 0U || item.route_width == 0U ||
      item.route_width > item.experts_per_layer || item.hidden_size == 0U ||
      item.intermediate_size == 0U || item.source_abi == 0U ||
      item.encoding_abi == 0U || item.execution_capability.empty() ||
      item.execution_abi == 0U || item.encoding.empty() ||
      item.hidden_size != model_hidden_size)
    return rejected("routed expert component geometry or identity is invalid");
  if (expert_table_entries(item) >
      std::numeric_limits<std::size_t>::max() / 128U)
    return rejected("routed expert table exceeds addressable metadata");
  return Status::success();
}

Status validate_model_descriptor(const ModelDescriptor& d) noexcept {
  try {
    if ((d.schema_version != 1U && d.schema_version != 2U &&
         d.schema_version != 3U) ||
        d.architecture_id.empty() || d.vocab_size == 0U ||
        d.max_context_tokens == 0U || d.hidden_size == 0U ||
        d.layer_program.empty() || d.required_kernels.empty())
      return rejected("model descriptor architecture is incomplete");
    if (!all_atoms(d.tensor_bindings))
      return rejected("model tensor binding is invalid");

    std::set<std::string, std::less<>> names;
    std::set<std::uint64_t> namespaces;
    for (const auto& component : d.routed_components) {
      auto status = validate_routed_component(component, d.hidden_size);
      if (!status.ok()) return status;
      if (!names.insert(component.name).second ||
          !namespaces.insert(component.namespace_id).second)
        return rejected("routed expert component geometry or identity is invalid");
    }

    RequirementSet requirements;
    for (const auto& kernel : d.required_kernels)
      if (kernel.capability.empty() || kernel.abi_version == 0U ||
          !requirements.emplace(kernel.capability, kernel.abi_version).second)
        return rejected("kernel requirement is invalid or duplicated");

    if (auto status = check_exact_decode(d, requirements); !status.ok())
      return status;
    if (auto status = check_component_kernels(d, requirements); !status.ok())
      return status;
    std::set<std::uint32_t> logical_layers;
    if (auto status = check_layers(d, requirements, logical_layers); !status.ok())
      return status;

    if (d.schema_version >= 2U && d.operation_program.empty())
      return rejected("schema v2 model descriptor lacks its operation program");
    if (!d.operation_program.empty())
      if (auto status = check_operations(d, requirements, logical_layers);
          !status.ok())
        return status;

    if (d.schema_version < 3U) {
      const bool has_flow =
          !d.program_inputs.empty() || !d.program_outputs.empty() ||
          d.exact_decode_program ||
          std::any_of(d.operation_program.begin(), d.operation_program.end(),
                      [](const OperationProgramDescriptor& operation) {
                        return !operation.input_bindings.empty() ||
                               !operation.output_bindings.empty();
                      });
      return has_flow
                 ? rejected("legacy model descriptor contains schema v3 data flow")
                 : Status::success();
    }
    return check_data_flow(d);
  } catch (const std::exception& error) {
    return {ErrorCode::internal,
            std::string("model descriptor validation failed: ") + error.what()};
  }
}

Status provider_supports_model(
    const ModelDescriptor& descriptor,
    std::span<const KernelCapability> capabilities) noexcept {
  try {
    if (auto status = validate_model_descriptor(descriptor); !status.ok())
      return status;
    for (const auto& kernel : descriptor.required_kernels) {
      const auto* available = first_match(capabilities, [&](const auto& item) {
        return item.capability == kernel.capability &&
               kernel.abi_version >= item.minimum_abi &&
               kernel.abi_version <= item.maximum_abi;
      });
      if (!available)
        return rejected("execution provider lacks required kernel capability: " +
                        kernel.capability);
      if (available->validate)
        if (auto status = available->validate(descriptor); !status.ok())
          return status;
    }
    return Status::success();
  } catch (const std::exception& error) {
    return {ErrorCode::internal,
            std::string("execution provider validation failed: ") + error.what()};
  }
}

// Names resolved to indices once (runtime/src/model_descriptor.cpp:374-490):
// kernel binding k stands for required kernel k and the position of the first
// capability that serves it; layers and operations refer to their kernel
// binding and component by index; under schema 3 every SSA value gets a slot -
// program inputs first (in role order), then each operation's outputs in
// program order - and ports refer to slots.
CompileModelProgramResult compile_model_program(
    const ModelDescriptor& descriptor,
    std::span<const KernelCapability> capabilities) noexcept {
  if (auto supported = provider_supports_model(descriptor, capabilities);
      !supported.ok())
    return {std::move(supported), {}};
  try {
    CompiledModelProgram program;
    const auto binding_of = [&](const std::string& capability,
                                std::uint32_t abi) -> std::uint32_t {
      for (std::uint32_t k = 0; k < descriptor.required_kernels.size(); ++k)
        if (descriptor.required_kernels[k].capability == capability &&
            descriptor.required_kernels[k].abi_version == abi)
          return k;
      throw std::out_of_range("kernel requirement is not declared");
    };
    const auto component_of =
        [&](const std::string& name) -> std::optional<std::uint32_t> {
      if (name.empty()) return std::nullopt;
      for (std::uint32_t c = 0; c < descriptor.routed_components.size(); ++c)
        if (descriptor.routed_components[c].name == name) return c;
      throw std::out_of_range("routed component is not declared");
    };
    for (std::uint32_t k = 0; k < descriptor.required_kernels.size(); ++k) {
      const auto& required = descriptor.required_kernels[k];
      std::uint32_t offered = 0;
      while (offered < capabilities.size() &&
             !(capabilities[offered].capability == required.capability &&
               required.abi_version >= capabilities[offered].minimum_abi &&
               required.abi_version <= capabilities[offered].maximum_abi))
        ++offered;
      program.kernels.push_back({k, 0U, offered});
    }
    for (const auto& layer : descriptor.layer_program)
      program.layers.push_back(
          {layer.logical_layer,
           binding_of(layer.block_capability, layer.block_abi_version),
           component_of(layer.routed_component), layer.component_layer,
           layer.parameters});
    if (descriptor.operation_program.empty()) {
      // schema 1: one block per layer stands for the operation program
      for (const auto& layer : descriptor.layer_program)
        program.operations.push_back(
            {static_cast<std::uint32_t>(program.operations.size()),
             layer.logical_layer,
             binding_of(layer.block_capability, layer.block_abi_version),
             component_of(layer.routed_component), layer.component_layer,
             layer.parameters, {}, {}, {}});
    } else {
      for (const auto& operation : descriptor.operation_program)
        program.operations.push_back(
            {operation.logical_operation, operation.logical_layer,
             binding_of(operation.capability, operation.abi_version),
             component_of(operation.routed_component), operation.component_layer,
             operation.parameters, operation.tensor_bindings, {}, {}});
    }
    if (descriptor.schema_version >= 3U) {
      std::map<std::string, std::uint32_t, std::less<>> slots;
      const auto new_slot = [&](const std::string& name, const std::string& abi) {
        const auto slot = static_cast<std::uint32_t>(program.values.size());
        program.values.push_back({name, abi});
        slots.emplace(name, slot);
        return slot;
      };
      for (const auto& [role, endpoint] : descriptor.program_inputs)
        program.inputs.push_back({role, new_slot(endpoint.value, endpoint.abi)});
      for (std::size_t index = 0; index < descriptor.operation_program.size();
           ++index) {
        const auto& source = descriptor.operation_program[index];
        auto& compiled = program.operations[index];
        for (const auto& [port, bound] : source.input_bindings)
          compiled.input_values.push_back({port, slots.at(bound.value)});
        for (const auto& [port, bound] : source.output_bindings)
          compiled.output_values.push_back(
              {port, new_slot(bound.value, bound.abi)});
      }
      for (const auto& [role, endpoint] : descriptor.program_outputs)
        program.outputs.push_back({role, slots.at(endpoint.value)});
    }
    if (descriptor.exact_decode_program) {
      const auto& decode = *descriptor.exact_decode_program;
      program.exact_decode = CompiledExactDecodeProgram{
          binding_of(decode.capability, decode.abi_version),
          decode.maximum_emitted_tokens, decode.parameters,
          decode.tensor_bindings};
    }
    return {Status::success(), std::move(program)};
  } catch (const std::exception& error) {
    return {{ErrorCode::internal,
             std::string("model program compilation failed: ") + error.what()},
            {}};
  }
}

ParseModelDescriptorResult parse_model_descriptor_artifact(
    std::string_view text, const Sha256Digest& content_hash,
    std::uint64_t namespace_base) noexcept {
  try {
    if (namespace_base == 0U)
      return {rejected("model descriptor namespace base is zero"), {}};
    ModelDescriptor descriptor;
    descriptor.content_hash = content_hash;
    ProgramReader reader(descriptor, namespace_base);
    bool header_seen = false;
    std::size_t line_number = 0;
    while (!text.empty()) {
      ++line_number;
      const auto newline = text.find('\n');
      std::string_view line = text.substr(0U, newline);
      text = newline == std::string_view::npos ? std::string_view{}
                                               : text.substr(newline + 1U);
      if (!line.empty() && line.back() == '\r') line.remove_suffix(1U);
      if (line.empty()) continue;
      if (!header_seen) {
        if (line != "expert-runtime-model-v1")
          return {rejected("unknown model descriptor artifact header"), {}};
        header_seen = true;
        continue;
      }
      if (!reader.accept(split_record(line)))
        return {rejected("malformed model descriptor line " +
                         std::to_string(line_number)),
                {}};
    }
    if (!header_seen || !reader.model_seen())
      return {rejected("model descriptor artifact is incomplete"), {}};
    if (auto status = validate_model_descriptor(descriptor); !status.ok())
      return {std::move(status), {}};
    return {Status::success(), std::move(descriptor)};
  } catch (const std::exception& error) {
    return {{ErrorCode::internal,
             std::string("model descriptor parsing failed: ") + error.what()},
            {}};
  }
}

ParseModelDescriptorResult load_model_descriptor_artifact(
    const std::filesystem::path& path, std::uint64_t expected_bytes,
    const Sha256Digest& expected_sha256, const Sha256Digest& content_hash,
    std::uint64_t namespace_base) noexcept {
  try {
    constexpr std::uint64_t kMaximumProgramBytes = 64ULL << 20U;
    if (expected_bytes == 0U || expected_bytes > kMaximumProgramBytes ||
        !std::filesystem::is_regular_file(path) ||
        std::filesystem::file_size(path) != expected_bytes)
      return {rejected("model descriptor artifact size is invalid"), {}};
    std::string bytes(static_cast<std::size_t>(expected_bytes), '\0');
    std::ifstream input(path, std::ios::binary);
    if (!input ||
        !input.read(bytes.data(), static_cast<std::streamsize>(bytes.size())) ||
        input.peek() != std::ifstream::traits_type::eof())
      return {rejected("model descriptor artifact read failed"), {}};
    const auto digest = sha256(std::as_bytes(std::span(bytes.data(), bytes.size())));
    if (digest != expected_sha256)
      return {rejected("model descriptor artifact checksum mismatch"), {}};
    return parse_model_descriptor_artifact(bytes, content_hash, namespace_base);
  } catch (const std::exception& error) {
    return {{ErrorCode::internal,
             std::string("model descriptor loading failed: ") + error.what()},
            {}};
  }
}

}  // namespace expert::runtime
