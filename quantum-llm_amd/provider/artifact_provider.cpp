#include "artifact_provider.hpp"

#include "dense_record.hpp"

#include <algorithm>
#include <bit>
#include <cmath>
#include <map>
#include <stdexcept>

namespace qllm {
namespace {

std::uint64_t attribute(const er::ModelDescriptor& model, std::string_view name) {
  const auto found = model.attributes.find(name);
  return found == model.attributes.end() ? 0U : found->second;
}

float attribute_f32(const er::ModelDescriptor& model, std::string_view name) {
  const auto found = model.attributes.find(name);
  if (found == model.attributes.end() ||
      found->second > std::numeric_limits<std::uint32_t>::max())
    throw std::runtime_error("artifact lacks the float attribute " +
                             std::string(name));
  const float value = std::bit_cast<float>(static_cast<std::uint32_t>(found->second));
  if (!std::isfinite(value) || !(value > 0.0F))
    throw std::runtime_error("artifact float attribute is not finite and positive: " +
                             std::string(name));
  return value;
}

bool is_full_attention(std::string_view capability) {
  return capability == "block.full-attention.output-gated.v1" ||
         capability == "block.full-attention.standard-gqa.v1";
}

bool is_ffn(std::string_view capability) {
  return capability.starts_with("ffn.swiglu.dense.");
}

er::Status invalid(std::string message) {
  return {er::ErrorCode::invalid_argument, std::move(message)};
}

// Resolves the tensors an operation names, once per tensor name.
class TensorBinder final {
 public:
  explicit TensorBinder(er::IModelTensorStore& store) : store_(store) {}

  er::Status bind(
      const std::map<std::string, std::string, std::less<>>& bindings,
                  std::vector<er::PreparedTensorBinding>& out, const char* what) {
    out.clear();
    out.reserve(bindings.size());
    for (const auto& [role, name] : bindings) {
      auto retained = cache_.find(name);
      if (retained == cache_.end()) {
        auto resolved = store_.resolve(name);
        if (!resolved.status.ok()) return resolved.status;
        if (!resolved.tensor || resolved.tensor->name != name ||
            resolved.tensor->encoding.empty() || resolved.tensor->shape.empty() ||
            !resolved.tensor->value.valid())
          return invalid(std::string("artifact tensor store returned an invalid ") +
                         what);
        retained = cache_.emplace(name, std::move(resolved.tensor)).first;
      }
      out.push_back({role, retained->second});
    }
    return er::Status::success();
  }

 private:
  er::IModelTensorStore& store_;
  std::map<std::string, std::shared_ptr<const er::ImmutableModelTensor>, std::less<>>
      cache_;
};

}  // namespace

er::Status validate_dense_fp4_descriptor(const er::ModelDescriptor& model) {
  if (model.schema_version < 3U || !model.routed_components.empty() ||
      model.operation_program.empty() || !model.hidden_size ||
      !model.vocab_size || !model.max_context_tokens)
    return invalid("FP4 provider requires a schema-v3 program");
  const auto query_heads = attribute(model, "attention_heads");
  const auto kv_heads = attribute(model, "kv_heads");
  const auto head_dim = attribute(model, "head_dim");
  const auto rotary = attribute(model, "rotary_dimension");
  const auto mtp = attribute(model, "mtp_layers");
  if (!query_heads || !kv_heads || query_heads % kv_heads ||
      attribute(model, "activation_bf16") > 1U ||
      attribute(model, "dense_activation_input_bf16") > 1U ||
      query_heads / kv_heads > 16U || !head_dim || head_dim > 256U ||
      head_dim % 32U || !rotary || rotary > head_dim || rotary % 2U ||
      (model.exact_decode_program.has_value() && mtp != 1U))
    return invalid("dense FP4 descriptor geometry is not supported");
  for (const auto& layer : model.layer_program)
    if (!is_full_attention(layer.block_capability))
      return invalid("dense FP4 provider executes full-attention layers only: " +
                     layer.block_capability);
  return er::Status::success();
}

er::Status dense_geometry_from_artifact(const er::ModelDescriptor& model,
                                        er::IModelTensorStore& tensors,
                                        const ArtifactProviderOptions& options,
                                        DenseGeometry& g) {
  try {
    if (auto status = validate_dense_fp4_descriptor(model); !status.ok())
      return status;
    g = DenseGeometry{};
    g.hidden = model.hidden_size;
    g.vocabulary = model.vocab_size;
    g.layers = static_cast<std::uint32_t>(model.layer_program.size());
    g.query_heads = static_cast<std::uint32_t>(attribute(model, "attention_heads"));
    g.kv_heads = static_cast<std::uint32_t>(attribute(model, "kv_heads"));
    g.head_dim = static_cast<std::uint32_t>(attribute(model, "head_dim"));
    g.rotary_dim = static_cast<std::uint32_t>(attribute(model, "rotary_dimension"));
    g.norm_epsilon = attribute_f32(model, "norm_epsilon_f32_bits");
    g.rope_theta = attribute_f32(model, "rope_theta_f32_bits");
    g.zero_centered_norm = attribute(model, "zero_centered_norm") == 1U;
    g.max_context = options.max_context ? options.max_context
                                        : model.max_context_tokens;
    if (g.max_context > model.max_context_tokens)
      return invalid("requested context exceeds the artifact's maximum");
    g.kv_page_tokens = options.kv_page_tokens;
    g.capacity = std::max(1U, options.capacity);
    g.profile_gpu_phases = options.profile_gpu_phases;
    if (options.kv_cache_dtype == "artifact" ||
        options.kv_cache_dtype == "q4-f16-per-head")
      g.kv_encoding = KvEncoding::q4_f16_per_head;
    else if (options.kv_cache_dtype == "fp16")
      g.kv_encoding = KvEncoding::fp16;
    else
      return invalid("unsupported KV cache dtype: " + options.kv_cache_dtype);

    bool attention_seen = false;
    bool ffn_seen = false;
    for (const auto& operation : model.operation_program) {
      if (is_full_attention(operation.capability)) {
        const bool gated = operation.capability.find("output-gated") !=
                           std::string::npos;
        const bool normed = operation.tensor_bindings.contains("query_norm") &&
                            operation.tensor_bindings.contains("key_norm");
        if (attention_seen && (gated != g.output_gated || normed != g.qk_norm))
          return invalid("attention layout changes between layers");
        g.output_gated = gated;
        g.qk_norm = normed;
        attention_seen = true;
      } else if (is_ffn(operation.capability)) {
        const auto gate = operation.tensor_bindings.find("gate_projection");
        if (gate == operation.tensor_bindings.end())
          return invalid("dense FFN operation names no gate projection");
        const auto resolved = tensors.resolve(gate->second);
        if (!resolved.status.ok()) return resolved.status;
        if (!resolved.tensor || resolved.tensor->shape.size() != 2U ||
            resolved.tensor->shape[1] != g.hidden)
          return invalid("dense FFN gate/up geometry is invalid");
        if (ffn_seen && g.intermediate != resolved.tensor->shape[0])
          return invalid("dense FFN width changes between layers");
        g.intermediate = resolved.tensor->shape[0];
        g.scale_scheme = operation.capability.find("fp4-f16-block16") !=
                                 std::string::npos
                             ? QLLM_SCALE_F16_BLOCK16
                             : QLLM_SCALE_UE8M0_BLOCK32;
        ffn_seen = true;
      }
    }
    if (!attention_seen || !ffn_seen)
      return invalid("program has no dense attention or FFN operation");

    // The activation contract (compiler/expert_pack/compile.py:256-279): an
    // artifact takes bf16 activation input only when it says so; the default
    // is per-row Q8, which exists for block-32 UE8M0 weights.
    g.activation_q8 = attribute(model, "dense_activation_input_bf16") != 1U &&
                      g.scale_scheme == QLLM_SCALE_UE8M0_BLOCK32;

    g.mtp_layers = 0U;
    g.draft_depth = 4U;
    if (model.exact_decode_program) {
      const auto& decode = *model.exact_decode_program;
      const auto depth = decode.parameters.find("draft_depth");
      if (depth == decode.parameters.end() || depth->second == 0U ||
          depth->second + 1U != decode.maximum_emitted_tokens)
        return invalid("exact decode program declares no usable draft depth");
      g.draft_depth = static_cast<std::uint32_t>(depth->second);
      g.mtp_layers = static_cast<std::uint32_t>(attribute(model, "mtp_layers"));
      const auto vocabulary = decode.parameters.find("draft_vocabulary_size");
      g.draft_vocabulary = vocabulary == decode.parameters.end()
                               ? 0U
                               : static_cast<std::uint32_t>(vocabulary->second);
    }
    return er::Status::success();
  } catch (const std::exception& error) {
    return invalid(error.what());
  }
}

er::CreateExecutionProviderModuleResult make_mi355_dense_fp4_module(
    std::shared_ptr<er::ModelArtifact> artifact,
    const ArtifactProviderOptions& options) {
  try {
    if (!artifact) return {invalid("artifact is absent"), {}};
    if (options.routed_vram_policy != "fixed")
      return {invalid("a dense resident provider has no routed VRAM policy but "
                      "\"fixed\""),
              {}};
    auto store = std::make_shared<er::MappedModelTensorStore>();
    if (auto status = er::MappedModelTensorStore::create(*artifact, *store);
        !status.ok())
      return {status, {}};
    // every record header must agree with its index entry
    for (const auto& entry : artifact->dense_tensors()) {
      const auto resolved = store->resolve(entry.name);
      if (!resolved.status.ok()) return {resolved.status, {}};
      if (auto status = er::validate_dense_record(entry, resolved.tensor->value.data,
                                                  resolved.tensor->value.bytes);
          !status.ok())
        return {status, {}};
    }

    const er::ModelDescriptor& model = artifact->model();
    auto metadata = make_mi355_dense_fp4_provider();
    if (auto status = er::provider_supports_model(model, metadata.capabilities);
        !status.ok())
      return {status, {}};
    DenseGeometry geometry;
    if (auto status = dense_geometry_from_artifact(model, *store, options, geometry);
        !status.ok())
      return {status, {}};

    auto implementation = std::make_shared<Mi355DenseFp4Provider>(geometry);
    er::ExecutionProviderModule module;
    module.definition = {metadata.name, metadata.priority,
                         std::move(metadata.capabilities), implementation};
    module.tensor_store = std::move(store);
    module.service = implementation->service_contract();
    const bool mtp = model.exact_decode_program.has_value();
    module.service.mtp_resource_available = mtp;
    module.service.mtp_runtime_ready = mtp;
    module.service.mtp_enabled = mtp;
    module.service.vram_cache_bytes = options.vram_cache_bytes;
    module.service.routed_vram_policy = options.routed_vram_policy;
    module.telemetry = [implementation] { return implementation->telemetry(); };
    // nothing to fit after the tensors are bound: weights and workspaces are
    // resident, KV pages are allocated on demand
    module.finalize_service =
        [](er::ExecutionProviderModule::ServiceContract&) {
          return er::Status::success();
        };
    return {er::Status::success(), std::move(module)};
  } catch (const std::exception& error) {
    return {{er::ErrorCode::internal,
             std::string("dense FP4 provider creation failed: ") + error.what()},
            {}};
  }
}

er::CreateExecutionProviderModuleResult make_mi355_dense_fp4_callable_provider(
    const std::filesystem::path& artifact_root, std::uint32_t max_context,
    std::uint32_t capacity, std::uint64_t /*ram_cache_bytes*/,
    std::uint64_t vram_cache_bytes, std::uint64_t kv_cache_bytes,
    std::uint32_t kv_page_tokens, std::string_view kv_cache_dtype,
    std::string_view /*placement_profile*/, std::string_view routed_vram_policy,
    bool profile_gpu_phases, bool /*discover_active_expert_devices*/,
    std::vector<int> /*active_expert_devices*/,
    std::uint64_t /*active_expert_device_cache_bytes*/,
    std::uint64_t /*active_expert_host_cache_bytes*/,
    std::uint32_t mtp_draft_depth) {
  try {
    // the launch contract of dense_fp4_provider.cpp:2330-2336
    if (!capacity || !max_context || !kv_cache_bytes || !kv_page_tokens)
      return {invalid("invalid dense FP4 provider launch contract"), {}};
    auto artifact = std::make_shared<er::ModelArtifact>();
    if (auto status = er::ModelArtifact::load(artifact_root, *artifact); !status.ok())
      return {status, {}};
    if (mtp_draft_depth != 0U)
      if (auto status = artifact->configure_mtp_draft_depth(mtp_draft_depth);
          !status.ok())
        return {status, {}};
    ArtifactProviderOptions options;
    options.max_context = max_context;
    options.kv_page_tokens = kv_page_tokens;
    options.kv_cache_dtype = std::string(kv_cache_dtype);
    options.vram_cache_bytes = vram_cache_bytes ? vram_cache_bytes : 1U;
    options.routed_vram_policy = std::string(routed_vram_policy);
    options.capacity = capacity;
    options.profile_gpu_phases = profile_gpu_phases;
    return make_mi355_dense_fp4_module(std::move(artifact), options);
  } catch (const std::exception& error) {
    return {{er::ErrorCode::internal, error.what()}, {}};
  }
}

er::Status prepare_program(const er::ModelDescriptor& model,
                           const er::ExecutionProviderModule& module,
                           PreparedProgram& prepared) {
  try {
    if (!module.definition.implementation || !module.tensor_store)
      return invalid("provider module is incomplete");
    er::ExecutionProviderRegistry registry;
    if (auto status = registry.add(module.definition); !status.ok()) return status;
    auto bound = registry.bind(model, er::ExecutionProviderBindingMode::executable);
    if (!bound.status.ok()) return bound.status;
    prepared = PreparedProgram{};
    prepared.bound = std::move(bound.provider);
    const auto& program = prepared.bound.program;
    auto& provider = *module.definition.implementation;
    if (program.operations.size() != model.operation_program.size())
      return invalid("compiled operation order or kernel binding is invalid");
    TensorBinder binder(*module.tensor_store);
    std::vector<er::PreparedTensorBinding> tensors;
    for (std::size_t index = 0; index < model.operation_program.size(); ++index) {
      const auto& operation = model.operation_program[index];
      const auto& compiled = program.operations[index];
      if (compiled.logical_operation != index ||
          compiled.kernel_binding >= program.kernels.size())
        return invalid("compiled operation order or kernel binding is invalid");
      if (auto status = binder.bind(operation.tensor_bindings, tensors, "tensor");
          !status.ok())
        return status;
      auto result = provider.prepare({model, operation, compiled, tensors});
      if (!result.status.ok()) return result.status;
      if (!result.operation)
        return invalid("callable provider returned no prepared operation");
      prepared.operations.push_back(std::move(result.operation));
    }
    if (model.exact_decode_program) {
      if (!program.exact_decode)
        return invalid("exact decode program was not compiled");
      const auto& decode = *model.exact_decode_program;
      if (auto status =
              binder.bind(decode.tensor_bindings, tensors, "exact decode tensor");
          !status.ok())
        return status;
      auto result = provider.prepare_exact_decode(
          {model, decode, *program.exact_decode, tensors});
      if (!result.status.ok()) return result.status;
      if (!result.operation)
        return invalid("callable provider returned no exact decode program");
      prepared.exact_decode = std::move(result.operation);
    }
    return er::Status::success();
  } catch (const std::exception& error) {
    return {er::ErrorCode::internal,
            std::string("program preparation failed: ") + error.what()};
  }
}

}  // namespace qllm
