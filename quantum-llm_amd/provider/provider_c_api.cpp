// extern "C" surface of the provider (include/qllm_provider.h).
#include "qllm_provider.h"

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include <hip/hip_runtime.h>

#include "artifact_provider.hpp"
#include "dense_fp4_provider.hpp"
#include "dense_record.hpp"
#include "expert/runtime/sha256.hpp"

namespace er = expert::runtime;

struct qllm_provider {
  std::shared_ptr<qllm::Mi355DenseFp4Provider> provider;
  // set when the provider was created from an artifact directory
  std::shared_ptr<er::ModelArtifact> artifact;
  std::shared_ptr<er::IModelTensorStore> tensor_store;
  // the compiled form of every prepared operation, in program order: what
  // execute() is invoked with
  std::vector<er::CompiledOperationProgram> compiled;
  std::vector<er::PreparedTensorBinding> staged;
  std::vector<std::shared_ptr<const er::IPreparedOperation>> operations;
  std::shared_ptr<const er::IPreparedOperation> exact;
  std::shared_ptr<er::IOperationProviderRequestState> state;
  er::ProgramRequestContext request;
};

namespace {

thread_local char last_error[512] = "";

int32_t fail(int32_t code, const std::string& message) {
  std::snprintf(last_error, sizeof(last_error), "%s", message.c_str());
  return code;
}

int32_t from_status(const er::Status& status) {
  if (status.ok()) return QLLM_OK;
  return fail(static_cast<int32_t>(status.code()), std::string(status.message()));
}

}  // namespace

extern "C" const char* qllm_provider_last_error(void) { return last_error; }

extern "C" qllm_provider* qllm_provider_create(
    const qllm_dense_geometry* geometry) {
  if (!geometry) {
    fail(QLLM_INVALID_ARGUMENT, "geometry is null");
    return nullptr;
  }
  try {
    qllm::DenseGeometry g;
    g.hidden = geometry->hidden;
    g.intermediate = geometry->intermediate;
    g.layers = geometry->layers;
    g.query_heads = geometry->query_heads;
    g.kv_heads = geometry->kv_heads;
    g.head_dim = geometry->head_dim;
    g.rotary_dim = geometry->rotary_dim;
    g.vocabulary = geometry->vocabulary;
    g.rope_theta = geometry->rope_theta;
    g.norm_epsilon = geometry->norm_epsilon;
    g.output_gated = geometry->output_gated != 0;
    g.qk_norm = geometry->qk_norm != 0;
    g.zero_centered_norm = geometry->zero_centered_norm != 0;
    g.scale_scheme = geometry->scale_scheme;
    g.kv_encoding = geometry->kv_encoding == 1U
                        ? qllm::KvEncoding::fp16
                        : qllm::KvEncoding::q4_f16_per_head;
    g.kv_page_tokens = geometry->kv_page_tokens;
    g.max_context = geometry->max_context;
    g.draft_depth = geometry->draft_depth;
    g.mtp_layers = geometry->mtp_layers;
    g.draft_vocabulary = geometry->draft_vocabulary;
    g.prefill_chunk_rows = geometry->prefill_chunk_rows;
    g.activation_q8 = geometry->activation_q8 != 0U;
    auto handle = std::make_unique<qllm_provider>();
    handle->provider = std::make_shared<qllm::Mi355DenseFp4Provider>(g);
    return handle.release();
  } catch (const std::exception& error) {
    fail(QLLM_INTERNAL, error.what());
    return nullptr;
  }
}

extern "C" qllm_provider* qllm_provider_create_from_artifact(
    const char* artifact_root, uint32_t max_context, uint32_t kv_page_tokens,
    const char* kv_cache_dtype, uint32_t mtp_draft_depth) {
  if (!artifact_root) {
    fail(QLLM_INVALID_ARGUMENT, "artifact root is null");
    return nullptr;
  }
  try {
    qllm::ArtifactProviderOptions options;
    options.max_context = max_context;
    if (kv_page_tokens) options.kv_page_tokens = kv_page_tokens;
    if (kv_cache_dtype) options.kv_cache_dtype = kv_cache_dtype;
    options.mtp_draft_depth = mtp_draft_depth;
    // what the runner's main does (moe_vm_runner.cpp:1501-1528): load the
    // artifact, create the one module that serves its program, bind, prepare
    auto artifact = std::make_shared<er::ModelArtifact>();
    if (auto status = er::ModelArtifact::load(artifact_root, *artifact);
        !status.ok()) {
      from_status(status);
      return nullptr;
    }
    if (mtp_draft_depth)
      if (auto status = artifact->configure_mtp_draft_depth(mtp_draft_depth);
          !status.ok()) {
        from_status(status);
        return nullptr;
      }
    auto created = qllm::make_mi355_dense_fp4_module(artifact, options);
    if (!created.status.ok()) {
      from_status(created.status);
      return nullptr;
    }
    qllm::PreparedProgram prepared;
    if (auto status =
            qllm::prepare_program(artifact->model(), created.module, prepared);
        !status.ok()) {
      from_status(status);
      return nullptr;
    }
    auto handle = std::make_unique<qllm_provider>();
    handle->provider = std::dynamic_pointer_cast<qllm::Mi355DenseFp4Provider>(
        created.module.definition.implementation);
    handle->artifact = std::move(artifact);
    handle->tensor_store = std::move(created.module.tensor_store);
    handle->operations = std::move(prepared.operations);
    handle->compiled = std::move(prepared.bound.program.operations);
    handle->exact = std::move(prepared.exact_decode);
    return handle.release();
  } catch (const std::exception& error) {
    fail(QLLM_INTERNAL, error.what());
    return nullptr;
  }
}

extern "C" void qllm_provider_destroy(qllm_provider* provider) {
  delete provider;
}

extern "C" uint32_t qllm_provider_capabilities(char* buffer, size_t capacity) {
  const auto definition = qllm::make_mi355_dense_fp4_provider();
  size_t used = 0;
  uint32_t count = 0;
  for (const auto& capability : definition.capabilities) {
    const auto bytes = capability.capability.size() + 1U;
    if (buffer && used + bytes <= capacity) {
      std::memcpy(buffer + used, capability.capability.c_str(), bytes);
      used += bytes;
    }
    ++count;
  }
  return count;
}

extern "C" int32_t qllm_provider_stage_tensor(
    qllm_provider* provider, const char* role, const char* encoding,
    uint32_t quant_abi, uint32_t rows, uint32_t columns, const void* data,
    size_t data_bytes, const void* scales, size_t scale_bytes) {
  if (!provider || !role || !encoding || !data || !data_bytes)
    return fail(QLLM_INVALID_ARGUMENT, "staged tensor is invalid");
  try {
    auto blob = std::make_shared<std::vector<std::byte>>(data_bytes + scale_bytes);
    std::memcpy(blob->data(), data, data_bytes);
    if (scale_bytes) std::memcpy(blob->data() + data_bytes, scales, scale_bytes);
    auto tensor = std::make_shared<er::ImmutableModelTensor>();
    tensor->name = role;
    tensor->encoding = encoding;
    tensor->quant_abi = quant_abi;
    tensor->shape = columns ? std::vector<uint32_t>{rows, columns}
                            : std::vector<uint32_t>{rows};
    tensor->data_offset = 0;
    tensor->data_bytes = data_bytes;
    tensor->scale_offset = data_bytes;
    tensor->scale_bytes = scale_bytes;
    tensor->value.abi = "artifact.dense-record.v1";
    tensor->value.memory_domain = "host.mmap.readonly";
    tensor->value.owner = blob;
    tensor->value.data = blob->data();
    tensor->value.bytes = blob->size();
    provider->staged.push_back({role, tensor});
    return QLLM_OK;
  } catch (const std::exception& error) {
    return fail(QLLM_INTERNAL, error.what());
  }
}

extern "C" int32_t qllm_provider_prepare(qllm_provider* provider,
                                         const char* capability) {
  if (!provider || !capability)
    return fail(QLLM_INVALID_ARGUMENT, "prepare arguments are invalid");
  try {
    // A one-operation program description for the staged tensors: the ports
    // and value ABIs the artifact compiler declares for this kind of block
    // (compiler/expert_pack/adapters.py:1422-1602).
    const std::string name = capability;
    const std::string hidden = "batch.hidden.f32.cuda.v1";
    const std::string token = "batch.token-id.u32.host.v1";
    const std::string position = "batch.position.u32.host.v1";
    const auto index = static_cast<uint32_t>(provider->operations.size());
    er::OperationProgramDescriptor operation;
    operation.logical_operation = index;
    operation.logical_layer = er::kModelLevelOperationLayer;
    operation.capability = name;
    operation.abi_version = 1U;
    const auto in = [&](const char* port, const std::string& abi) {
      operation.input_bindings[port] = {std::string("staged.") + port, abi};
    };
    const auto out = [&](const char* port, const std::string& abi) {
      operation.output_bindings[port] = {std::string("staged.out.") + port, abi};
    };
    if (name.starts_with("embedding.")) {
      in("token_ids", token);
      out("hidden", hidden);
    } else if (name.starts_with("block.")) {
      in("hidden", hidden);
      in("positions", position);
      out("hidden", hidden);
    } else if (name.starts_with("head.")) {
      in("hidden", hidden);
      out("token_ids", token);
    } else {
      in("hidden", hidden);
      out("hidden", hidden);
    }
    er::CompiledOperationProgram compiled;
    compiled.logical_operation = index;
    compiled.logical_layer = operation.logical_layer;
    uint32_t slot = 0;
    for (const auto& [port, binding] : operation.input_bindings)
      compiled.input_values.push_back({port, slot++});
    for (const auto& [port, binding] : operation.output_bindings)
      compiled.output_values.push_back({port, slot++});
    const er::ModelDescriptor model{};
    auto result = provider->provider->prepare(
        {model, operation, compiled, provider->staged});
    provider->staged.clear();
    if (!result.status.ok()) return from_status(result.status);
    provider->operations.push_back(result.operation);
    provider->compiled.push_back(std::move(compiled));
    return QLLM_OK;
  } catch (const std::exception& error) {
    provider->staged.clear();
    return fail(QLLM_INTERNAL, error.what());
  }
}

extern "C" int32_t qllm_provider_prepare_exact_decode(qllm_provider* provider,
                                                      const char* capability) {
  if (!provider || !capability)
    return fail(QLLM_INVALID_ARGUMENT, "prepare arguments are invalid");
  try {
    // the exact-decode contract the artifact declares (:2934-2966)
    const auto& geometry = provider->provider->geometry();
    er::ExactDecodeProgramDescriptor program;
    program.capability = capability;
    program.abi_version = 2U;
    program.maximum_emitted_tokens = geometry.draft_depth + 1U;
    program.parameters["draft_depth"] = geometry.draft_depth;
    program.parameters["source_mtp_layers"] = 1U;
    er::CompiledExactDecodeProgram compiled;
    compiled.maximum_emitted_tokens = program.maximum_emitted_tokens;
    compiled.parameters = program.parameters;
    const er::ModelDescriptor model{};
    auto result = provider->provider->prepare_exact_decode(
        {model, program, compiled, provider->staged});
    provider->staged.clear();
    if (!result.status.ok()) return from_status(result.status);
    provider->exact = result.operation;
    return QLLM_OK;
  } catch (const std::exception& error) {
    provider->staged.clear();
    return fail(QLLM_INTERNAL, error.what());
  }
}

extern "C" int32_t qllm_provider_load_synthetic_weights(qllm_provider* provider,
                                                        uint64_t seed) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return from_status(provider->provider->load_synthetic_weights(seed));
}

extern "C" int32_t qllm_provider_prefill_synthetic_kv(qllm_provider* provider,
                                                      uint32_t tokens,
                                                      uint64_t seed) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return from_status(provider->provider->prefill_synthetic_kv(tokens, seed));
}

extern "C" int32_t qllm_provider_begin_request(qllm_provider* provider,
                                               uint32_t temperature_ppm,
                                               uint32_t top_p_ppm,
                                               uint32_t top_k,
                                               uint32_t min_p_ppm,
                                               uint64_t seed) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  provider->request = {};
  provider->request.parameters["sampling_temperature_ppm"] = temperature_ppm;
  provider->request.parameters["sampling_top_p_ppm"] = top_p_ppm;
  provider->request.parameters["sampling_top_k"] = top_k;
  provider->request.parameters["sampling_min_p_ppm"] = min_p_ppm;
  provider->request.parameters["sampling_seed"] = seed;
  provider->request.parameters["sampling_presence_penalty_biased_ppm"] =
      2'000'000U;
  provider->request.parameters["sampling_first_output_position"] = 0U;
  provider->request.parameters["exact_decode_enabled"] = 1U;
  // the handle's previous request gives its slot back first
  provider->state.reset();
  auto result = provider->provider->create_request_state(provider->request);
  if (!result.status.ok()) return from_status(result.status);
  provider->state = result.state;
  return QLLM_OK;
}

extern "C" int32_t qllm_provider_begin_request_with(qllm_provider* provider,
                                                    const char* const* names,
                                                    const uint64_t* values,
                                                    uint32_t count) {
  if (!provider || (count && (!names || !values)))
    return fail(QLLM_INVALID_ARGUMENT, "request parameters are invalid");
  try {
    provider->request = {};
    for (uint32_t index = 0; index < count; ++index) {
      if (!names[index])
        return fail(QLLM_INVALID_ARGUMENT, "request parameter name is null");
      provider->request.parameters[names[index]] = values[index];
    }
    provider->state.reset();
    auto result = provider->provider->create_request_state(provider->request);
    if (!result.status.ok()) return from_status(result.status);
    provider->state = result.state;
    return QLLM_OK;
  } catch (const std::exception& error) {
    return fail(QLLM_INTERNAL, error.what());
  }
}

extern "C" int32_t qllm_provider_synchronize(qllm_provider* provider,
                                             uint32_t token,
                                             uint32_t position) {
  if (!provider || !provider->exact || !provider->state)
    return fail(QLLM_INVALID_ARGUMENT, "exact decode is not prepared");
  // `token` stands at `position`; it was chosen from the target's hidden state
  // one position earlier, which is where the synchronisation batch starts
  if (position == 0U)
    return from_status(
        provider->provider->begin_stream(provider->state, token));
  const uint32_t tokens[1] = {token};
  er::ExactDecodeSynchronizationBatch batch{provider->request, tokens,
                                            position - 1U, true};
  return from_status(provider->provider->synchronize_exact_decode_batch(
      *provider->exact, provider->state, batch));
}

extern "C" int32_t qllm_provider_prefill(qllm_provider* provider,
                                         const uint32_t* tokens, uint32_t count,
                                         uint32_t first_position,
                                         uint32_t* predicted) {
  if (!provider || !tokens || !count || !predicted)
    return fail(QLLM_INVALID_ARGUMENT, "prompt arguments are invalid");
  const auto result = provider->provider->prefill(
      provider->state, {tokens, count}, first_position, provider->request);
  if (!result.status.ok()) return from_status(result.status);
  *predicted = result.predicted;
  return QLLM_OK;
}

extern "C" int32_t qllm_provider_set_drafts(
    qllm_provider* provider, const uint32_t* draft_tokens, uint32_t draft_count,
    const uint32_t* distribution_counts, const uint32_t* distribution_tokens,
    const double* distribution_probabilities) {
  if (!provider || !provider->state || !draft_tokens || !draft_count)
    return fail(QLLM_INVALID_ARGUMENT, "draft arguments are invalid");
  try {
    std::vector<qllm::DraftPrediction> drafts(draft_count);
    size_t offset = 0;
    for (uint32_t index = 0; index < draft_count; ++index) {
      drafts[index].token = draft_tokens[index];
      const uint32_t count = distribution_counts ? distribution_counts[index] : 0U;
      if (count == 0U) {
        drafts[index].distribution.entries = {{draft_tokens[index], 1.0}};
      } else {
        if (!distribution_tokens || !distribution_probabilities)
          return fail(QLLM_INVALID_ARGUMENT, "draft distribution is missing");
        drafts[index].distribution.entries.reserve(count);
        for (uint32_t entry = 0; entry < count; ++entry)
          drafts[index].distribution.entries.push_back(
              {distribution_tokens[offset + entry],
               distribution_probabilities[offset + entry]});
        offset += count;
      }
    }
    return from_status(provider->provider->set_draft_predictions(
        provider->state, std::move(drafts)));
  } catch (const std::exception& error) {
    return fail(QLLM_INTERNAL, error.what());
  }
}

extern "C" int32_t qllm_provider_verify(qllm_provider* provider,
                                        uint32_t guaranteed_token,
                                        uint32_t position,
                                        uint32_t context_limit,
                                        uint32_t* emitted,
                                        uint32_t* emitted_count,
                                        uint32_t* next_token,
                                        uint32_t* positions_advanced) {
  if (!provider || !provider->exact || !provider->state || !emitted ||
      !emitted_count || !next_token || !positions_advanced)
    return fail(QLLM_INVALID_ARGUMENT, "verify arguments are invalid");
  er::ExactDecodeInvocation invocation{provider->request, guaranteed_token,
                                       position, context_limit};
  auto handle = provider->provider->execute_exact_decode(
      *provider->exact, provider->state, invocation);
  if (!handle.valid())
    return fail(QLLM_INVALID_ARGUMENT, "exact decode invocation was rejected");
  auto result = handle.poll();
  if (!result) return fail(QLLM_INTERNAL, "exact decode did not complete");
  if (!result->status.ok()) return from_status(result->status);
  *emitted_count = static_cast<uint32_t>(result->emitted_tokens.size());
  for (size_t index = 0; index < result->emitted_tokens.size(); ++index)
    emitted[index] = result->emitted_tokens[index];
  *next_token = result->next_token;
  *positions_advanced = result->positions_advanced;
  return QLLM_OK;
}

extern "C" int32_t qllm_provider_run_target(qllm_provider* provider,
                                            const uint32_t* tokens,
                                            uint32_t rows,
                                            uint32_t first_position) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return from_status(provider->provider->run_target(tokens, rows, first_position));
}

extern "C" int32_t qllm_provider_execute_program(qllm_provider* provider,
                                                 const uint32_t* tokens,
                                                 const uint32_t* positions,
                                                 uint32_t rows,
                                                 uint32_t* next_token) {
  if (!provider || !tokens || !positions || !rows || !next_token ||
      !provider->state || provider->operations.empty() ||
      provider->operations.size() != provider->compiled.size())
    return fail(QLLM_INVALID_ARGUMENT, "program execution arguments are invalid");
  try {
    // The operations in program order, each fed through its ports: token ids
    // and positions are the program's inputs, the hidden state is whatever
    // the operation before produced (the dense program is a chain).
    const auto host_value = [](const char* abi, const uint32_t* words,
                               uint32_t count) {
      auto owner = std::make_shared<std::vector<uint32_t>>(words, words + count);
      return er::ExecutionValue{abi, "host", owner,
                                reinterpret_cast<const std::byte*>(owner->data()),
                                owner->size() * sizeof(uint32_t)};
    };
    const auto token_value = host_value("batch.token-id.u32.host.v1", tokens, rows);
    const auto position_value =
        host_value("batch.position.u32.host.v1", positions, rows);
    er::ExecutionValue hidden;
    er::ExecutionValue selected;
    for (size_t index = 0; index < provider->operations.size(); ++index) {
      const auto& compiled = provider->compiled[index];
      std::vector<er::ExecutionValue> inputs;
      for (const auto& binding : compiled.input_values) {
        if (binding.port == "token_ids")
          inputs.push_back(token_value);
        else if (binding.port == "positions")
          inputs.push_back(position_value);
        else if (binding.port == "hidden")
          inputs.push_back(hidden);
        else
          return fail(QLLM_INVALID_ARGUMENT,
                      "operation input port is not part of a dense program: " +
                          binding.port);
      }
      auto handle = provider->provider->execute(
          *provider->operations[index], provider->state,
          er::OperationInvocation{provider->request, compiled, inputs});
      if (!handle.valid())
        return fail(QLLM_INVALID_ARGUMENT, "operation invocation was rejected");
      auto result = handle.poll();
      if (!result) return fail(QLLM_INTERNAL, "operation did not complete");
      if (!result->status.ok()) return from_status(result->status);
      if (result->outputs.size() != compiled.output_values.size())
        return fail(QLLM_INTERNAL, "operation returned a partial output set");
      for (size_t port = 0; port < compiled.output_values.size(); ++port) {
        if (compiled.output_values[port].port == "hidden")
          hidden = result->outputs[port];
        else if (compiled.output_values[port].port == "token_ids")
          selected = result->outputs[port];
      }
    }
    if (!selected.valid() || selected.bytes < sizeof(uint32_t))
      return fail(QLLM_INTERNAL, "program produced no token");
    std::memcpy(next_token, selected.data + selected.bytes - sizeof(uint32_t),
                sizeof(uint32_t));
    return QLLM_OK;
  } catch (const std::exception& error) {
    return fail(QLLM_INTERNAL, error.what());
  }
}

extern "C" int32_t qllm_provider_synchronize_batch(qllm_provider* provider,
                                                   const uint32_t* next_tokens,
                                                   uint32_t count,
                                                   uint32_t first_target_position,
                                                   int32_t produce_final_draft) {
  if (!provider || !provider->exact || !provider->state || !next_tokens || !count)
    return fail(QLLM_INVALID_ARGUMENT, "exact decode is not prepared");
  er::ExactDecodeSynchronizationBatch batch{
      provider->request, {next_tokens, count}, first_target_position,
      produce_final_draft != 0};
  return from_status(provider->provider->synchronize_exact_decode_batch(
      *provider->exact, provider->state, batch));
}

extern "C" int32_t qllm_provider_copy_matrix_rows(qllm_provider* provider,
                                                  const char* name,
                                                  uint32_t first_row,
                                                  uint32_t rows, void* host_codes,
                                                  void* host_scales) {
  if (!provider || !name) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return from_status(provider->provider->copy_matrix_rows(
      name, first_row, rows, host_codes, host_scales));
}

extern "C" int32_t qllm_provider_capture_target(qllm_provider* provider,
                                                const uint32_t* tokens,
                                                uint32_t rows,
                                                uint32_t first_position) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return from_status(
      provider->provider->capture_target_graph(tokens, rows, first_position));
}

extern "C" int32_t qllm_provider_replay_target(qllm_provider* provider) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return from_status(provider->provider->replay_target_graph());
}

extern "C" int32_t qllm_provider_synchronize_stream(qllm_provider* provider) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return from_status(provider->provider->synchronize());
}

namespace {
int32_t copy_rows(qllm_provider* provider, const float* source, size_t count,
                  float* host_output) {
  if (!provider || !source || !host_output || !count)
    return fail(QLLM_INVALID_ARGUMENT, "copy arguments are invalid");
  auto status = provider->provider->synchronize();
  if (!status.ok()) return from_status(status);
  const auto error = hipMemcpy(host_output, source, count * sizeof(float),
                               hipMemcpyDeviceToHost);
  if (error != hipSuccess) return fail(QLLM_INTERNAL, hipGetErrorString(error));
  return QLLM_OK;
}
}  // namespace

extern "C" int32_t qllm_provider_copy_logits(qllm_provider* provider,
                                             uint32_t rows,
                                             float* host_output) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return copy_rows(provider, provider->provider->logits(),
                   size_t{rows} * provider->provider->geometry().vocabulary,
                   host_output);
}

extern "C" int32_t qllm_provider_copy_hidden(qllm_provider* provider,
                                             uint32_t rows,
                                             float* host_output) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return copy_rows(provider, provider->provider->hidden(),
                   size_t{rows} * provider->provider->geometry().hidden,
                   host_output);
}

extern "C" int32_t qllm_provider_time_kernel(qllm_provider* provider,
                                             const char* which, uint32_t rounds,
                                             uint32_t context_tokens,
                                             double* microseconds,
                                             uint64_t* launches) {
  if (!provider || !which) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return from_status(provider->provider->time_kernel(
      which, rounds, context_tokens, microseconds, launches));
}

extern "C" uint64_t qllm_provider_kv_page_bytes(const qllm_provider* provider) {
  return provider ? provider->provider->kv_page_bytes() : 0U;
}

extern "C" int32_t qllm_provider_copy_kv_page(qllm_provider* provider,
                                              uint32_t page_index,
                                              void* host_output) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return from_status(provider->provider->copy_kv_page(page_index, host_output));
}

extern "C" int32_t qllm_provider_copy_mtp_state(qllm_provider* provider,
                                                float* host_last_hidden,
                                                float* host_draft_logits) {
  if (!provider) return fail(QLLM_INVALID_ARGUMENT, "provider is null");
  return from_status(
      provider->provider->copy_mtp_state(host_last_hidden, host_draft_logits));
}

extern "C" uint32_t qllm_provider_drafts(const qllm_provider* provider,
                                         uint32_t* tokens, uint32_t capacity) {
  if (!provider || !provider->state) return 0U;
  const auto state =
      std::dynamic_pointer_cast<qllm::DenseFp4RequestState>(provider->state);
  if (!state || !state->draft_valid) return 0U;
  const auto count = static_cast<uint32_t>(state->draft_predictions.size());
  for (uint32_t index = 0; tokens && index < count && index < capacity; ++index)
    tokens[index] = state->draft_predictions[index].token;
  return count;
}

extern "C" uint32_t qllm_provider_draft_vocabulary(const qllm_provider* provider) {
  return provider ? provider->provider->geometry().draft_vocabulary : 0U;
}

extern "C" const float* qllm_provider_logits(const qllm_provider* provider) {
  return provider ? provider->provider->logits() : nullptr;
}

extern "C" const float* qllm_provider_hidden(const qllm_provider* provider) {
  return provider ? provider->provider->hidden() : nullptr;
}

extern "C" void* qllm_provider_stream(const qllm_provider* provider) {
  return provider ? provider->provider->stream() : nullptr;
}

extern "C" uint64_t qllm_provider_weight_bytes(const qllm_provider* provider) {
  return provider ? provider->provider->weight_bytes() : 0U;
}

extern "C" uint64_t qllm_provider_telemetry(const qllm_provider* provider,
                                            const char* name) {
  if (!provider || !name) return 0U;
  const auto values = provider->provider->telemetry();
  const auto found = values.find(name);
  return found == values.end() ? 0U : found->second;
}

// ---- host sampling mathematics ----------------------------------------------

namespace {

er::SamplingDistribution distribution_from(const uint32_t* tokens,
                                           const double* probabilities,
                                           uint32_t count) {
  er::SamplingDistribution distribution;
  distribution.entries.reserve(count);
  for (uint32_t i = 0; i < count; ++i)
    distribution.entries.push_back({tokens[i], probabilities[i]});
  return distribution;
}

template <typename Body>
int32_t guarded(Body&& body) {
  try {
    body();
    return QLLM_OK;
  } catch (const std::invalid_argument& error) {
    return fail(QLLM_INVALID_ARGUMENT, error.what());
  } catch (const std::exception& error) {
    return fail(QLLM_INTERNAL, error.what());
  }
}

}  // namespace

extern "C" int32_t qllm_sampling_make_distribution(
    const float* sorted_logits, const uint32_t* sorted_tokens, uint32_t count,
    uint32_t temperature_ppm, uint32_t top_p_ppm, uint32_t min_p_ppm,
    uint32_t* tokens_out, double* probabilities_out, uint32_t* count_out) {
  if ((count && (!sorted_logits || !sorted_tokens || !tokens_out ||
                 !probabilities_out)) || !count_out)
    return fail(QLLM_INVALID_ARGUMENT, "null sampling buffer");
  return guarded([&] {
    const auto distribution = er::make_sampling_distribution(
        {sorted_logits, count}, {sorted_tokens, count}, temperature_ppm,
        top_p_ppm, min_p_ppm);
    *count_out = static_cast<uint32_t>(distribution.entries.size());
    for (std::size_t i = 0; i < distribution.entries.size(); ++i) {
      tokens_out[i] = distribution.entries[i].token;
      probabilities_out[i] = distribution.entries[i].probability;
    }
  });
}

extern "C" int32_t qllm_sampling_sample(const uint32_t* tokens,
                                        const double* probabilities,
                                        uint32_t count, double uniform,
                                        uint32_t* token_out) {
  if ((count && (!tokens || !probabilities)) || !token_out)
    return fail(QLLM_INVALID_ARGUMENT, "null sampling buffer");
  return guarded([&] {
    *token_out = er::sample_distribution(
        distribution_from(tokens, probabilities, count), uniform);
  });
}

extern "C" int32_t qllm_sampling_rejection(
    uint32_t proposal, const uint32_t* target_tokens,
    const double* target_probabilities, uint32_t target_count,
    const uint32_t* draft_tokens, const double* draft_probabilities,
    uint32_t draft_count, double acceptance_uniform, double correction_uniform,
    int32_t* accepted_out, uint32_t* token_out, double* target_probability_out,
    double* draft_probability_out) {
  if ((target_count && (!target_tokens || !target_probabilities)) ||
      (draft_count && (!draft_tokens || !draft_probabilities)) ||
      !accepted_out || !token_out)
    return fail(QLLM_INVALID_ARGUMENT, "null sampling buffer");
  return guarded([&] {
    const auto result = er::rejection_sample(
        proposal,
        distribution_from(target_tokens, target_probabilities, target_count),
        distribution_from(draft_tokens, draft_probabilities, draft_count),
        acceptance_uniform, correction_uniform);
    *accepted_out = result.accepted ? 1 : 0;
    *token_out = result.token;
    if (target_probability_out)
      *target_probability_out = result.target_probability;
    if (draft_probability_out)
      *draft_probability_out = result.draft_probability;
  });
}

extern "C" double qllm_sampling_counter_uniform(uint64_t seed,
                                                uint32_t position,
                                                uint32_t stream,
                                                uint32_t index) {
  return er::counter_uniform(seed, position, stream, index);
}


// ---- artifact reader ----------------------------------------------------------

struct qllm_artifact {
  er::ModelArtifact artifact;
  er::MappedModelTensorStore store;
};

extern "C" int32_t qllm_sha256(const void* data, size_t bytes, uint8_t* digest) {
  if ((!data && bytes) || !digest)
    return fail(QLLM_INVALID_ARGUMENT, "SHA-256 arguments are invalid");
  const auto result =
      er::sha256({static_cast<const std::byte*>(data), bytes});
  std::memcpy(digest, result.data(), result.size());
  return QLLM_OK;
}

extern "C" int32_t qllm_sha256_portable(const void* data, size_t bytes,
                                        uint8_t* digest) {
  if ((!data && bytes) || !digest)
    return fail(QLLM_INVALID_ARGUMENT, "SHA-256 arguments are invalid");
  const auto result =
      er::sha256_portable({static_cast<const std::byte*>(data), bytes});
  std::memcpy(digest, result.data(), result.size());
  return QLLM_OK;
}

extern "C" int32_t qllm_artifact_open(const char* root, uint32_t mtp_draft_depth,
                                      int32_t map_tensors, qllm_artifact** out) {
  if (!root || !out) return fail(QLLM_INVALID_ARGUMENT, "artifact root is null");
  *out = nullptr;
  try {
    auto handle = std::make_unique<qllm_artifact>();
    if (auto status = er::ModelArtifact::load(root, handle->artifact); !status.ok())
      return from_status(status);
    if (mtp_draft_depth)
      if (auto status = handle->artifact.configure_mtp_draft_depth(mtp_draft_depth);
          !status.ok())
        return from_status(status);
    if (map_tensors)
      if (auto status =
              er::MappedModelTensorStore::create(handle->artifact, handle->store);
          !status.ok())
        return from_status(status);
    *out = handle.release();
    return QLLM_OK;
  } catch (const std::exception& error) {
    return fail(QLLM_INTERNAL, error.what());
  }
}

extern "C" void qllm_artifact_close(qllm_artifact* artifact) { delete artifact; }

extern "C" int32_t qllm_artifact_tensor(qllm_artifact* artifact, const char* name,
                                        int32_t check_header, const void** record,
                                        uint64_t* record_bytes) {
  if (!artifact || !name || !record || !record_bytes)
    return fail(QLLM_INVALID_ARGUMENT, "artifact tensor query is invalid");
  const auto resolved = artifact->store.resolve(name);
  if (!resolved.status.ok()) return from_status(resolved.status);
  if (check_header) {
    const auto& entries = artifact->artifact.dense_tensors();
    const auto entry = std::find_if(
        entries.begin(), entries.end(),
        [name](const er::ArtifactDenseTensor& item) { return item.name == name; });
    if (entry == entries.end())
      return fail(QLLM_INVALID_ARGUMENT, "tensor is absent from the dense index");
    if (auto status = er::validate_dense_record(*entry, resolved.tensor->value.data,
                                                resolved.tensor->value.bytes);
        !status.ok())
      return from_status(status);
  }
  *record = resolved.tensor->value.data;
  *record_bytes = resolved.tensor->value.bytes;
  return QLLM_OK;
}
