// The reference's common VM driving the MI355X provider.  TEST INFRASTRUCTURE
// ONLY.  Built into oracle/_ref/libqllm_ref_vm.so from
//   - the reference's own runtime sources, read where they lie in the
//     reference tree: model program parser and compiler, provider registry,
//     program executor (sessions, SSA interpreter, exact-decode handle
//     validation), artifact reader, tensor store, SHA-256, sampling;
//   - this repository's provider sources (dense_fp4_provider.cpp,
//     artifact_provider.cpp, dense_record.cpp) compiled against the
//     reference's headers instead of the restated ones.
// The shim only forwards: what the runner's main does at start-up
// (runtime/tools/moe_vm_runner.cpp:1501-1532) and what its worker loop calls
// on a session (:679-745, :1107-1183).
#include "expert/runtime/execution_provider.hpp"
#include "expert/runtime/model_artifact.hpp"
#include "expert/runtime/program_executor.hpp"

#include "artifact_provider.hpp"
#include "dense_fp4_provider.hpp"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace er = expert::runtime;

namespace {

constexpr const char* kTokenAbi = "batch.token-id.u32.host.v1";
constexpr const char* kPositionAbi = "batch.position.u32.host.v1";

struct Machine {
  er::ModelArtifact artifact;
  er::ExecutionProviderModule module;
  er::MoeProgramExecutor executor;
  // one session per request slot and one more, so that a test can ask for a
  // request the provider has no slot for; `session` is the selected one
  std::vector<er::ProgramExecutionSession> sessions;
  std::size_t selected = 0;
  er::ProgramExecutionSession& session() { return sessions[selected]; }
  std::string error;
};

int fail(Machine* machine, const er::Status& status) {
  machine->error = std::string(status.message());
  return static_cast<int>(status.code()) ? static_cast<int>(status.code()) : 10;
}

er::ExecutionValue host_words(const char* abi, const std::uint32_t* words,
                              std::uint32_t count) {
  auto owner = std::make_shared<std::vector<std::uint32_t>>(words, words + count);
  return {abi, "host", owner, reinterpret_cast<const std::byte*>(owner->data()),
          owner->size() * sizeof(std::uint32_t)};
}

}  // namespace

extern "C" {

const char* qvm_error(void* machine) {
  return static_cast<Machine*>(machine)->error.c_str();
}

void* qvm_open(const char* root, std::uint32_t max_context,
               std::uint32_t kv_page_tokens, const char* kv_cache_dtype,
               std::uint32_t mtp_draft_depth, std::uint32_t request_capacity,
               char* message, std::size_t capacity) {
  auto machine = std::make_unique<Machine>();
  machine->sessions.resize(std::size_t{request_capacity} + 1U);
  const auto give_up = [&](const er::Status& status) -> void* {
    if (message && capacity) {
      const auto text = std::string(status.message());
      std::snprintf(message, capacity, "%s", text.c_str());
    }
    return nullptr;
  };
  auto status = er::ModelArtifact::load(root, machine->artifact);
  if (!status.ok()) return give_up(status);
  if (mtp_draft_depth) {
    status = machine->artifact.configure_mtp_draft_depth(mtp_draft_depth);
    if (!status.ok()) return give_up(status);
  }
  // the factory with the runner's sixteen arguments (moe_vm_runner.cpp:459-468)
  auto created = qllm::make_mi355_dense_fp4_callable_provider(
      root, max_context, request_capacity, std::uint64_t{1} << 30U, std::uint64_t{1} << 30U,
      std::uint64_t{64} << 20U, kv_page_tokens, kv_cache_dtype, "latency", "fixed",
      false, false, {}, 0U, 0U, mtp_draft_depth);
  if (!created.status.ok()) return give_up(created.status);
  machine->module = std::move(created.module);
  er::ExecutionProviderRegistry registry;
  status = registry.add(machine->module.definition);
  if (!status.ok()) return give_up(status);
  auto bound = registry.bind(machine->artifact.model(),
                             er::ExecutionProviderBindingMode::executable);
  if (!bound.status.ok()) return give_up(bound.status);
  status = er::MoeProgramExecutor::create(machine->artifact.model(),
                                          std::move(bound.provider),
                                          machine->module.tensor_store.get(),
                                          machine->executor);
  if (!status.ok()) return give_up(status);
  if (machine->module.finalize_service) {
    status = machine->module.finalize_service(machine->module.service);
    if (!status.ok()) return give_up(status);
  }
  return machine.release();
}

void qvm_close(void* opaque) {
  auto* machine = static_cast<Machine*>(opaque);
  if (machine)
    for (auto& session : machine->sessions)
      if (session.valid()) session.cancel();
  delete machine;
}

// the service contract fields the runner validates (moe_vm_runner.cpp:540-568)
int qvm_service(void* opaque, char* kv_dtype, std::size_t capacity,
                std::uint32_t* kv_page_tokens, std::uint32_t* prefill_chunk_tokens,
                int* mtp_enabled, int* sampling_supported) {
  const auto& service = static_cast<Machine*>(opaque)->module.service;
  std::snprintf(kv_dtype, capacity, "%s", service.kv_dtype.c_str());
  *kv_page_tokens = service.kv_page_tokens;
  *prefill_chunk_tokens = service.prefill_chunk_tokens;
  *mtp_enabled = service.mtp_enabled && service.mtp_resource_available &&
                 service.mtp_runtime_ready;
  *sampling_supported = service.sampling_supported;
  return 0;
}

int qvm_begin_session(void* opaque, const char* const* names,
                      const std::uint64_t* values, std::uint32_t count) {
  auto* machine = static_cast<Machine*>(opaque);
  // the selected session's previous request ends (and gives its slot back)
  // before the new one begins
  if (machine->session().valid()) machine->session().cancel();
  machine->session() = er::ProgramExecutionSession{};
  er::ProgramRequestContext request;
  request.request_id = machine->selected + 1U;
  for (std::uint32_t index = 0; index < count; ++index)
    request.parameters[names[index]] = values[index];
  auto begun = machine->executor.begin_session(std::move(request));
  if (!begun.status.ok()) return fail(machine, begun.status);
  machine->session() = std::move(begun.session);
  return 0;
}

// which session the calls below address
int qvm_select_session(void* opaque, std::uint32_t index) {
  auto* machine = static_cast<Machine*>(opaque);
  if (index >= machine->sessions.size())
    return fail(machine, {er::ErrorCode::invalid_argument, "no such session"});
  machine->selected = index;
  return 0;
}

// ends the selected session's request
int qvm_end_session(void* opaque) {
  auto* machine = static_cast<Machine*>(opaque);
  if (machine->session().valid()) machine->session().cancel();
  machine->session() = er::ProgramExecutionSession{};
  return 0;
}

// one step of the artifact's program: `rows` tokens at consecutive positions
int qvm_execute(void* opaque, const std::uint32_t* tokens,
                const std::uint32_t* positions, std::uint32_t rows,
                std::uint32_t* next_token) {
  auto* machine = static_cast<Machine*>(opaque);
  std::map<std::string, er::ExecutionValue, std::less<>> inputs;
  for (const auto& [role, endpoint] : machine->artifact.model().program_inputs) {
    if (endpoint.abi == kTokenAbi)
      inputs.emplace(role, host_words(kTokenAbi, tokens, rows));
    else if (endpoint.abi == kPositionAbi)
      inputs.emplace(role, host_words(kPositionAbi, positions, rows));
  }
  auto started = machine->session().execute(std::move(inputs));
  if (!started.status.ok()) return fail(machine, started.status);
  std::optional<er::ProgramExecutionResult> result;
  for (int attempt = 0; attempt < 1000000 && !result; ++attempt)
    result = started.handle.poll();
  if (!result) return fail(machine, {er::ErrorCode::internal, "program never completed"});
  if (!result->status.ok()) return fail(machine, result->status);
  for (const auto& [role, value] : result->outputs)
    if (value.abi == kTokenAbi && value.bytes >= 4U)
      std::memcpy(next_token, value.data + value.bytes - 4U, 4U);
  return 0;
}

int qvm_exact_available(void* opaque) {
  return static_cast<Machine*>(opaque)->session().exact_decode_available() ? 1 : 0;
}

int qvm_synchronize(void* opaque, const std::uint32_t* next_tokens,
                    std::uint32_t count, std::uint32_t first_target_position,
                    int produce_final_draft) {
  auto* machine = static_cast<Machine*>(opaque);
  const auto status = machine->session().synchronize_exact_decode_batch(
      {next_tokens, count}, first_target_position, produce_final_draft != 0);
  return status.ok() ? 0 : fail(machine, status);
}

int qvm_exact_decode(void* opaque, std::uint32_t guaranteed_token,
                     std::uint32_t position, std::uint32_t context_limit,
                     std::uint32_t* emitted, std::uint32_t* emitted_count,
                     std::uint32_t* next_token, std::uint32_t* positions_advanced) {
  auto* machine = static_cast<Machine*>(opaque);
  auto started =
      machine->session().execute_exact_decode(guaranteed_token, position, context_limit);
  if (!started.status.ok()) return fail(machine, started.status);
  std::optional<er::ExactDecodeExecutionResult> result;
  for (int attempt = 0; attempt < 1000000 && !result; ++attempt)
    result = started.handle.poll();
  if (!result) return fail(machine, {er::ErrorCode::internal, "exact decode never completed"});
  if (!result->status.ok()) return fail(machine, result->status);
  *emitted_count = static_cast<std::uint32_t>(result->emitted_tokens.size());
  std::copy(result->emitted_tokens.begin(), result->emitted_tokens.end(), emitted);
  *next_token = result->next_token;
  *positions_advanced = result->positions_advanced;
  return 0;
}

// the provider's logits of the last head, for comparing two ways of driving it
int qvm_copy_logits(void* opaque, std::uint32_t rows, float* host) {
  auto* machine = static_cast<Machine*>(opaque);
  const auto provider = std::dynamic_pointer_cast<qllm::Mi355DenseFp4Provider>(
      machine->module.definition.implementation);
  if (!provider) return 10;
  if (!provider->synchronize().ok()) return 10;
  const auto bytes =
      std::size_t{rows} * provider->geometry().vocabulary * sizeof(float);
  return hipMemcpy(host, provider->logits(), bytes, hipMemcpyDeviceToHost) ==
                 hipSuccess
             ? 0
             : 10;
}

std::uint64_t qvm_telemetry(void* opaque, const char* name) {
  auto* machine = static_cast<Machine*>(opaque);
  if (!machine->module.telemetry) return 0;
  const auto counters = machine->module.telemetry();
  const auto found = counters.find(name);
  return found == counters.end() ? 0U : found->second;
}

}  // extern "C"
