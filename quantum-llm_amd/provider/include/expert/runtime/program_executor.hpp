// The operation-provider boundary of the common runtime, as a provider sees
// it: immutable values and tensors, preparation contexts, request contexts,
// execution results and their handles, IOperationProvider and the loadable
// module (runtime/include/expert/runtime/program_executor.hpp:24-430).  Same
// type names, member names, member order and meanings, so that a provider
// source compiles against either header.  The interpreter side of that file
// (ProgramExecutionSession, MoeProgramExecutor, :432-596) is the common VM's
// business and is not restated.
#pragma once

#include "expert/runtime/execution_provider.hpp"

#include <chrono>
#include <cstddef>
#include <cstdint>
#include <filesystem>
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <span>
#include <string>
#include <string_view>
#include <vector>

namespace expert::runtime {

// :24-36  A value between operations: what it is (abi), where it lives
// (memory_domain), who keeps it alive (owner).
struct ExecutionValue final {
  std::string abi;
  std::string memory_domain;
  std::shared_ptr<const void> owner;
  const std::byte* data{};
  std::uint64_t bytes{};

  [[nodiscard]] bool valid() const noexcept {
    return !abi.empty() && !memory_domain.empty() && owner && data != nullptr &&
           bytes != 0U;
  }
};

// :41-51
struct ImmutableModelTensor final {
  std::string name;
  std::string encoding;
  std::uint32_t quant_abi{};
  std::vector<std::uint32_t> shape;
  std::uint64_t data_offset{};
  std::uint64_t data_bytes{};
  std::uint64_t scale_offset{};
  std::uint64_t scale_bytes{};
  ExecutionValue value;
};

// :53-63
struct ResolveModelTensorResult final {
  Status status;
  std::shared_ptr<const ImmutableModelTensor> tensor;
};

class IModelTensorStore {
 public:
  virtual ~IModelTensorStore() = default;
  [[nodiscard]] virtual ResolveModelTensorResult resolve(
      std::string_view name) = 0;
};

// :65-78
struct PreparedTensorBinding final {
  std::string role;
  std::shared_ptr<const ImmutableModelTensor> tensor;
};

class IPreparedOperation {
 public:
  virtual ~IPreparedOperation() = default;
};

class IOperationProviderRequestState {
 public:
  virtual ~IOperationProviderRequestState() = default;
};

// :79-84
struct OperationPreparationContext final {
  const ModelDescriptor& model;
  const OperationProgramDescriptor& operation;
  const CompiledOperationProgram& compiled;
  std::span<const PreparedTensorBinding> tensors;
};

struct PrepareOperationResult final {
  Status status;
  std::shared_ptr<const IPreparedOperation> operation;
};

// :91-98
struct ProgramRequestContext final {
  std::uint64_t request_id{};
  std::chrono::steady_clock::time_point deadline{
      std::chrono::steady_clock::time_point::max()};
  std::map<std::string, std::uint64_t, std::less<>> parameters;
};

struct CreateOperationRequestStateResult final {
  Status status;
  std::shared_ptr<IOperationProviderRequestState> state;  // null = stateless
};

// :109-127
struct RequestStateParkingResult final {
  Status status;
  std::uint64_t populated_pages{};
  std::uint64_t parked_bytes{};
};

struct RequestStateSnapshotResult final {
  Status status;
  std::uint64_t generation{};
  std::uint64_t populated_pages{};
  std::uint64_t logical_bytes{};
  std::uint64_t written_bytes{};
};

// :129-134  Outputs in the artifact's output-port order.
struct OperationExecutionResult final {
  Status status;
  std::vector<ExecutionValue> outputs;
};

// :136-160  A default-constructed handle is invalid: the invocation was
// rejected.  poll() yields the result once; cancel() is idempotent.
class OperationExecutionHandle final {
 public:
  using Poll = std::function<std::optional<OperationExecutionResult>()>;
  using Cancel = std::function<void()>;

  OperationExecutionHandle();
  OperationExecutionHandle(const OperationExecutionHandle&) = delete;
  OperationExecutionHandle& operator=(const OperationExecutionHandle&) = delete;
  OperationExecutionHandle(OperationExecutionHandle&&) noexcept;
  OperationExecutionHandle& operator=(OperationExecutionHandle&&) noexcept;
  ~OperationExecutionHandle();

  [[nodiscard]] bool valid() const noexcept;
  [[nodiscard]] std::optional<OperationExecutionResult> poll();
  void cancel() noexcept;

  [[nodiscard]] static OperationExecutionHandle from_callbacks(Poll poll,
                                                               Cancel cancel);

 private:
  struct Core;
  explicit OperationExecutionHandle(std::unique_ptr<Core> core) noexcept;
  std::unique_ptr<Core> core_;
};

// :162-166
struct OperationInvocation final {
  ProgramRequestContext request;
  const CompiledOperationProgram& operation;
  std::span<const ExecutionValue> inputs;
};

// :171-176
struct ProgramSequenceInvocation final {
  ProgramRequestContext request;
  const CompiledModelProgram& program;
  std::span<const IPreparedOperation* const> operations;
  std::span<const ExecutionValue> inputs;
};

// :178-183
struct ExactDecodePreparationContext final {
  const ModelDescriptor& model;
  const ExactDecodeProgramDescriptor& program;
  const CompiledExactDecodeProgram& compiled;
  std::span<const PreparedTensorBinding> tensors;
};

// :185-212
struct ExactDecodeSynchronization final {
  ProgramRequestContext request;
  std::uint32_t next_token{};
  std::uint32_t target_position{};
  bool produce_draft{};
};

struct ExactDecodeSynchronizationBatch final {
  ProgramRequestContext request;
  std::span<const std::uint32_t> next_tokens;
  std::uint32_t first_target_position{};
  bool produce_final_draft{};
};

struct ExactDecodeInvocation final {
  ProgramRequestContext request;
  std::uint32_t guaranteed_token{};
  std::uint32_t position{};
  std::uint32_t context_limit{};
};

// emitted_tokens[0] is the guaranteed token, the rest were accepted by the
// target; next_token is chosen but not yet emitted.
struct ExactDecodeExecutionResult final {
  Status status;
  std::vector<std::uint32_t> emitted_tokens;
  std::uint32_t next_token{};
  std::uint32_t positions_advanced{};
};

// :214-238
class ExactDecodeExecutionHandle final {
 public:
  using Poll = std::function<std::optional<ExactDecodeExecutionResult>()>;
  using Cancel = std::function<void()>;

  ExactDecodeExecutionHandle();
  ExactDecodeExecutionHandle(const ExactDecodeExecutionHandle&) = delete;
  ExactDecodeExecutionHandle& operator=(const ExactDecodeExecutionHandle&) =
      delete;
  ExactDecodeExecutionHandle(ExactDecodeExecutionHandle&&) noexcept;
  ExactDecodeExecutionHandle& operator=(ExactDecodeExecutionHandle&&) noexcept;
  ~ExactDecodeExecutionHandle();

  [[nodiscard]] bool valid() const noexcept;
  [[nodiscard]] std::optional<ExactDecodeExecutionResult> poll();
  void cancel() noexcept;
  [[nodiscard]] static ExactDecodeExecutionHandle from_callbacks(Poll poll,
                                                                 Cancel cancel);

 private:
  struct Core;
  explicit ExactDecodeExecutionHandle(std::unique_ptr<Core> core) noexcept;
  std::unique_ptr<Core> core_;
};

// :244-370  Preparation happens once at start-up; execute() and
// execute_exact_decode() are the hot-path entries.  Everything a provider
// does not implement keeps the default, which says so.
class IOperationProvider {
 public:
  virtual ~IOperationProvider() = default;
  [[nodiscard]] virtual PrepareOperationResult prepare(
      const OperationPreparationContext& context) = 0;
  [[nodiscard]] virtual CreateOperationRequestStateResult create_request_state(
      const ProgramRequestContext& request) = 0;
  [[nodiscard]] virtual OperationExecutionHandle execute(
      const IPreparedOperation& operation,
      const std::shared_ptr<IOperationProviderRequestState>& request_state,
      const OperationInvocation& invocation) = 0;
  [[nodiscard]] virtual bool supports_program_sequence(
      const CompiledModelProgram&) const noexcept {
    return false;
  }
  [[nodiscard]] virtual OperationExecutionHandle execute_program_sequence(
      const std::shared_ptr<IOperationProviderRequestState>&,
      const ProgramSequenceInvocation&) {
    return {};
  }
  [[nodiscard]] virtual bool supports_request_state_retention() const noexcept {
    return false;
  }
  [[nodiscard]] virtual Status checkpoint_request_state(
      const std::shared_ptr<IOperationProviderRequestState>&, std::uint32_t) {
    return {ErrorCode::invalid_argument,
            "operation provider has no retention checkpoint implementation"};
  }
  [[nodiscard]] virtual Status rewind_request_state(
      const std::shared_ptr<IOperationProviderRequestState>&, std::uint32_t) {
    return {ErrorCode::invalid_argument,
            "operation provider has no retention rewind implementation"};
  }
  [[nodiscard]] virtual Status rebind_request_state(
      const std::shared_ptr<IOperationProviderRequestState>&,
      const ProgramRequestContext&) {
    return Status::success();
  }
  [[nodiscard]] virtual bool supports_request_state_parking() const noexcept {
    return false;
  }
  [[nodiscard]] virtual RequestStateParkingResult park_request_state(
      const std::shared_ptr<IOperationProviderRequestState>&, std::uint32_t) {
    return {{ErrorCode::invalid_argument,
             "operation provider has no request-state parking implementation"},
            0U, 0U};
  }
  [[nodiscard]] virtual RequestStateParkingResult restore_request_state(
      const std::shared_ptr<IOperationProviderRequestState>&) {
    return {{ErrorCode::invalid_argument,
             "operation provider has no request-state restore implementation"},
            0U, 0U};
  }
  [[nodiscard]] virtual bool supports_request_state_persistence()
      const noexcept {
    return false;
  }
  [[nodiscard]] virtual RequestStateSnapshotResult save_request_state_snapshot(
      const std::shared_ptr<IOperationProviderRequestState>&,
      const std::filesystem::path&, std::uint64_t) {
    return {{ErrorCode::invalid_argument,
             "operation provider has no request-state persistence "
             "implementation"},
            0U, 0U, 0U, 0U};
  }
  [[nodiscard]] virtual RequestStateSnapshotResult load_request_state_snapshot(
      const std::shared_ptr<IOperationProviderRequestState>&,
      const std::filesystem::path&, std::uint64_t) {
    return {{ErrorCode::invalid_argument,
             "operation provider has no request-state persistence "
             "implementation"},
            0U, 0U, 0U, 0U};
  }
  [[nodiscard]] virtual Status prune_request_state_snapshots(
      const std::filesystem::path&, std::uint64_t) {
    return {ErrorCode::invalid_argument,
            "operation provider has no request-state persistence "
            "implementation"};
  }
  [[nodiscard]] virtual PrepareOperationResult prepare_exact_decode(
      const ExactDecodePreparationContext&) {
    return {{ErrorCode::invalid_argument,
             "operation provider has no exact decode implementation"},
            {}};
  }
  [[nodiscard]] virtual Status synchronize_exact_decode(
      const IPreparedOperation&,
      const std::shared_ptr<IOperationProviderRequestState>&,
      const ExactDecodeSynchronization&) {
    return {ErrorCode::invalid_argument,
            "operation provider has no exact decode implementation"};
  }
  // one synchronize_exact_decode per token unless the provider batches them
  [[nodiscard]] virtual Status synchronize_exact_decode_batch(
      const IPreparedOperation& operation,
      const std::shared_ptr<IOperationProviderRequestState>& state,
      const ExactDecodeSynchronizationBatch& synchronization) {
    if (synchronization.next_tokens.empty())
      return {ErrorCode::invalid_argument,
              "exact decode synchronization batch is empty"};
    for (std::size_t index = 0U; index < synchronization.next_tokens.size();
         ++index) {
      auto status = synchronize_exact_decode(
          operation, state,
          {synchronization.request, synchronization.next_tokens[index],
           synchronization.first_target_position +
               static_cast<std::uint32_t>(index),
           synchronization.produce_final_draft &&
               index + 1U == synchronization.next_tokens.size()});
      if (!status.ok()) return status;
    }
    return Status::success();
  }
  [[nodiscard]] virtual ExactDecodeExecutionHandle execute_exact_decode(
      const IPreparedOperation&,
      const std::shared_ptr<IOperationProviderRequestState>&,
      const ExactDecodeInvocation&) {
    return {};
  }
};

// :375-425  What a provider module hands the common runner: the service
// contract the runner validates and publishes, the provider definition for
// the registry, the tensor store, counters, and a hook that runs after every
// tensor is bound and before readiness is published.
struct ExecutionProviderModule final {
  struct ServiceContract final {
    std::string prefill_mode;
    std::uint32_t prefill_chunk_tokens{};
    bool session_retention{};
    std::string request_stream_mode;
    std::string rope_mode;
    std::string kv_dtype;
    std::string kv_allocation;
    std::uint32_t kv_page_tokens{};
    std::uint64_t kv_page_bytes{};
    std::uint64_t kv_page_capacity{};
    std::string placement_mode;
    std::string placement_profile;
    std::uint64_t ram_cache_bytes{};
    std::uint64_t vram_cache_bytes{};
    bool placement_prefetch_enabled{};
    std::string placement_prefetch_state;
    std::uint32_t placement_minimum_observations{};
    bool mtp_resource_available{};
    bool mtp_runtime_ready{};
    bool mtp_enabled{};
    bool retain_previous_route{};
    bool cpu_hybrid_enabled{};
    bool sampling_supported{};
    bool session_parking{};
    bool session_persistence{};
    std::uint64_t session_park_ram_bytes{};
    std::uint64_t session_park_page_capacity{};
    std::string routed_vram_policy{"fixed"};
  } service;
  ExecutionProviderDefinition definition;
  std::shared_ptr<IModelTensorStore> tensor_store;
  std::function<std::map<std::string, std::uint64_t, std::less<>>()> telemetry;
  std::function<Status(ServiceContract&)> finalize_service;
};

struct CreateExecutionProviderModuleResult final {
  Status status;
  ExecutionProviderModule module;
};

}  // namespace expert::runtime
