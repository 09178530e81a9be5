// Provider-side view of the common runtime's operation-provider boundary.
//
// The reference links providers into its runner as C++ objects that implement
// IOperationProvider (runtime/include/expert/runtime/program_executor.hpp:
// 244-370) and are advertised by a metadata factory returning
// WorkerProviderDefinition (runtime/include/expert/runtime/worker_provider.hpp:
// 16-21) with KernelCapability entries (model_descriptor.hpp:60-80).  This
// header declares the slice of that boundary the verify path crosses, with
// the same type names, member names and meanings, so that the provider source
// compiles against the reference's own headers by swapping this include.
// Types the verify path never touches (the compiled SSA program, parking and
// snapshot results) are reduced to what prepare() needs; the model descriptor
// itself is in model_descriptor.hpp.
#pragma once

#include "model_descriptor.hpp"
#include "status.hpp"

#include <chrono>
#include <cstddef>
#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <span>
#include <string>
#include <string_view>
#include <utility>
#include <vector>

namespace expert::runtime {

// program_executor.hpp:24-50
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

struct ImmutableModelTensor final {
  std::string name;
  std::string encoding;     // "FP4_E2M1", "F32", "BF16", ...
  std::uint32_t quant_abi{};  // 3 = UE8M0 per 32; 16 = binary16 per 16
  std::vector<std::uint32_t> shape;
  std::uint64_t data_offset{};
  std::uint64_t data_bytes{};
  std::uint64_t scale_offset{};
  std::uint64_t scale_bytes{};
  ExecutionValue value;
};

// program_executor.hpp:52-62
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

// Reduced form of OperationPreparationContext / ExactDecodePreparationContext
// (program_executor.hpp:79-84,176-181): the capability the artifact declared
// for the operation, its integer parameters (floats travel as IEEE-754 bits
// under "*_f32_bits" keys, dense_fp4_provider.cpp:3455-3484) and the tensors
// bound to its roles.
struct OperationPreparationContext final {
  std::string capability;
  std::uint32_t abi{};
  std::map<std::string, std::uint64_t, std::less<>> parameters;
  std::span<const PreparedTensorBinding> tensors;
};
using ExactDecodePreparationContext = OperationPreparationContext;

struct PrepareOperationResult final {
  Status status;
  std::shared_ptr<const IPreparedOperation> operation;
};

struct ProgramRequestContext final {
  std::uint64_t request_id{};
  std::chrono::steady_clock::time_point deadline{
      std::chrono::steady_clock::time_point::max()};
  std::map<std::string, std::uint64_t, std::less<>> parameters;
};

struct CreateOperationRequestStateResult final {
  Status status;
  std::shared_ptr<IOperationProviderRequestState> state;
};

// program_executor.hpp:183-212
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

struct ExactDecodeExecutionResult final {
  Status status;
  std::vector<std::uint32_t> emitted_tokens;
  std::uint32_t next_token{};
  std::uint32_t positions_advanced{};
};

// program_executor.hpp:214-238.  The provider returns handles that are
// already complete (dense_fp4_provider.cpp:5622); poll() yields the result
// once, an invalid handle means the invocation was rejected.
class ExactDecodeExecutionHandle final {
 public:
  using Poll = std::function<std::optional<ExactDecodeExecutionResult>()>;
  using Cancel = std::function<void()>;
  ExactDecodeExecutionHandle() = default;
  [[nodiscard]] bool valid() const noexcept { return static_cast<bool>(poll_); }
  [[nodiscard]] std::optional<ExactDecodeExecutionResult> poll() {
    return poll_ ? poll_() : std::nullopt;
  }
  void cancel() noexcept {
    if (cancel_) cancel_();
  }
  [[nodiscard]] static ExactDecodeExecutionHandle from_callbacks(Poll poll,
                                                                 Cancel cancel) {
    ExactDecodeExecutionHandle handle;
    handle.poll_ = std::move(poll);
    handle.cancel_ = std::move(cancel);
    return handle;
  }

 private:
  Poll poll_;
  Cancel cancel_;
};

// program_executor.hpp:244-370, the members the exact-decode path uses.
class IOperationProvider {
 public:
  virtual ~IOperationProvider() = default;
  [[nodiscard]] virtual PrepareOperationResult prepare(
      const OperationPreparationContext& context) = 0;
  [[nodiscard]] virtual CreateOperationRequestStateResult create_request_state(
      const ProgramRequestContext& request) = 0;
  [[nodiscard]] virtual PrepareOperationResult prepare_exact_decode(
      const ExactDecodePreparationContext&) {
    return {{ErrorCode::invalid_argument,
             "operation provider has no exact decode implementation"},
            {}};
  }
  [[nodiscard]] virtual Status synchronize_exact_decode_batch(
      const IPreparedOperation&,
      const std::shared_ptr<IOperationProviderRequestState>&,
      const ExactDecodeSynchronizationBatch&) {
    return {ErrorCode::invalid_argument,
            "operation provider has no exact decode implementation"};
  }
  [[nodiscard]] virtual ExactDecodeExecutionHandle execute_exact_decode(
      const IPreparedOperation&,
      const std::shared_ptr<IOperationProviderRequestState>&,
      const ExactDecodeInvocation&) {
    return {};
  }
};

// worker_provider.hpp:16-21 (KernelCapability is in model_descriptor.hpp)
struct WorkerProviderDefinition final {
  std::string name;
  std::uint32_t priority{};
  std::vector<KernelCapability> capabilities;
  void* entry{};
};

// Fields of ExecutionProviderModule::ServiceContract the runner checks for a
// dense resident provider (program_executor.hpp:375-425,
// moe_vm_runner.cpp:540-568).
struct ServiceContract final {
  std::string kv_dtype;
  std::string kv_allocation;
  std::uint32_t kv_page_tokens{};
  std::uint64_t kv_page_bytes{};
  std::uint64_t kv_page_capacity{};
  std::string placement_mode;
  bool mtp_resource_available{};
  bool mtp_runtime_ready{};
  bool mtp_enabled{};
  bool sampling_supported{};
};

}  // namespace expert::runtime
