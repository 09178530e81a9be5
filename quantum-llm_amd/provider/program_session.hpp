// A request's walk through a prepared program for hosts without the common
// VM: the subset of MoeProgramExecutor / ProgramExecutionSession
// (runtime/include/expert/runtime/program_executor.hpp:460-596,
// runtime/src/program_executor.cpp:926-1572) a token-step service needs.  One
// state object per request, inputs by role, operations in program order with
// values handed over by SSA slot, outputs by role; exact-decode results are
// held to the artifact contract before they are passed on.
#pragma once

#include "expert/runtime/program_executor.hpp"

#include "artifact_provider.hpp"

#include <cstdint>
#include <map>
#include <memory>
#include <span>
#include <string>
#include <vector>

namespace qllm {

class ProgramSession final {
 public:
  // `model`, `module` and `prepared` must outlive the session.
  [[nodiscard]] static er::Status begin(const er::ModelDescriptor& model,
                                        const er::ExecutionProviderModule& module,
                                        const PreparedProgram& prepared,
                                        er::ProgramRequestContext request,
                                        std::unique_ptr<ProgramSession>& session);

  struct Outputs final {
    er::Status status;
    std::map<std::string, er::ExecutionValue, std::less<>> values;
  };
  // One pass over the program (SessionState::start, :926-971): the role set
  // must be exactly the program's inputs, every value must carry the ABI the
  // artifact declares for its slot.
  [[nodiscard]] Outputs execute(
      std::map<std::string, er::ExecutionValue, std::less<>> inputs);

  [[nodiscard]] bool exact_decode_available() const noexcept;
  [[nodiscard]] er::Status synchronize_exact_decode_batch(
      std::span<const std::uint32_t> next_tokens,
      std::uint32_t first_target_position, bool produce_final_draft);
  // The result has passed the checks of ExactDecodeState::poll (:825-855).
  [[nodiscard]] er::ExactDecodeExecutionResult execute_exact_decode(
      std::uint32_t guaranteed_token, std::uint32_t position,
      std::uint32_t context_limit);

  [[nodiscard]] const er::ProgramRequestContext& request() const noexcept {
    return request_;
  }
  [[nodiscard]] const std::shared_ptr<er::IOperationProviderRequestState>& state()
      const noexcept {
    return state_;
  }

 private:
  ProgramSession() = default;
  const er::ModelDescriptor* model_{};
  const PreparedProgram* prepared_{};
  std::shared_ptr<er::IOperationProvider> provider_;
  std::shared_ptr<er::IOperationProviderRequestState> state_;
  er::ProgramRequestContext request_;
};

}  // namespace qllm
