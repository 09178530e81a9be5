#include "program_session.hpp"

#include <stdexcept>
#include <utility>

namespace qllm {
namespace {

er::Status rejected(std::string message) {
  return {er::ErrorCode::invalid_argument, std::move(message)};
}

}  // namespace

er::Status ProgramSession::begin(const er::ModelDescriptor& model,
                                 const er::ExecutionProviderModule& module,
                                 const PreparedProgram& prepared,
                                 er::ProgramRequestContext request,
                                 std::unique_ptr<ProgramSession>& session) {
  try {
    if (!module.definition.implementation ||
        prepared.operations.size() != prepared.bound.program.operations.size())
      return rejected("program session needs a prepared program");
    auto created = module.definition.implementation->create_request_state(request);
    if (!created.status.ok()) return created.status;
    std::unique_ptr<ProgramSession> fresh(new ProgramSession());
    fresh->model_ = &model;
    fresh->prepared_ = &prepared;
    fresh->provider_ = module.definition.implementation;
    fresh->state_ = std::move(created.state);
    fresh->request_ = std::move(request);
    session = std::move(fresh);
    return er::Status::success();
  } catch (const std::exception& error) {
    return {er::ErrorCode::internal,
            std::string("model execution session start failed: ") + error.what()};
  }
}

ProgramSession::Outputs ProgramSession::execute(
    std::map<std::string, er::ExecutionValue, std::less<>> inputs) {
  try {
    const auto& program = prepared_->bound.program;
    if (inputs.size() != program.inputs.size())
      return {rejected("model execution input role set is incomplete"), {}};
    std::vector<er::ExecutionValue> values(program.values.size());
    for (const auto& endpoint : program.inputs) {
      const auto found = inputs.find(endpoint.role);
      if (found == inputs.end() || !found->second.valid() ||
          found->second.abi != program.values.at(endpoint.value_index).abi)
        return {rejected("model execution input role or ABI is invalid: " +
                         endpoint.role),
                {}};
      values[endpoint.value_index] = std::move(found->second);
    }
    for (std::size_t index = 0; index < program.operations.size(); ++index) {
      const auto& compiled = program.operations[index];
      std::vector<er::ExecutionValue> operands;
      operands.reserve(compiled.input_values.size());
      for (const auto& binding : compiled.input_values) {
        const auto& value = values.at(binding.value_index);
        if (!value.valid())
          return {rejected("operation input value is unavailable"), {}};
        operands.push_back(value);
      }
      auto handle = provider_->execute(
          *prepared_->operations[index], state_,
          er::OperationInvocation{request_, compiled, operands});
      if (!handle.valid())
        return {rejected("operation provider rejected invocation"), {}};
      std::optional<er::OperationExecutionResult> result;
      while (!(result = handle.poll())) {
      }
      if (!result->status.ok()) return {result->status, {}};
      if (result->outputs.size() != compiled.output_values.size())
        return {{er::ErrorCode::internal,
                 "operation provider returned a partial output set"},
                {}};
      for (std::size_t port = 0; port < compiled.output_values.size(); ++port) {
        const auto slot = compiled.output_values[port].value_index;
        if (!result->outputs[port].valid() ||
            result->outputs[port].abi != program.values.at(slot).abi)
          return {{er::ErrorCode::internal,
                   "operation provider returned an invalid output ABI"},
                  {}};
        values[slot] = std::move(result->outputs[port]);
      }
    }
    Outputs outputs;
    outputs.status = er::Status::success();
    for (const auto& endpoint : program.outputs) {
      if (!values.at(endpoint.value_index).valid())
        return {{er::ErrorCode::internal,
                 "model program did not produce its output: " + endpoint.role},
                {}};
      outputs.values.emplace(endpoint.role, values[endpoint.value_index]);
    }
    return outputs;
  } catch (const std::exception& error) {
    return {{er::ErrorCode::internal,
             std::string("model execution failed: ") + error.what()},
            {}};
  }
}

bool ProgramSession::exact_decode_available() const noexcept {
  return static_cast<bool>(prepared_->exact_decode);
}

er::Status ProgramSession::synchronize_exact_decode_batch(
    std::span<const std::uint32_t> next_tokens,
    std::uint32_t first_target_position, bool produce_final_draft) {
  if (!prepared_->exact_decode)
    return rejected("exact decode service is unavailable");
  for (const auto token : next_tokens)
    if (token >= model_->vocab_size)
      return rejected("exact decode synchronization token is outside the vocabulary");
  return provider_->synchronize_exact_decode_batch(
      *prepared_->exact_decode, state_,
      er::ExactDecodeSynchronizationBatch{request_, next_tokens,
                                          first_target_position,
                                          produce_final_draft});
}

er::ExactDecodeExecutionResult ProgramSession::execute_exact_decode(
    std::uint32_t guaranteed_token, std::uint32_t position,
    std::uint32_t context_limit) {
  const auto failure = [](er::ErrorCode code, std::string message) {
    er::ExactDecodeExecutionResult result;
    result.status = {code, std::move(message)};
    return result;
  };
  try {
    if (!prepared_->exact_decode || !model_->exact_decode_program)
      return failure(er::ErrorCode::invalid_argument,
                     "exact decode service is unavailable");
    if (guaranteed_token >= model_->vocab_size || position >= context_limit)
      return failure(er::ErrorCode::invalid_argument,
                     "exact decode invocation is invalid");
    auto handle = provider_->execute_exact_decode(
        *prepared_->exact_decode, state_,
        er::ExactDecodeInvocation{request_, guaranteed_token, position,
                                  context_limit});
    if (!handle.valid())
      return failure(er::ErrorCode::invalid_argument,
                     "exact decode provider rejected invocation");
    std::optional<er::ExactDecodeExecutionResult> result;
    while (!(result = handle.poll())) {
    }
    if (!result->status.ok()) return std::move(*result);
    // the artifact contract on what a provider may return (:835-851)
    const auto maximum = model_->exact_decode_program->maximum_emitted_tokens;
    const auto count = result->emitted_tokens.size();
    bool sound = count >= 1U && count <= maximum &&
                 result->emitted_tokens.front() == guaranteed_token &&
                 result->positions_advanced == count &&
                 count <= context_limit - position &&
                 result->next_token < model_->vocab_size;
    for (const auto token : result->emitted_tokens)
      sound = sound && token < model_->vocab_size;
    if (!sound)
      return failure(er::ErrorCode::internal,
                     "exact decode provider violated the artifact contract");
    return std::move(*result);
  } catch (const std::exception& error) {
    return failure(er::ErrorCode::internal,
                   std::string("exact decode failed: ") + error.what());
  }
}

}  // namespace qllm
