// C-callable shim over the reference's own host code.  TEST INFRASTRUCTURE
// ONLY.  It is compiled together with the reference source files
// runtime/src/speculative_sampling.cpp (sampling) and
// runtime/src/cpu/fp4_host_executor.cpp (the all-core FP4 x Q8 SwiGLU
// executor), read where they lie in the reference tree, into
// oracle/_ref/libqllm_ref.so.  The shim adds no arithmetic: it only flattens
// std::vector / std::span / exceptions into plain C.
#include "expert/runtime/cpu/fp4_host_executor.hpp"
#include "expert/runtime/speculative_sampling.hpp"

#include <chrono>
#include <memory>

#include <algorithm>
#include <cstdint>
#include <exception>
#include <span>
#include <stdexcept>
#include <string>
#include <vector>

namespace er = expert::runtime;

namespace {

er::SamplingDistribution to_distribution(const std::uint32_t* tokens,
                                         const double* probabilities,
                                         std::uint32_t count) {
  er::SamplingDistribution result;
  result.entries.reserve(count);
  for (std::uint32_t index = 0; index < count; ++index)
    result.entries.push_back({tokens[index], probabilities[index]});
  return result;
}

template <typename Body>
int guarded(Body&& body) {
  try {
    body();
    return 0;
  } catch (const std::invalid_argument&) {
    return 1;
  } catch (const std::exception&) {
    return 2;
  }
}

}  // namespace

extern "C" {

int qref_make_sampling_distribution(const float* sorted_logits,
                                    const std::uint32_t* sorted_tokens,
                                    std::uint32_t count,
                                    std::uint32_t temperature_ppm,
                                    std::uint32_t top_p_ppm,
                                    std::uint32_t min_p_ppm,
                                    std::uint32_t* out_tokens,
                                    double* out_probabilities,
                                    std::uint32_t* out_count) {
  return guarded([&] {
    const auto distribution = er::make_sampling_distribution(
        std::span<const float>(sorted_logits, count),
        std::span<const std::uint32_t>(sorted_tokens, count), temperature_ppm,
        top_p_ppm, min_p_ppm);
    *out_count = static_cast<std::uint32_t>(distribution.entries.size());
    for (std::size_t index = 0; index < distribution.entries.size(); ++index) {
      out_tokens[index] = distribution.entries[index].token;
      out_probabilities[index] = distribution.entries[index].probability;
    }
  });
}

int qref_sample_distribution(const std::uint32_t* tokens,
                             const double* probabilities,
                             std::uint32_t count, double uniform,
                             std::uint32_t* out_token) {
  return guarded([&] {
    *out_token = er::sample_distribution(
        to_distribution(tokens, probabilities, count), uniform);
  });
}

int qref_rejection_sample(std::uint32_t proposal,
                          const std::uint32_t* target_tokens,
                          const double* target_probabilities,
                          std::uint32_t target_count,
                          const std::uint32_t* draft_tokens,
                          const double* draft_probabilities,
                          std::uint32_t draft_count,
                          double acceptance_uniform,
                          double correction_uniform, int* out_accepted,
                          std::uint32_t* out_token,
                          double* out_target_probability,
                          double* out_draft_probability) {
  return guarded([&] {
    const auto decision = er::rejection_sample(
        proposal,
        to_distribution(target_tokens, target_probabilities, target_count),
        to_distribution(draft_tokens, draft_probabilities, draft_count),
        acceptance_uniform, correction_uniform);
    *out_accepted = decision.accepted ? 1 : 0;
    *out_token = decision.token;
    *out_target_probability = decision.target_probability;
    *out_draft_probability = decision.draft_probability;
  });
}

// One dense SwiGLU block, out = down(silu(gate(x)) * up(x)), on `rows` rows with
// the reference's CPU executor (runtime/src/cpu/fp4_host_executor.cpp:397-480):
// ABI-3 weights (E2M1 codes, one UE8M0 scale per 32 columns), Q8 activations.
// `record` holds the six sections at the given byte offsets.  The call is
// repeated `repeats` times; *seconds receives the best wall time of one call.
int qref_fp4_swiglu(const std::uint8_t* record, std::uint64_t record_bytes,
                    const std::uint64_t* offsets /* w1,w1s,w3,w3s,w2,w2s */,
                    std::uint32_t hidden, std::uint32_t intermediate,
                    const float* inputs, std::uint32_t rows, float* outputs,
                    std::uint32_t threads, int bf16_intermediate,
                    std::uint32_t repeats, double* seconds) {
  return guarded([&] {
    static std::unique_ptr<er::cpu::Fp4HostExecutor> executor;
    static std::uint32_t executor_threads = 0;
    static int executor_bf16 = -1;
    if (!executor || executor_threads != threads ||
        executor_bf16 != bf16_intermediate) {
      executor = std::make_unique<er::cpu::Fp4HostExecutor>(
          er::cpu::Fp4HostExecutorConfig{threads, 8U, 8U, 0.0F,
                                         bf16_intermediate != 0, false});
      executor_threads = threads;
      executor_bf16 = bf16_intermediate;
    }
    er::cpu::Fp4HostWorkGroup group;
    group.record_bytes = std::span<const std::byte>(
        reinterpret_cast<const std::byte*>(record), record_bytes);
    const std::uint64_t gate_bytes = std::uint64_t{intermediate} * hidden / 2U;
    const std::uint64_t gate_scales = std::uint64_t{intermediate} * hidden / 32U;
    group.sections = {offsets[0], gate_bytes, offsets[1], gate_scales,
                      offsets[2], gate_bytes, offsets[3], gate_scales,
                      offsets[4], gate_bytes, offsets[5], gate_scales};
    group.hidden = hidden;
    group.intermediate = intermediate;
    for (std::uint32_t row = 0; row < rows; ++row) {
      group.selections.push_back(row);
      group.output_slots.push_back(row);
    }
    double best = 1.0e300;
    for (std::uint32_t repeat = 0; repeat < (repeats ? repeats : 1U); ++repeat) {
      const auto begin = std::chrono::steady_clock::now();
      const auto status = executor->execute(
          std::span<const er::cpu::Fp4HostWorkGroup>(&group, 1U),
          std::span<const float>(inputs, std::size_t{rows} * hidden), rows, 1U,
          std::span<float>(outputs, std::size_t{rows} * hidden));
      const auto end = std::chrono::steady_clock::now();
      if (!status.ok()) throw std::runtime_error(std::string(status.message()));
      best = std::min(best, std::chrono::duration<double>(end - begin).count());
    }
    if (seconds) *seconds = best;
  });
}

double qref_counter_uniform(std::uint64_t seed, std::uint32_t position,
                            std::uint32_t stream, std::uint32_t index) {
  return er::counter_uniform(seed, position, stream, index);
}

}  // extern "C"
