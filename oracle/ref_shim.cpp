// C-callable shim over the reference's own host sampling code.  TEST
// INFRASTRUCTURE ONLY.  It is compiled together with the reference source
// file runtime/src/speculative_sampling.cpp, read where it lies in the
// reference tree, into oracle/_ref/libqllm_ref.so.  The shim adds no
// arithmetic: it only flattens std::vector / exceptions into plain C.
#include "expert/runtime/speculative_sampling.hpp"

#include <cstdint>
#include <exception>
#include <span>
#include <stdexcept>
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

double qref_counter_uniform(std::uint64_t seed, std::uint32_t position,
                            std::uint32_t stream, std::uint32_t index) {
  return er::counter_uniform(seed, position, stream, index);
}

}  // extern "C"
