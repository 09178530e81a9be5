// Host-side sampling mathematics of the verify step, double precision with
// the summation orders of the reference
// (runtime/include/expert/runtime/speculative_sampling.hpp, same four
// functions; runtime/src/speculative_sampling.cpp).
#pragma once

#include <cstdint>
#include <span>
#include <vector>

namespace expert::runtime {

struct TokenProbability final {
  std::uint32_t token{};
  double probability{};
};

struct SamplingDistribution final {
  std::vector<TokenProbability> entries;
  [[nodiscard]] double probability(std::uint32_t token) const noexcept;
};

[[nodiscard]] SamplingDistribution make_sampling_distribution(
    std::span<const float> sorted_logits,
    std::span<const std::uint32_t> sorted_tokens,
    std::uint32_t temperature_ppm, std::uint32_t top_p_ppm,
    std::uint32_t min_p_ppm);

[[nodiscard]] std::uint32_t sample_distribution(
    const SamplingDistribution& distribution, double uniform);

struct RejectionSamplingResult final {
  bool accepted{};
  std::uint32_t token{};
  double target_probability{};
  double draft_probability{};
};

[[nodiscard]] RejectionSamplingResult rejection_sample(
    std::uint32_t proposal, const SamplingDistribution& target,
    const SamplingDistribution& draft, double acceptance_uniform,
    double correction_uniform);

[[nodiscard]] double counter_uniform(std::uint64_t seed,
                                     std::uint32_t position,
                                     std::uint32_t stream,
                                     std::uint32_t index = 0U) noexcept;

}  // namespace expert::runtime
