#include "expert/runtime/speculative_sampling.hpp"

#include <algorithm>
#include <cmath>
#include <stdexcept>

namespace expert::runtime {
namespace {

// A distribution is usable when it is non-empty, finite, non-negative, has no
// repeated token and sums to one within 1e-10
// (runtime/src/speculative_sampling.cpp:25-41).
void check_distribution(const SamplingDistribution& distribution) {
  const auto& entries = distribution.entries;
  if (entries.empty())
    throw std::invalid_argument("sampling distribution is empty");
  double mass = 0.0;
  std::vector<std::uint32_t> seen;
  seen.reserve(entries.size());
  for (const auto& [token, probability] : entries) {
    if (!(probability >= 0.0) || !std::isfinite(probability))
      throw std::invalid_argument("sampling probability is invalid");
    mass += probability;
    seen.push_back(token);
  }
  std::sort(seen.begin(), seen.end());
  const bool repeated =
      std::adjacent_find(seen.begin(), seen.end()) != seen.end();
  if (repeated || !std::isfinite(mass) || std::abs(mass - 1.0) > 1e-10)
    throw std::invalid_argument("sampling distribution is not normalized");
}

void check_uniform(double u) {
  if (!(u >= 0.0 && u < 1.0))
    throw std::invalid_argument("sampling uniform must be in [0, 1)");
}

}  // namespace

double SamplingDistribution::probability(std::uint32_t token) const noexcept {
  for (const auto& entry : entries)
    if (entry.token == token) return entry.probability;
  return 0.0;
}

// speculative_sampling.cpp:52-111
SamplingDistribution make_sampling_distribution(
    std::span<const float> sorted_logits,
    std::span<const std::uint32_t> sorted_tokens,
    std::uint32_t temperature_ppm, std::uint32_t top_p_ppm,
    std::uint32_t min_p_ppm) {
  const std::size_t count = sorted_logits.size();
  const bool bad_arguments =
      count == 0 || sorted_tokens.size() != count || temperature_ppm == 0 ||
      temperature_ppm > 2'000'000U || top_p_ppm == 0 ||
      top_p_ppm > 1'000'000U || min_p_ppm > 1'000'000U ||
      !std::isfinite(sorted_logits[0]);
  if (bad_arguments)
    throw std::invalid_argument("invalid sorted sampling candidates");
  for (std::size_t i = 1; i < count; ++i) {
    const float before = sorted_logits[i - 1];
    const float here = sorted_logits[i];
    const bool rises = !std::isnan(here) && here > before;
    const bool tie_out_of_order =
        here == before && sorted_tokens[i] < sorted_tokens[i - 1];
    if (rises || tie_out_of_order)
      throw std::invalid_argument("sampling candidates are not ordered");
  }

  const double beta = 1'000'000.0 / static_cast<double>(temperature_ppm);
  const double top = static_cast<double>(sorted_logits[0]);
  const double floor_weight = static_cast<double>(min_p_ppm) / 1'000'000.0;
  SamplingDistribution kept;
  kept.entries.reserve(count);
  double mass = 0.0;
  for (std::size_t i = 0; i < count; ++i) {
    const double logit = static_cast<double>(sorted_logits[i]);
    const double weight =
        std::isfinite(logit) ? std::exp((logit - top) * beta) : 0.0;
    if (weight < floor_weight) continue;
    kept.entries.push_back({sorted_tokens[i], weight});
    mass += weight;
  }
  if (kept.entries.empty() || !std::isfinite(mass) || !(mass > 0.0))
    throw std::invalid_argument("sampling distribution has no retained mass");

  // nucleus: shortest prefix whose running share reaches top_p (inclusive)
  const double top_p = static_cast<double>(top_p_ppm) / 1'000'000.0;
  std::size_t nucleus = kept.entries.size();
  double running = 0.0;
  for (std::size_t i = 0; i < kept.entries.size(); ++i) {
    running += kept.entries[i].probability / mass;
    if (running >= top_p) {
      nucleus = i + 1;
      break;
    }
  }
  kept.entries.resize(nucleus);
  double nucleus_mass = 0.0;
  for (const auto& entry : kept.entries) nucleus_mass += entry.probability;
  for (auto& entry : kept.entries) entry.probability /= nucleus_mass;
  return kept;
}

// speculative_sampling.cpp:113-123
std::uint32_t sample_distribution(const SamplingDistribution& distribution,
                                  double uniform) {
  check_distribution(distribution);
  check_uniform(uniform);
  double running = 0.0;
  for (const auto& entry : distribution.entries) {
    running += entry.probability;
    if (uniform < running) return entry.token;
  }
  return distribution.entries.back().token;
}

// speculative_sampling.cpp:125-171.  The residual max(p - q, 0) is walked in
// ascending token id; a sorted vector of (token, value) stands in for the
// reference's ordered map.
RejectionSamplingResult rejection_sample(
    std::uint32_t proposal, const SamplingDistribution& target,
    const SamplingDistribution& draft, double acceptance_uniform,
    double correction_uniform) {
  check_distribution(target);
  check_distribution(draft);
  check_uniform(acceptance_uniform);
  check_uniform(correction_uniform);
  const double p = target.probability(proposal);
  const double q = draft.probability(proposal);
  if (!(q > 0.0))
    throw std::invalid_argument("proposal has zero draft probability");
  if (acceptance_uniform < std::min(1.0, p / q)) return {true, proposal, p, q};

  struct Item {
    std::uint32_t token;
    double value;
    bool from_draft;
  };
  std::vector<Item> items;
  items.reserve(target.entries.size() + draft.entries.size());
  for (const auto& entry : target.entries)
    items.push_back({entry.token, entry.probability, false});
  for (const auto& entry : draft.entries)
    items.push_back({entry.token, entry.probability, true});
  std::stable_sort(items.begin(), items.end(),
                   [](const Item& a, const Item& b) { return a.token < b.token; });
  std::vector<TokenProbability> residual;
  residual.reserve(items.size());
  for (std::size_t i = 0; i < items.size();) {
    double value = 0.0;
    std::size_t j = i;
    for (; j < items.size() && items[j].token == items[i].token; ++j)
      value = items[j].from_draft ? std::max(0.0, value - items[j].value)
                                  : items[j].value;
    residual.push_back({items[i].token, value});
    i = j;
  }
  double mass = 0.0;
  for (const auto& entry : residual) mass += entry.probability;
  if (!std::isfinite(mass) || !(mass > 0.0))
    throw std::runtime_error("rejected proposal has no correction mass");
  const double threshold = correction_uniform * mass;
  double running = 0.0;
  std::uint32_t last_positive = 0;
  bool any_positive = false;
  for (const auto& entry : residual) {
    if (entry.probability > 0.0) {
      last_positive = entry.token;
      any_positive = true;
    }
    running += entry.probability;
    if (threshold < running) return {false, entry.token, p, q};
  }
  if (!any_positive)
    throw std::runtime_error("rejected proposal has no positive correction");
  return {false, last_positive, p, q};
}

// speculative_sampling.cpp:13-18,173-182
double counter_uniform(std::uint64_t seed, std::uint32_t position,
                       std::uint32_t stream, std::uint32_t index) noexcept {
  std::uint64_t z = seed ^ (std::uint64_t{position} * 0xd2b74407b1ce6e93ULL) ^
                    (std::uint64_t{stream} * 0xca5a826395121157ULL) ^
                    (std::uint64_t{index} * 0x9e3779b185ebca87ULL);
  z += 0x9e3779b97f4a7c15ULL;
  z = (z ^ (z >> 30U)) * 0xbf58476d1ce4e5b9ULL;
  z = (z ^ (z >> 27U)) * 0x94d049bb133111ebULL;
  z ^= z >> 31U;
  return static_cast<double>(z >> 11U) * 0x1p-53;
}

}  // namespace expert::runtime
