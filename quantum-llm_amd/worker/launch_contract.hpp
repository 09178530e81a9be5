// The worker's launch contract (runtime/src/worker_contract.cpp:67-180): the
// resource options every worker must be given, in their canonical spelling,
// each at most once; options that belong to one provider are refused.
#pragma once

#include <algorithm>
#include <cstdint>
#include <limits>
#include <map>
#include <optional>
#include <stdexcept>
#include <string>
#include <string_view>

namespace qllm::worker {

inline void require(bool condition, std::string_view message) {
  if (!condition) throw std::runtime_error(std::string(message));
}

struct LaunchOptions final {
  std::uint32_t max_context{};
  std::uint64_t ram_cache_gib{};
  std::uint64_t vram_cache_gib{};
  std::string routed_vram_policy{"fixed"};
  std::uint32_t capacity{};
  std::uint64_t kv_cache_mib{};
  std::uint32_t kv_page_tokens{};
  std::string kv_cache_dtype{"artifact"};
  std::string placement_profile;
  bool profile_gpu_phases{};
  std::optional<std::uint32_t> mtp_draft_depth;
  // the service's ceiling on prompt rows per program step, when it sets one
  std::optional<std::uint32_t> prefill_chunk_limit;
};

inline std::uint64_t unsigned_integer(const std::string& text) {
  require(!text.empty() &&
              std::all_of(text.begin(), text.end(),
                          [](char c) { return c >= '0' && c <= '9'; }) &&
              text.size() <= 19U,
          "invalid worker launch contract: worker option is not an unsigned integer");
  return std::stoull(text);
}

inline LaunchOptions parse_launch_options(int argc, char** argv) {
  std::map<std::string, std::optional<std::string>, std::less<>> raw;
  for (int index = 3; index < argc; ++index) {
    const std::string_view argument(argv[index]);
    require(argument.starts_with("--") && argument.size() > 2U,
            "invalid worker launch contract: worker launch contains a positional "
            "option");
    const auto separator = argument.find('=');
    const auto name = argument.substr(
        2U, separator == std::string_view::npos ? std::string_view::npos
                                                : separator - 2U);
    const auto canonical = [](char c) {
      return (c >= 'a' && c <= 'z') || (c >= '0' && c <= '9') || c == '-';
    };
    require(!name.empty() && name.front() != '-' && name.back() != '-' &&
                std::all_of(name.begin(), name.end(), canonical),
            "invalid worker launch contract: worker option name is not canonical");
    std::optional<std::string> value;
    if (separator != std::string_view::npos) {
      require(separator + 1U < argument.size(),
              "invalid worker launch contract: worker option value is empty");
      value = std::string(argument.substr(separator + 1U));
    }
    require(raw.emplace(std::string(name), std::move(value)).second,
            "invalid worker launch contract: worker option is duplicated");
  }
  const auto value_of = [&](const char* name) -> const std::string& {
    const auto found = raw.find(name);
    require(found != raw.end() && found->second.has_value(),
            std::string("invalid worker launch contract: missing worker option --") +
                name);
    return *found->second;
  };
  const auto u32 = [&](const char* name) {
    const auto value = unsigned_integer(value_of(name));
    require(value != 0U && value <= std::numeric_limits<std::uint32_t>::max(),
            "invalid worker launch contract: worker option is out of range");
    return static_cast<std::uint32_t>(value);
  };
  LaunchOptions options;
  options.max_context = u32("max-context");
  options.ram_cache_gib = unsigned_integer(value_of("ram-cache-gib"));
  options.vram_cache_gib = unsigned_integer(value_of("vram-cache-gib"));
  if (raw.contains("routed-vram-policy"))
    options.routed_vram_policy = value_of("routed-vram-policy");
  options.capacity = u32("capacity");
  options.kv_cache_mib = unsigned_integer(value_of("kv-cache-mib"));
  options.kv_page_tokens = u32("kv-page-tokens");
  if (raw.contains("kv-cache-dtype"))
    options.kv_cache_dtype = value_of("kv-cache-dtype");
  options.placement_profile = value_of("placement-profile");
  if (raw.contains("mtp-draft-depth"))
    options.mtp_draft_depth = u32("mtp-draft-depth");
  require(options.ram_cache_gib != 0U && options.vram_cache_gib != 0U &&
              options.kv_cache_mib != 0U &&
              (options.routed_vram_policy == "fixed" ||
               options.routed_vram_policy == "fit") &&
              (options.placement_profile == "latency" ||
               options.placement_profile == "balanced" ||
               options.placement_profile == "capacity"),
          "invalid worker launch contract: worker resource contract is invalid");
  if (raw.contains("prefill-chunk-limit"))
    options.prefill_chunk_limit = u32("prefill-chunk-limit");
  // a resident decoder places nothing after start-up: read and not used
  if (raw.contains("placement-settle-steps"))
    static_cast<void>(unsigned_integer(value_of("placement-settle-steps")));
  if (const auto found = raw.find("profile-gpu-phases"); found != raw.end()) {
    require(!found->second.has_value(),
            "invalid worker launch contract: boolean worker option "
            "profile-gpu-phases has a value");
    options.profile_gpu_phases = true;
  }
  constexpr std::string_view known[]{
      "max-context",       "ram-cache-gib",      "vram-cache-gib",
      "routed-vram-policy", "capacity",          "kv-cache-mib",
      "kv-page-tokens",    "kv-cache-dtype",     "mtp-draft-depth",
      "placement-profile", "profile-gpu-phases", "prefill-chunk-limit",
      "placement-settle-steps"};
  for (const auto& [name, value] : raw)
    require(std::find(std::begin(known), std::end(known), name) != std::end(known),
            "callable VM service does not accept provider-specific launch flags");
  require(options.ram_cache_gib <= (std::numeric_limits<std::uint64_t>::max() >> 30U) &&
              options.vram_cache_gib <=
                  (std::numeric_limits<std::uint64_t>::max() >> 30U) &&
              options.kv_cache_mib <=
                  (std::numeric_limits<std::uint64_t>::max() >> 20U),
          "worker resource byte count overflows");
  return options;
}

}  // namespace qllm::worker
