// Worker process for the MI355X dense FP4 provider: the line protocol of the
// reference's native runner (runtime/tools/moe_vm_runner.cpp, protocol 13) on
// stdin / stdout, so that the service above it (ops/python/expert_server.py,
// CudaWorker :489) talks to this worker unchanged.
//
//   usage: qllm-worker <artifact> --worker --max-context=N --ram-cache-gib=N
//            --vram-cache-gib=N --capacity=1 --kv-cache-mib=N --kv-page-tokens=N
//            --placement-profile=latency|balanced|capacity
//            [--kv-cache-dtype=artifact|q4-f16-per-head|fp16]
//            [--mtp-draft-depth=N] [--routed-vram-policy=fixed]
//
// Start-up follows main() of the runner (:1472-1538): artifact load, the one
// module whose capability table covers the program, registry add + bind,
// preparation of every operation, service contract check, the ready line
// (:577-652).  Commands (worker_loop, :655-1470): PING, BEGIN <id> <context>
// <t,t,...> [SAMPLING <temperature_ppm> <top_p_ppm> <top_k> <min_p_ppm>
// <presence_ppm> <seed>], STEP <id>,<mode>..., NEXT <id> <mode>, CANCEL <id>,
// END <id>, STATS, SHUTDOWN; modes: 0 = decode (an exact-decode step when the
// request is eligible), 1 = emit the pending token and close, 2 = one plain
// program step.  Session retention, parking and persistence are not offered
// (the ready line says so), so RESUME / CHECKPOINT / RETAIN / DROP / SAVE /
// LOAD / PRUNE answer with the runner's "does not support" errors; MULTIMODAL
// needs a program input this provider's programs do not have.  Every failure
// is one {"type":"error"} line; the process keeps serving.
#include "expert/runtime/model_artifact.hpp"
#include "expert/runtime/program_executor.hpp"

#include "artifact_provider.hpp"
#include "dense_fp4_provider.hpp"
#include "program_session.hpp"

#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstring>
#include <filesystem>
#include <iostream>
#include <limits>
#include <map>
#include <memory>
#include <optional>
#include <set>
#include <span>
#include <stdexcept>
#include <string>
#include <string_view>
#include <unordered_map>
#include <vector>

namespace er = expert::runtime;

namespace {

constexpr std::string_view kTokenAbi = "batch.token-id.u32.host.v1";
constexpr std::string_view kPositionAbi = "batch.position.u32.host.v1";

void require(bool condition, std::string_view message) {
  if (!condition) throw std::runtime_error(std::string(message));
}

// ---- launch options (worker_contract.cpp:67-180) ---------------------------

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
};

std::uint64_t unsigned_integer(const std::string& text) {
  require(!text.empty() &&
              std::all_of(text.begin(), text.end(),
                          [](char c) { return c >= '0' && c <= '9'; }) &&
              text.size() <= 19U,
          "invalid worker launch contract: worker option is not an unsigned integer");
  return std::stoull(text);
}

LaunchOptions parse_launch_options(int argc, char** argv) {
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
      "placement-profile", "profile-gpu-phases"};
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

// ---- protocol helpers --------------------------------------------------------

std::vector<std::string_view> split_tabs(std::string_view line) {
  std::vector<std::string_view> fields;
  for (;;) {
    const auto tab = line.find('\t');
    fields.push_back(line.substr(0U, tab));
    if (tab == std::string_view::npos) return fields;
    line.remove_prefix(tab + 1U);
  }
}

std::vector<std::uint32_t> parse_tokens(std::string_view text,
                                        std::uint32_t vocabulary) {
  std::vector<std::uint32_t> tokens;
  while (!text.empty()) {
    const auto comma = text.find(',');
    const auto value = std::stoull(std::string(text.substr(0U, comma)));
    require(value < vocabulary, "token is outside model vocabulary");
    tokens.push_back(static_cast<std::uint32_t>(value));
    if (comma == std::string_view::npos) break;
    text.remove_prefix(comma + 1U);
  }
  return tokens;
}

std::string json_text(std::string_view value) {
  std::string text;
  for (const char c : value) {
    if (c == '"' || c == '\\') {
      text.push_back('\\');
      text.push_back(c);
    } else if (c == '\n' || c == '\r' || c == '\t') {
      text.push_back(' ');
    } else {
      text.push_back(c);
    }
  }
  return text;
}

er::ExecutionValue host_words(std::span<const std::uint32_t> words,
                              std::string_view abi) {
  auto owner = std::make_shared<std::vector<std::uint32_t>>(words.begin(), words.end());
  return {std::string(abi), "host", owner,
          reinterpret_cast<const std::byte*>(owner->data()),
          owner->size() * sizeof(std::uint32_t)};
}

struct Sampling final {
  std::uint32_t temperature_ppm{};
  std::uint32_t top_p_ppm{1000000U};
  std::uint32_t top_k{};
  std::uint32_t min_p_ppm{};
  std::int32_t presence_penalty_ppm{};
  std::uint64_t seed{};
  [[nodiscard]] bool enabled() const noexcept { return temperature_ppm != 0U; }
};

// moe_vm_runner.cpp:318-347
er::ProgramRequestContext request_context(std::uint64_t id, std::uint32_t reserved,
                                          std::uint32_t first_output_position,
                                          const Sampling& sampling, bool exact) {
  er::ProgramRequestContext request;
  request.request_id = id;
  request.parameters.emplace("reserved_context_tokens", reserved);
  request.parameters.emplace("sampling_temperature_ppm", sampling.temperature_ppm);
  request.parameters.emplace("sampling_top_p_ppm", sampling.top_p_ppm);
  request.parameters.emplace("sampling_top_k", sampling.top_k);
  request.parameters.emplace("sampling_min_p_ppm", sampling.min_p_ppm);
  request.parameters.emplace(
      "sampling_presence_penalty_biased_ppm",
      static_cast<std::uint64_t>(
          static_cast<std::int64_t>(sampling.presence_penalty_ppm) + 2'000'000LL));
  request.parameters.emplace("sampling_first_output_position", first_output_position);
  request.parameters.emplace("sampling_seed", sampling.seed);
  request.parameters.emplace("exact_decode_enabled", exact ? 1U : 0U);
  return request;
}

struct Ports final {
  std::string token_input;
  std::string position_input;
  std::string token_output;
};

// :297-316
Ports service_ports(const er::ModelDescriptor& model) {
  Ports ports;
  for (const auto& [role, endpoint] : model.program_inputs) {
    if (endpoint.abi == kTokenAbi) {
      require(ports.token_input.empty(), "multiple token program inputs");
      ports.token_input = role;
    } else if (endpoint.abi == kPositionAbi) {
      require(ports.position_input.empty(), "multiple position program inputs");
      ports.position_input = role;
    }
  }
  for (const auto& [role, endpoint] : model.program_outputs) {
    if (endpoint.abi != kTokenAbi) continue;
    require(ports.token_output.empty(), "multiple token program outputs");
    ports.token_output = role;
  }
  require(!ports.token_input.empty() && !ports.position_input.empty() &&
              !ports.token_output.empty() && model.program_inputs.size() == 2U,
          "artifact does not implement the token-step service ABI");
  return ports;
}

struct ActiveRequest final {
  std::unique_ptr<qllm::ProgramSession> session;
  std::uint32_t predicted{};
  std::uint32_t next_position{};
  std::uint32_t context_limit{};
  Sampling sampling;
};

// :540-568, the checks that apply to a resident provider without retention
void validate_service_contract(const er::ModelDescriptor& model,
                               const er::ExecutionProviderModule& module,
                               const LaunchOptions& options) {
  const auto& service = module.service;
  const auto& provider = module.definition.implementation;
  require(!service.prefill_mode.empty() && service.prefill_chunk_tokens != 0U &&
              provider != nullptr &&
              service.session_retention ==
                  provider->supports_request_state_retention() &&
              service.session_parking ==
                  provider->supports_request_state_parking() &&
              service.session_persistence ==
                  provider->supports_request_state_persistence() &&
              !service.session_parking && service.session_park_ram_bytes == 0U &&
              service.session_park_page_capacity == 0U &&
              !service.request_stream_mode.empty() && !service.rope_mode.empty() &&
              !service.kv_dtype.empty() &&
              (options.kv_cache_dtype == "artifact" ||
               service.kv_dtype == options.kv_cache_dtype) &&
              !service.kv_allocation.empty() &&
              service.kv_page_tokens == options.kv_page_tokens &&
              service.kv_page_bytes != 0U && service.kv_page_capacity != 0U &&
              service.routed_vram_policy == options.routed_vram_policy &&
              service.placement_mode == "resident" &&
              service.placement_profile == "resident" &&
              service.ram_cache_bytes == 0U && service.vram_cache_bytes != 0U &&
              !service.placement_prefetch_enabled &&
              service.placement_minimum_observations == 0U &&
              !service.placement_prefetch_state.empty() &&
              service.mtp_enabled == model.exact_decode_program.has_value() &&
              (!service.mtp_enabled ||
               (service.mtp_resource_available && service.mtp_runtime_ready)),
          "callable provider returned an invalid service contract");
}

// :577-652
void print_ready(const er::ModelDescriptor& model,
                 const er::ExecutionProviderModule::ServiceContract& service,
                 const LaunchOptions& options) {
  const auto flag = [](bool value) { return value ? "true" : "false"; };
  std::uint64_t draft_depth = 0U;
  if (model.exact_decode_program) {
    const auto found = model.exact_decode_program->parameters.find("draft_depth");
    if (found != model.exact_decode_program->parameters.end())
      draft_depth = found->second;
  }
  auto& out = std::cout;
  out << "{\"type\":\"ready\",\"protocol\":13,\"capacity\":" << options.capacity
      << ",\"architecture_id\":\"" << json_text(model.architecture_id)
      << "\",\"vocab_size\":" << model.vocab_size
      << ",\"max_context_tokens\":" << model.max_context_tokens
      << ",\"routed_layers\":0,\"experts_per_layer\":0,\"route_width\":0"
      << ",\"expert_encoding\":\"\",\"operation_capabilities\":[";
  for (std::size_t index = 0; index < model.required_kernels.size(); ++index)
    out << (index ? "," : "") << '"'
        << json_text(model.required_kernels[index].capability) << '"';
  out << "],\"prefill_mode\":\"" << service.prefill_mode
      << "\",\"prefill_chunk_tokens\":" << service.prefill_chunk_tokens
      << ",\"session_retention\":" << flag(service.session_retention)
      << ",\"session_parking\":" << flag(service.session_parking)
      << ",\"session_persistence\":" << flag(service.session_persistence)
      << ",\"session_park_ram_bytes\":" << service.session_park_ram_bytes
      << ",\"session_park_page_capacity\":" << service.session_park_page_capacity
      << ",\"request_stream_mode\":\"" << service.request_stream_mode
      << "\",\"gpu_phase_timing\":" << flag(options.profile_gpu_phases)
      << ",\"sampling_supported\":" << flag(service.sampling_supported)
      << ",\"sampling_presence_penalty_supported\":" << flag(service.sampling_supported)
      << ",\"mtp_resource_available\":" << flag(service.mtp_resource_available)
      << ",\"mtp_runtime_ready\":" << flag(service.mtp_runtime_ready)
      << ",\"mtp_enabled\":" << flag(service.mtp_enabled)
      << ",\"mtp_draft_depth\":" << draft_depth
      << ",\"retain_previous_route\":" << flag(service.retain_previous_route)
      << ",\"cpu_hybrid_enabled\":" << flag(service.cpu_hybrid_enabled)
      << ",\"rope_mode\":\"" << service.rope_mode << "\",\"kv_dtype\":\""
      << service.kv_dtype << "\",\"kv_allocation\":\"" << service.kv_allocation
      << "\",\"kv_page_tokens\":" << service.kv_page_tokens
      << ",\"kv_page_bytes\":" << service.kv_page_bytes
      << ",\"kv_page_capacity\":" << service.kv_page_capacity
      << ",\"placement_mode\":\"" << service.placement_mode
      << "\",\"placement_profile\":\"" << service.placement_profile
      << "\",\"ram_cache_bytes\":" << service.ram_cache_bytes
      << ",\"vram_cache_bytes\":" << service.vram_cache_bytes
      << ",\"routed_vram_policy\":\"" << service.routed_vram_policy << '"'
      << ",\"placement_prefetch_enabled\":"
      << flag(service.placement_prefetch_enabled)
      << ",\"placement_prefetch_state\":\"" << service.placement_prefetch_state
      << "\",\"placement_minimum_observations\":"
      << service.placement_minimum_observations << "}\n"
      << std::flush;
}

int worker_loop(const er::ModelDescriptor& model,
                const er::ExecutionProviderModule& module,
                const qllm::PreparedProgram& prepared,
                const LaunchOptions& options) {
  const auto ports = service_ports(model);
  const auto provider = std::dynamic_pointer_cast<qllm::Mi355DenseFp4Provider>(
      module.definition.implementation);
  require(provider != nullptr, "callable provider module has no implementation");
  std::unordered_map<std::uint64_t, ActiveRequest> active;
  std::uint64_t program_steps{}, program_step_ns{}, useful_tokens{};
  std::uint64_t exact_calls{}, exact_positions{}, exact_accepted{}, cancelled{};
  // :670-676
  const auto exact_eligible = [&](const Sampling& sampling) {
    if (!model.exact_decode_program) return false;
    if (!sampling.enabled()) return true;
    return model.exact_decode_program->abi_version >= 2U && sampling.top_k != 0U &&
           sampling.top_k <= 64U;
  };
  const auto page_count = [&](std::uint32_t tokens) {
    return (std::uint64_t{tokens} + module.service.kv_page_tokens - 1U) /
           module.service.kv_page_tokens;
  };
  print_ready(model, module.service, options);

  // one program step on `tokens` at consecutive positions; the head's token
  const auto run_program = [&](ActiveRequest& request,
                               std::span<const std::uint32_t> tokens,
                               std::uint32_t first_position) {
    std::vector<std::uint32_t> positions(tokens.size());
    for (std::size_t index = 0; index < positions.size(); ++index)
      positions[index] = first_position + static_cast<std::uint32_t>(index);
    std::map<std::string, er::ExecutionValue, std::less<>> inputs;
    inputs.emplace(ports.token_input, host_words(tokens, kTokenAbi));
    inputs.emplace(ports.position_input, host_words(positions, kPositionAbi));
    auto result = request.session->execute(std::move(inputs));
    require(result.status.ok(), result.status.message());
    const auto output = result.values.find(ports.token_output);
    require(output != result.values.end(),
            "model program did not publish its token output");
    const auto& value = output->second;
    require(value.valid() && value.abi == kTokenAbi && value.memory_domain == "host" &&
                value.bytes >= sizeof(std::uint32_t) &&
                value.bytes % sizeof(std::uint32_t) == 0U,
            "callable VM returned an invalid token value");
    std::uint32_t token{};
    std::memcpy(&token, value.data + value.bytes - sizeof(token), sizeof(token));
    return token;
  };

  // The prompt (feed, :679-857).  Long prompts go through the provider's tall
  // prefill, which also feeds the proposer and rolls the first drafts out when
  // the request will be decoded speculatively; short ones take the program in
  // batches of prefill_chunk_tokens with a synchronisation after each.
  const auto feed = [&](ActiveRequest& request,
                        std::span<const std::uint32_t> tokens,
                        std::uint32_t first_position) {
    const auto began = std::chrono::steady_clock::now();
    const bool exact = exact_eligible(request.sampling) &&
                       request.session->exact_decode_available();
    const std::uint32_t chunk =
        std::max<std::uint32_t>(1U, module.service.prefill_chunk_tokens);
    if (tokens.size() > chunk) {
      const auto result = provider->prefill(request.session->state(), tokens,
                                            first_position,
                                            request.session->request());
      require(result.status.ok(), result.status.message());
      request.predicted = result.predicted;
    } else {
      for (std::size_t offset = 0; offset < tokens.size();) {
        const auto count = std::min<std::size_t>(chunk, tokens.size() - offset);
        const auto position = first_position + static_cast<std::uint32_t>(offset);
        request.predicted = run_program(request, tokens.subspan(offset, count), position);
        if (exact) {
          std::vector<std::uint32_t> successors(count);
          for (std::size_t row = 0; row < count; ++row)
            successors[row] = offset + row + 1U == tokens.size()
                                  ? request.predicted
                                  : tokens[offset + row + 1U];
          const auto status = request.session->synchronize_exact_decode_batch(
              successors, position, offset + count == tokens.size());
          require(status.ok(), status.message());
        }
        offset += count;
      }
    }
    program_steps += tokens.size();
    program_step_ns += static_cast<std::uint64_t>(
        std::chrono::duration_cast<std::chrono::nanoseconds>(
            std::chrono::steady_clock::now() - began)
            .count());
    request.next_position = first_position + static_cast<std::uint32_t>(tokens.size());
  };

  std::string line;
  while (std::getline(std::cin, line)) {
    try {
      const auto fields = split_tabs(line);
      require(!fields.empty(), "empty worker command");
      if (fields[0] == "PING") {
        require(fields.size() == 1U, "invalid PING");
        std::cout << "{\"type\":\"pong\"}\n" << std::flush;
      } else if (fields[0] == "BEGIN") {
        require(fields.size() >= 4U, "invalid BEGIN");
        const auto id = std::stoull(std::string(fields[1]));
        const auto context = std::stoull(std::string(fields[2]));
        require(id != 0U && !active.contains(id) && context >= 2U &&
                    context <= options.max_context,
                "invalid BEGIN request identity or context");
        const auto prompt = parse_tokens(fields[3], model.vocab_size);
        require(prompt.size() < context, "prompt exhausts request context");
        std::size_t field = 4U;
        if (field < fields.size() && fields[field] == "RESUME")
          throw std::runtime_error(
              "callable provider does not support session retention");
        require(!prompt.empty(), "fresh BEGIN has no prompt");
        if (field < fields.size() && fields[field] == "MULTIMODAL")
          throw std::runtime_error("artifact does not accept multimodal input");
        if (field < fields.size() && fields[field] == "CHECKPOINT")
          throw std::runtime_error(
              "callable provider does not support session retention");
        Sampling sampling;
        if (field < fields.size() && fields[field] == "SAMPLING") {
          require(field + 6U < fields.size(), "invalid BEGIN sampling marker");
          const auto temperature = std::stoull(std::string(fields[field + 1U]));
          const auto top_p = std::stoull(std::string(fields[field + 2U]));
          const auto top_k = std::stoull(std::string(fields[field + 3U]));
          const auto min_p = std::stoull(std::string(fields[field + 4U]));
          const auto presence = std::stoll(std::string(fields[field + 5U]));
          sampling.seed = std::stoull(std::string(fields[field + 6U]));
          require(temperature <= 2000000U && top_p != 0U && top_p <= 1000000U &&
                      top_k <= model.vocab_size && min_p <= 1000000U &&
                      presence >= -2000000LL && presence <= 2000000LL,
                  "invalid BEGIN sampling values");
          sampling.temperature_ppm = static_cast<std::uint32_t>(temperature);
          sampling.top_p_ppm = static_cast<std::uint32_t>(top_p);
          sampling.top_k = static_cast<std::uint32_t>(top_k);
          sampling.min_p_ppm = static_cast<std::uint32_t>(min_p);
          sampling.presence_penalty_ppm = static_cast<std::int32_t>(presence);
          field += 7U;
        }
        require(field == fields.size(), "unknown BEGIN request fields");
        require(active.size() < options.capacity,
                "callable provider capacity is exhausted");
        ActiveRequest request;
        request.sampling = sampling;
        const auto status = qllm::ProgramSession::begin(
            model, module, prepared,
            request_context(id, static_cast<std::uint32_t>(context),
                            static_cast<std::uint32_t>(prompt.size() - 1U), sampling,
                            exact_eligible(sampling)),
            request.session);
        require(status.ok(), status.message());
        feed(request, prompt, 0U);
        request.context_limit = static_cast<std::uint32_t>(context);
        active.emplace(id, std::move(request));
        std::cout << "{\"type\":\"begun\",\"id\":" << id << "}\n" << std::flush;
      } else if (fields[0] == "STEP" || fields[0] == "NEXT") {
        std::vector<std::pair<std::uint64_t, std::uint32_t>> items;
        std::set<std::uint64_t> unique;
        const auto parse_item = [&](std::string_view item) {
          const auto comma = item.find(',');
          require(comma != std::string_view::npos, "invalid STEP item");
          const auto id = std::stoull(std::string(item.substr(0U, comma)));
          const auto mode = item.substr(comma + 1U);
          require(active.contains(id) && unique.insert(id).second &&
                      (mode == "0" || mode == "1" || mode == "2"),
                  "STEP request mismatch");
          items.emplace_back(id, mode == "1" ? 1U : mode == "2" ? 2U : 0U);
        };
        if (fields[0] == "NEXT") {
          require(fields.size() == 3U, "invalid NEXT");
          parse_item(std::string(fields[1]) + "," + std::string(fields[2]));
        } else {
          require(fields.size() >= 2U && fields.size() <= options.capacity + 1U,
                  "invalid STEP");
          for (std::size_t index = 1U; index < fields.size(); ++index)
            parse_item(fields[index]);
        }
        std::vector<std::vector<std::uint32_t>> emitted(items.size());
        const auto began = std::chrono::steady_clock::now();
        for (std::size_t index = 0; index < items.size(); ++index) {
          const auto [id, mode] = items[index];
          auto& request = active.at(id);
          if (mode == 1U) {
            emitted[index] = {request.predicted};
            continue;
          }
          require(request.next_position < request.context_limit,
                  "request context is exhausted");
          const bool exact = exact_eligible(request.sampling) &&
                             request.session->exact_decode_available();
          if (mode == 0U && exact &&
              request.next_position + 1U < request.context_limit) {
            auto result = request.session->execute_exact_decode(
                request.predicted, request.next_position, request.context_limit);
            require(result.status.ok(), result.status.message());
            emitted[index] = std::move(result.emitted_tokens);
            request.predicted = result.next_token;
            request.next_position += result.positions_advanced;
            program_steps += result.positions_advanced;
            ++exact_calls;
            exact_positions += result.positions_advanced;
            exact_accepted += result.positions_advanced - 1U;
            continue;
          }
          emitted[index] = {request.predicted};
          const std::uint32_t token[1] = {request.predicted};
          request.predicted = run_program(request, token, request.next_position);
          ++request.next_position;
          if (exact) {
            const std::uint32_t successor[1] = {request.predicted};
            const auto status = request.session->synchronize_exact_decode_batch(
                successor, request.next_position - 1U, true);
            require(status.ok(), status.message());
          }
          ++program_steps;
        }
        program_step_ns += static_cast<std::uint64_t>(
            std::chrono::duration_cast<std::chrono::nanoseconds>(
                std::chrono::steady_clock::now() - began)
                .count());
        for (const auto& tokens : emitted) useful_tokens += tokens.size();
        const auto print_tokens = [](const std::vector<std::uint32_t>& tokens) {
          for (std::size_t index = 0; index < tokens.size(); ++index)
            std::cout << (index ? "," : "") << tokens[index];
        };
        if (fields[0] == "NEXT") {
          std::cout << "{\"type\":\"token\",\"id\":" << items[0].first
                    << ",\"tokens\":[";
          print_tokens(emitted[0]);
          std::cout << "]}\n";
        } else {
          std::cout << "{\"type\":\"batch\",\"items\":[";
          for (std::size_t index = 0; index < items.size(); ++index) {
            std::cout << (index ? "," : "") << "{\"id\":" << items[index].first
                      << ",\"tokens\":[";
            print_tokens(emitted[index]);
            std::cout << "]}";
          }
          std::cout << "]}\n";
        }
        std::cout << std::flush;
        for (const auto [id, mode] : items)
          if (mode == 1U) active.erase(id);
      } else if (fields[0] == "CANCEL") {
        require(fields.size() == 2U, "invalid CANCEL");
        if (active.erase(std::stoull(std::string(fields[1])))) ++cancelled;
      } else if (fields[0] == "END") {
        require(fields.size() == 2U || fields.size() == 4U || fields.size() == 6U,
                "invalid END");
        const auto id = std::stoull(std::string(fields[1]));
        const auto found = active.find(id);
        require(found != active.end(), "unknown active request");
        require(fields.size() == 2U,
                "callable provider does not support session retention");
        active.erase(found);
        ++cancelled;
        std::cout << "{\"type\":\"ended\",\"id\":" << id << "}\n" << std::flush;
      } else if (fields[0] == "DROP") {
        require(fields.size() == 2U, "invalid DROP");
        throw std::runtime_error(
            "callable provider does not support session retention");
      } else if (fields[0] == "SAVE" || fields[0] == "LOAD" || fields[0] == "PRUNE") {
        require(fields.size() == (fields[0] == "LOAD" ? 15U : 4U),
                std::string("invalid ") + std::string(fields[0]));
        throw std::runtime_error(
            "callable provider does not support session persistence");
      } else if (fields[0] == "STATS") {
        require(fields.size() == 1U, "invalid STATS");
        std::uint64_t reserved_pages{};
        for (const auto& [id, request] : active)
          reserved_pages += page_count(request.next_position);
        auto telemetry = module.telemetry
                             ? module.telemetry()
                             : std::map<std::string, std::uint64_t, std::less<>>{};
        telemetry["program_steps"] = program_steps;
        telemetry["program_step_ns"] = program_step_ns;
        telemetry["useful_tokens"] = useful_tokens;
        telemetry["exact_decode_calls"] = exact_calls;
        telemetry["exact_decode_positions"] = exact_positions;
        telemetry["exact_decode_accepted_tokens"] = exact_accepted;
        telemetry["cancelled_requests"] = cancelled;
        telemetry["active_requests"] = active.size();
        telemetry["retained_sessions"] = 0U;
        telemetry["parked_sessions"] = 0U;
        telemetry["parked_pages"] = 0U;
        telemetry.try_emplace("kv_allocated_pages", reserved_pages);
        telemetry["kv_reserved_pages"] = reserved_pages;
        std::cout << "{\"type\":\"stats\"";
        for (const auto& [name, value] : telemetry)
          std::cout << ",\"" << json_text(name) << "\":" << value;
        std::cout << "}\n" << std::flush;
      } else if (fields[0] == "SHUTDOWN") {
        require(fields.size() == 1U && active.empty(),
                "SHUTDOWN requires no retained state");
        std::cout << "{\"type\":\"shutdown\"}\n" << std::flush;
        return 0;
      } else {
        throw std::runtime_error("unknown worker command");
      }
    } catch (const std::exception& error) {
      std::cout << "{\"type\":\"error\",\"message\":\"" << json_text(error.what())
                << "\"}\n"
                << std::flush;
    }
  }
  return 0;
}

}  // namespace

int main(int argc, char** argv) {
  try {
    if (argc < 3 || std::string_view(argv[2]) != "--worker") {
      std::cerr << "usage: qllm-worker <artifact> --worker <resource-options>\n";
      return 64;
    }
    const auto options = parse_launch_options(argc, argv);
    const std::filesystem::path root(argv[1]);
    auto artifact = std::make_shared<er::ModelArtifact>();
    auto status = er::ModelArtifact::load(root, *artifact);
    require(status.ok(), status.message());
    if (options.mtp_draft_depth) {
      status = artifact->configure_mtp_draft_depth(*options.mtp_draft_depth);
      require(status.ok(), status.message());
    }
    require(artifact->model().schema_version >= 3U,
            "callable VM service requires a schema v3 artifact");
    // create_module (:431-497): exactly one module must cover the program;
    // this worker links one
    const auto metadata = qllm::make_mi355_dense_fp4_provider();
    require(er::provider_supports_model(artifact->model(), metadata.capabilities).ok(),
            "no callable provider implements the artifact program");
    qllm::ArtifactProviderOptions provider_options;
    provider_options.max_context = options.max_context;
    provider_options.kv_page_tokens = options.kv_page_tokens;
    provider_options.kv_cache_dtype = options.kv_cache_dtype;
    provider_options.vram_cache_bytes = options.vram_cache_gib << 30U;
    provider_options.routed_vram_policy = options.routed_vram_policy;
    require(options.capacity == 1U,
            "this provider serves one request at a time (--capacity=1)");
    auto created = qllm::make_mi355_dense_fp4_module(artifact, provider_options);
    require(created.status.ok(), created.status.message());
    require(created.module.definition.implementation != nullptr,
            "callable provider module has no implementation");
    qllm::PreparedProgram prepared;
    status = qllm::prepare_program(artifact->model(), created.module, prepared);
    require(status.ok(), status.message());
    if (created.module.finalize_service) {
      status = created.module.finalize_service(created.module.service);
      require(status.ok(), status.message());
    }
    validate_service_contract(artifact->model(), created.module, options);
    return worker_loop(artifact->model(), created.module, prepared, options);
  } catch (const std::exception& error) {
    std::cerr << "qllm worker: " << error.what() << '\n';
    return 1;
  }
}
