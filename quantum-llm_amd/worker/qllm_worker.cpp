// Worker process for the MI355X dense FP4 provider: the line protocol of the
// reference's native runner (runtime/tools/moe_vm_runner.cpp, protocol 13) on
// stdin / stdout, so that the service above it (ops/python/expert_server.py,
// CudaWorker :489) talks to this worker unchanged.
//
//   usage: qllm-worker <artifact> --worker --max-context=N --ram-cache-gib=N
//            --vram-cache-gib=N --capacity=N --kv-cache-mib=N --kv-page-tokens=N
//            --placement-profile=latency|balanced|capacity
//            [--kv-cache-dtype=artifact|q4-f16-per-head|fp16]
//            [--mtp-draft-depth=N] [--routed-vram-policy=fixed]
//            [--prefill-chunk-limit=N] [--profile-gpu-phases]
//
// Structure: Engine is what every request runs on (model, prepared program,
// provider, the program's token ports); Request owns one conversation - its
// program session, the token the model has predicted but not yet emitted, its
// position and limit - and moves it forward by prompt, by speculative step,
// by plain step or by its closing token; Service maps each command verb to a
// handler through a table, reads the handler's arguments with a typed field
// cursor and answers with one JSON line.  Every failure is an
// {"type":"error"} line; the process keeps serving.
//
// Commands: PING, BEGIN <id> <context> <t,t,...> [SAMPLING <temperature_ppm>
// <top_p_ppm> <top_k> <min_p_ppm> <presence_ppm> <seed>], STEP <id>,<mode>...,
// NEXT <id> <mode>, CANCEL <id>, END <id>, STATS, SHUTDOWN; modes: 0 = decode
// (an exact-decode step when the request is eligible), 1 = emit the pending
// token and close, 2 = one plain program step.  Session retention, parking and
// persistence are not offered (the ready line says so), so RESUME / CHECKPOINT
// / RETAIN / DROP / SAVE / LOAD / PRUNE answer with the runner's "does not
// support" errors; MULTIMODAL needs a program input this provider's programs
// do not have.
#include "expert/runtime/model_artifact.hpp"
#include "expert/runtime/program_executor.hpp"

#include "artifact_provider.hpp"
#include "dense_fp4_provider.hpp"
#include "launch_contract.hpp"
#include "program_session.hpp"
#include "wire.hpp"

#include <algorithm>
#include <array>
#include <chrono>
#include <cstdint>
#include <cstring>
#include <filesystem>
#include <iostream>
#include <map>
#include <memory>
#include <span>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

namespace er = expert::runtime;

namespace qllm::worker {
namespace {

using wire::expect;
using wire::FieldCursor;
using wire::JsonLine;

constexpr std::string_view kTokenAbi = "batch.token-id.u32.host.v1";
constexpr std::string_view kPositionAbi = "batch.position.u32.host.v1";
constexpr char kNoRetention[] = "callable provider does not support session retention";
constexpr char kNoPersistence[] =
    "callable provider does not support session persistence";

void expect_ok(const er::Status& status) { expect(status.ok(), status.message()); }

class Stopwatch final {
 public:
  [[nodiscard]] std::uint64_t nanoseconds() const {
    return static_cast<std::uint64_t>(
        std::chrono::duration_cast<std::chrono::nanoseconds>(
            std::chrono::steady_clock::now() - start_)
            .count());
  }

 private:
  std::chrono::steady_clock::time_point start_{std::chrono::steady_clock::now()};
};

// What the worker counts itself; the provider's own telemetry joins it in the
// STATS reply.
struct Counters final {
  std::uint64_t program_steps{};
  std::uint64_t program_step_ns{};
  std::uint64_t useful_tokens{};
  std::uint64_t exact_calls{};
  std::uint64_t exact_positions{};
  std::uint64_t exact_accepted{};
  std::uint64_t cancelled{};
};

// The SAMPLING group of a BEGIN line; without one a request is greedy.
struct SamplingProfile final {
  std::uint32_t temperature_ppm{};
  std::uint32_t top_p_ppm{1000000U};
  std::uint32_t top_k{};
  std::uint32_t min_p_ppm{};
  std::int32_t presence_penalty_ppm{};
  std::uint64_t seed{};

  [[nodiscard]] bool greedy() const noexcept { return temperature_ppm == 0U; }

  static SamplingProfile read(FieldCursor& fields, std::uint32_t vocabulary) {
    expect(fields.left() >= 6U, "invalid BEGIN sampling marker");
    const auto temperature = fields.natural();
    const auto top_p = fields.natural();
    const auto top_k = fields.natural();
    const auto min_p = fields.natural();
    const auto presence = fields.integer();
    SamplingProfile profile;
    profile.seed = fields.natural();
    expect(temperature <= 2000000U && top_p >= 1U && top_p <= 1000000U &&
               top_k <= vocabulary && min_p <= 1000000U && presence >= -2000000 &&
               presence <= 2000000,
           "invalid BEGIN sampling values");
    profile.temperature_ppm = static_cast<std::uint32_t>(temperature);
    profile.top_p_ppm = static_cast<std::uint32_t>(top_p);
    profile.top_k = static_cast<std::uint32_t>(top_k);
    profile.min_p_ppm = static_cast<std::uint32_t>(min_p);
    profile.presence_penalty_ppm = static_cast<std::int32_t>(presence);
    return profile;
  }

  // the request parameters a provider reads (moe_vm_runner.cpp:318-347)
  void publish(std::map<std::string, std::uint64_t, std::less<>>& parameters) const {
    parameters["sampling_temperature_ppm"] = temperature_ppm;
    parameters["sampling_top_p_ppm"] = top_p_ppm;
    parameters["sampling_top_k"] = top_k;
    parameters["sampling_min_p_ppm"] = min_p_ppm;
    parameters["sampling_presence_penalty_biased_ppm"] = static_cast<std::uint64_t>(
        std::int64_t{presence_penalty_ppm} + 2'000'000);
    parameters["sampling_seed"] = seed;
  }
};

enum class StepMode : std::uint8_t { decode = 0, finish = 1, plain = 2 };

[[nodiscard]] StepMode step_mode(std::string_view text) {
  expect(text.size() == 1U && text[0] >= '0' && text[0] <= '2',
         "STEP request mismatch");
  return static_cast<StepMode>(text[0] - '0');
}

// The model, its prepared program and the provider behind it: shared by all
// requests, changed by none.
class Engine final {
 public:
  Engine(const er::ModelDescriptor& model, const er::ExecutionProviderModule& module,
         const PreparedProgram& prepared, const LaunchOptions& options)
      : model_(model), module_(module), prepared_(prepared) {
    provider_ = std::dynamic_pointer_cast<Mi355DenseFp4Provider>(
        module.definition.implementation);
    expect(provider_ != nullptr, "callable provider module has no implementation");
    find_ports();
    chunk_ = std::max<std::uint32_t>(1U, module.service.prefill_chunk_tokens);
    if (options.prefill_chunk_limit)
      chunk_ = std::min(chunk_, *options.prefill_chunk_limit);
  }

  [[nodiscard]] const er::ModelDescriptor& model() const noexcept { return model_; }
  [[nodiscard]] const er::ExecutionProviderModule& module() const noexcept {
    return module_;
  }
  [[nodiscard]] const PreparedProgram& prepared() const noexcept { return prepared_; }
  [[nodiscard]] Mi355DenseFp4Provider& provider() const noexcept { return *provider_; }
  [[nodiscard]] std::uint32_t chunk_tokens() const noexcept { return chunk_; }

  // Whether a request with this profile may be decoded speculatively
  // (moe_vm_runner.cpp:670-676): greedy always, sampled only through the
  // version-2 exact-decode contract with a top-k the device selection serves.
  [[nodiscard]] bool speculative(const SamplingProfile& profile) const noexcept {
    const auto& decode = model_.exact_decode_program;
    if (!decode) return false;
    if (profile.greedy()) return true;
    return decode->abi_version >= 2U && profile.top_k >= 1U && profile.top_k <= 64U;
  }

  // One pass of the program over `tokens` at first_position, first_position +
  // 1, ...; returns the token the head selected for the last row.
  [[nodiscard]] std::uint32_t run(ProgramSession& session,
                                  std::span<const std::uint32_t> tokens,
                                  std::uint32_t first_position) const {
    std::vector<std::uint32_t> positions(tokens.size());
    for (std::uint32_t row = 0U; row < positions.size(); ++row)
      positions[row] = first_position + row;
    std::map<std::string, er::ExecutionValue, std::less<>> inputs;
    inputs.emplace(token_input_, words(tokens, kTokenAbi));
    inputs.emplace(position_input_, words(positions, kPositionAbi));
    auto outputs = session.execute(std::move(inputs));
    expect_ok(outputs.status);
    const auto found = outputs.values.find(token_output_);
    expect(found != outputs.values.end(),
           "model program did not publish its token output");
    const er::ExecutionValue& value = found->second;
    expect(value.valid() && value.abi == kTokenAbi && value.memory_domain == "host" &&
               value.bytes != 0U && value.bytes % sizeof(std::uint32_t) == 0U,
           "callable VM returned an invalid token value");
    std::uint32_t last{};
    std::memcpy(&last, value.data + (value.bytes - sizeof(last)), sizeof(last));
    return last;
  }

 private:
  static er::ExecutionValue words(std::span<const std::uint32_t> values,
                                  std::string_view abi) {
    auto storage =
        std::make_shared<std::vector<std::uint32_t>>(values.begin(), values.end());
    const auto* bytes = reinterpret_cast<const std::byte*>(storage->data());
    return {std::string(abi), "host", storage, bytes,
            storage->size() * sizeof(std::uint32_t)};
  }

  // The token-step service ABI (moe_vm_runner.cpp:297-316): exactly a token
  // and a position input and one token output.
  void find_ports() {
    const auto claim = [](std::string& port, const std::string& role,
                          std::string_view complaint) {
      expect(port.empty(), complaint);
      port = role;
    };
    for (const auto& [role, endpoint] : model_.program_inputs) {
      if (endpoint.abi == kTokenAbi)
        claim(token_input_, role, "multiple token program inputs");
      else if (endpoint.abi == kPositionAbi)
        claim(position_input_, role, "multiple position program inputs");
    }
    for (const auto& [role, endpoint] : model_.program_outputs)
      if (endpoint.abi == kTokenAbi)
        claim(token_output_, role, "multiple token program outputs");
    expect(model_.program_inputs.size() == 2U && !token_input_.empty() &&
               !position_input_.empty() && !token_output_.empty(),
           "artifact does not implement the token-step service ABI");
  }

  const er::ModelDescriptor& model_;
  const er::ExecutionProviderModule& module_;
  const PreparedProgram& prepared_;
  std::shared_ptr<Mi355DenseFp4Provider> provider_;
  std::string token_input_, position_input_, token_output_;
  std::uint32_t chunk_{1U};
};

// One conversation.  `pending_` is the token the model has chosen for
// position `position_` and the service has not been given yet.
class Request final {
 public:
  Request(const Engine& engine, std::uint64_t id, std::uint32_t context_limit,
          const SamplingProfile& profile, std::size_t prompt_tokens)
      : engine_(engine), limit_(context_limit), speculative_(engine.speculative(profile)) {
    er::ProgramRequestContext context;
    context.request_id = id;
    context.parameters["reserved_context_tokens"] = context_limit;
    context.parameters["sampling_first_output_position"] = prompt_tokens - 1U;
    context.parameters["exact_decode_enabled"] = speculative_ ? 1U : 0U;
    profile.publish(context.parameters);
    expect_ok(ProgramSession::begin(engine.model(), engine.module(), engine.prepared(),
                                    std::move(context), session_));
    speculative_ = speculative_ && session_->exact_decode_available();
  }

  [[nodiscard]] std::uint32_t position() const noexcept { return position_; }

  // The prompt (the runner's feed, moe_vm_runner.cpp:679-857).  Prompts longer
  // than one program batch take the provider's tall prefill, which also feeds
  // the proposer and rolls the first drafts out; short ones walk the program
  // batch by batch and tell the proposer each batch's successors.
  void ingest(std::span<const std::uint32_t> prompt, Counters& counters) {
    const Stopwatch watch;
    const std::size_t batch = engine_.chunk_tokens();
    if (prompt.size() > batch && engine_.provider().supports_tall_prefill()) {
      const auto result = engine_.provider().prefill(session_->state(), prompt,
                                                     position_, session_->request());
      expect_ok(result.status);
      pending_ = result.predicted;
    } else {
      for (std::size_t done = 0U; done < prompt.size(); done += batch) {
        const auto rows = prompt.subspan(done, std::min(batch, prompt.size() - done));
        const auto first = position_ + static_cast<std::uint32_t>(done);
        pending_ = engine_.run(*session_, rows, first);
        if (!speculative_) continue;
        // row r's successor is the next prompt token; the last row's is the
        // head's prediction
        std::vector<std::uint32_t> successors(rows.begin() + 1, rows.end());
        const bool last = done + rows.size() == prompt.size();
        successors.push_back(last ? pending_ : prompt[done + rows.size()]);
        expect_ok(session_->synchronize_exact_decode_batch(successors, first, last));
      }
    }
    position_ += static_cast<std::uint32_t>(prompt.size());
    counters.program_steps += prompt.size();
    counters.program_step_ns += watch.nanoseconds();
  }

  // The tokens one step hands to the service.
  [[nodiscard]] std::vector<std::uint32_t> advance(StepMode mode, Counters& counters) {
    if (mode == StepMode::finish) return {pending_};
    expect(position_ < limit_, "request context is exhausted");
    // a verify step needs room for the guaranteed token and one more
    if (mode == StepMode::decode && speculative_ && position_ + 1U < limit_)
      return verify(counters);
    // the position is taken once the program has run: a proposer that cannot
    // follow (its rollout would start past the context) fails the step, and
    // the request still stands one token further
    const std::uint32_t emitted = pending_;
    const std::uint32_t here = position_;
    pending_ = engine_.run(*session_, {&emitted, 1U}, here);
    position_ = here + 1U;
    if (speculative_)
      expect_ok(session_->synchronize_exact_decode_batch({&pending_, 1U}, here, true));
    ++counters.program_steps;
    return {emitted};
  }

 private:
  std::vector<std::uint32_t> verify(Counters& counters) {
    auto result = session_->execute_exact_decode(pending_, position_, limit_);
    expect_ok(result.status);
    pending_ = result.next_token;
    position_ += result.positions_advanced;
    counters.program_steps += result.positions_advanced;
    counters.exact_calls += 1U;
    counters.exact_positions += result.positions_advanced;
    counters.exact_accepted += result.positions_advanced - 1U;
    return std::move(result.emitted_tokens);
  }

  const Engine& engine_;
  std::unique_ptr<ProgramSession> session_;
  std::uint32_t pending_{};
  std::uint32_t position_{};
  std::uint32_t limit_{};
  bool speculative_{};
};

// The service contract a resident provider without retention must return
// (moe_vm_runner.cpp:540-568).
void check_service_contract(const er::ModelDescriptor& model,
                            const er::ExecutionProviderModule& module,
                            const LaunchOptions& options) {
  const auto& s = module.service;
  const auto* provider = module.definition.implementation.get();
  const bool retention_agrees =
      provider != nullptr &&
      s.session_retention == provider->supports_request_state_retention() &&
      s.session_parking == provider->supports_request_state_parking() &&
      s.session_persistence == provider->supports_request_state_persistence() &&
      !s.session_parking && s.session_park_ram_bytes == 0U &&
      s.session_park_page_capacity == 0U;
  const bool kv_agrees =
      !s.kv_dtype.empty() && !s.kv_allocation.empty() &&
      (options.kv_cache_dtype == "artifact" || s.kv_dtype == options.kv_cache_dtype) &&
      s.kv_page_tokens == options.kv_page_tokens && s.kv_page_bytes != 0U &&
      s.kv_page_capacity != 0U;
  const bool placement_agrees =
      s.placement_mode == "resident" && s.placement_profile == "resident" &&
      s.routed_vram_policy == options.routed_vram_policy && s.ram_cache_bytes == 0U &&
      s.vram_cache_bytes != 0U && !s.placement_prefetch_enabled &&
      s.placement_minimum_observations == 0U && !s.placement_prefetch_state.empty();
  const bool mtp_agrees =
      s.mtp_enabled == model.exact_decode_program.has_value() &&
      (!s.mtp_enabled || (s.mtp_resource_available && s.mtp_runtime_ready));
  require(!s.prefill_mode.empty() && s.prefill_chunk_tokens != 0U &&
              !s.request_stream_mode.empty() && !s.rope_mode.empty() &&
              retention_agrees && kv_agrees && placement_agrees && mtp_agrees,
          "callable provider returned an invalid service contract");
}

class Service final {
 public:
  Service(const Engine& engine, const LaunchOptions& options)
      : engine_(engine), options_(options) {}

  int serve(std::istream& in, std::ostream& out) {
    out_ = &out;
    announce();
    std::string line;
    while (open_ && std::getline(in, line)) {
      try {
        dispatch(line);
      } catch (const std::exception& error) {
        JsonLine("error").string("message", error.what()).send(out);
      }
    }
    return 0;
  }

 private:
  using Handler = void (Service::*)(FieldCursor&);
  struct Command final {
    std::string_view verb;
    Handler handler;
  };
  void dispatch(std::string_view line) {
    static constexpr std::array<Command, 12> kCommands{{
        {"PING", &Service::ping},
        {"BEGIN", &Service::begin},
        {"STEP", &Service::step},
        {"NEXT", &Service::next},
        {"CANCEL", &Service::cancel},
        {"END", &Service::end},
        {"DROP", &Service::drop},
        {"SAVE", &Service::persistence},
        {"LOAD", &Service::persistence},
        {"PRUNE", &Service::persistence},
        {"STATS", &Service::stats},
        {"SHUTDOWN", &Service::shutdown},
    }};
    FieldCursor fields(line);
    verb_ = fields.text();
    for (const auto& command : kCommands)
      if (command.verb == verb_) return (this->*command.handler)(fields);
    wire::fail("unknown worker command");
  }

  // the ready line: every field the service's worker client reads
  // (ops/python/expert_server.py:575-700)
  void announce() {
    const auto& model = engine_.model();
    const auto& s = engine_.module().service;
    std::uint64_t draft_depth = 0U;
    if (const auto& decode = model.exact_decode_program)
      if (const auto found = decode->parameters.find("draft_depth");
          found != decode->parameters.end())
        draft_depth = found->second;
    std::vector<std::string> capabilities;
    for (const auto& kernel : model.required_kernels)
      capabilities.push_back(kernel.capability);
    JsonLine("ready")
        .number("protocol", 13U)
        .number("capacity", options_.capacity)
        .string("architecture_id", model.architecture_id)
        .number("vocab_size", model.vocab_size)
        .number("max_context_tokens", model.max_context_tokens)
        .number("routed_layers", 0U)
        .number("experts_per_layer", 0U)
        .number("route_width", 0U)
        .string("expert_encoding", "")
        .strings("operation_capabilities", capabilities)
        .string("prefill_mode", s.prefill_mode)
        .number("prefill_chunk_tokens", engine_.chunk_tokens())
        .boolean("session_retention", s.session_retention)
        .boolean("session_parking", s.session_parking)
        .boolean("session_persistence", s.session_persistence)
        .number("session_park_ram_bytes", s.session_park_ram_bytes)
        .number("session_park_page_capacity", s.session_park_page_capacity)
        .string("request_stream_mode", s.request_stream_mode)
        .boolean("gpu_phase_timing", engine_.provider().profiles_gpu_phases())
        .boolean("sampling_supported", s.sampling_supported)
        .boolean("sampling_presence_penalty_supported", s.sampling_supported)
        .boolean("mtp_resource_available", s.mtp_resource_available)
        .boolean("mtp_runtime_ready", s.mtp_runtime_ready)
        .boolean("mtp_enabled", s.mtp_enabled)
        .number("mtp_draft_depth", draft_depth)
        .boolean("retain_previous_route", s.retain_previous_route)
        .boolean("cpu_hybrid_enabled", s.cpu_hybrid_enabled)
        .string("rope_mode", s.rope_mode)
        .string("kv_dtype", s.kv_dtype)
        .string("kv_allocation", s.kv_allocation)
        .number("kv_page_tokens", s.kv_page_tokens)
        .number("kv_page_bytes", s.kv_page_bytes)
        .number("kv_page_capacity", s.kv_page_capacity)
        .string("placement_mode", s.placement_mode)
        .string("placement_profile", s.placement_profile)
        .number("ram_cache_bytes", s.ram_cache_bytes)
        .number("vram_cache_bytes", s.vram_cache_bytes)
        .string("routed_vram_policy", s.routed_vram_policy)
        .boolean("placement_prefetch_enabled", s.placement_prefetch_enabled)
        .string("placement_prefetch_state", s.placement_prefetch_state)
        .number("placement_minimum_observations", s.placement_minimum_observations)
        .send(*out_);
  }

  void ping(FieldCursor& fields) {
    expect(fields.done(), "invalid PING");
    JsonLine("pong").send(*out_);
  }

  // BEGIN <id> <context> <tokens> [RESUME ..|MULTIMODAL ..|CHECKPOINT ..]
  //       [SAMPLING t p k m presence seed]
  void begin(FieldCursor& fields) {
    expect(fields.left() >= 3U, "invalid BEGIN");
    const auto id = fields.natural();
    const auto context = fields.natural();
    expect(id != 0U && requests_.find(id) == requests_.end() && context >= 2U &&
               context <= options_.max_context,
           "invalid BEGIN request identity or context");
    const auto prompt = wire::token_list(fields.text(), engine_.model().vocab_size);
    expect(prompt.size() < context, "prompt exhausts request context");
    if (fields.keyword("RESUME")) wire::fail(kNoRetention);
    expect(!prompt.empty(), "fresh BEGIN has no prompt");
    if (fields.keyword("MULTIMODAL"))
      wire::fail("artifact does not accept multimodal input");
    if (fields.keyword("CHECKPOINT")) wire::fail(kNoRetention);
    SamplingProfile profile;
    if (fields.keyword("SAMPLING"))
      profile = SamplingProfile::read(fields, engine_.model().vocab_size);
    expect(fields.done(), "unknown BEGIN request fields");
    expect(requests_.size() < options_.capacity,
           "callable provider capacity is exhausted");
    auto request = std::make_unique<Request>(
        engine_, id, static_cast<std::uint32_t>(context), profile, prompt.size());
    request->ingest(prompt, counters_);
    requests_.emplace(id, std::move(request));
    JsonLine("begun").number("id", id).send(*out_);
  }

  struct Turn final {
    std::uint64_t id{};
    StepMode mode{};
    std::vector<std::uint32_t> emitted;
  };

  Turn turn(std::string_view id_text, std::string_view mode_text,
            std::span<const Turn> earlier) const {
    Turn next;
    next.id = wire::decimal<std::uint64_t>(id_text);
    const bool repeated = std::any_of(
        earlier.begin(), earlier.end(),
        [&](const Turn& other) { return other.id == next.id; });
    expect(!repeated && requests_.find(next.id) != requests_.end(),
           "STEP request mismatch");
    next.mode = step_mode(mode_text);
    return next;
  }

  // runs the turns in order, then retires the requests that emitted their
  // closing token
  void take_turns(std::vector<Turn>& turns) {
    const Stopwatch watch;
    for (auto& item : turns)
      item.emitted = requests_.at(item.id)->advance(item.mode, counters_);
    counters_.program_step_ns += watch.nanoseconds();
    for (const auto& item : turns) counters_.useful_tokens += item.emitted.size();
  }

  void retire(std::span<const Turn> turns) {
    for (const auto& item : turns)
      if (item.mode == StepMode::finish) requests_.erase(item.id);
  }

  // STEP <id>,<mode> [<id>,<mode> ...]: one batch reply for all of them
  void step(FieldCursor& fields) {
    expect(fields.left() >= 1U && fields.left() <= options_.capacity, "invalid STEP");
    std::vector<Turn> turns;
    while (!fields.done()) {
      const auto item = fields.text();
      const auto comma = item.find(',');
      expect(comma != std::string_view::npos, "invalid STEP item");
      turns.push_back(turn(item.substr(0U, comma), item.substr(comma + 1U), turns));
    }
    take_turns(turns);
    JsonLine reply("batch");
    reply.begin_items("items");
    for (const auto& item : turns) reply.item(item.id, item.emitted);
    reply.end_items().send(*out_);
    retire(turns);
  }

  // NEXT <id> <mode>: the single-request form, answered with a token line
  void next(FieldCursor& fields) {
    expect(fields.left() == 2U, "invalid NEXT");
    const auto id_text = fields.text();
    std::vector<Turn> turns{turn(id_text, fields.text(), {})};
    take_turns(turns);
    JsonLine("token").number("id", turns[0].id).numbers("tokens", turns[0].emitted)
        .send(*out_);
    retire(turns);
  }

  // CANCEL <id>: no reply line; an unknown id is not an error (the request
  // may have ended on its own meanwhile)
  void cancel(FieldCursor& fields) {
    expect(fields.left() == 1U, "invalid CANCEL");
    counters_.cancelled += requests_.erase(fields.natural());
  }

  // END <id> [RETAIN <key> [AT <tokens>]]
  void end(FieldCursor& fields) {
    expect(fields.left() == 1U || fields.left() == 3U || fields.left() == 5U,
           "invalid END");
    const auto id = fields.natural();
    const auto found = requests_.find(id);
    expect(found != requests_.end(), "unknown active request");
    expect(fields.done(), kNoRetention);
    requests_.erase(found);
    ++counters_.cancelled;
    JsonLine("ended").number("id", id).send(*out_);
  }

  void drop(FieldCursor& fields) {
    expect(fields.left() == 1U, "invalid DROP");
    wire::fail(kNoRetention);
  }

  // SAVE / PRUNE <a> <b> <c>, LOAD with its fourteen fields
  void persistence(FieldCursor& fields) {
    const std::size_t arguments = verb_ == "LOAD" ? 14U : 3U;
    expect(fields.left() == arguments, "invalid " + std::string(verb_));
    wire::fail(kNoPersistence);
  }

  void stats(FieldCursor& fields) {
    expect(fields.done(), "invalid STATS");
    const std::uint64_t page_tokens = engine_.module().service.kv_page_tokens;
    std::uint64_t reserved_pages = 0U;
    for (const auto& [id, request] : requests_)
      reserved_pages += (request->position() + page_tokens - 1U) / page_tokens;
    std::map<std::string, std::uint64_t, std::less<>> figures;
    if (engine_.module().telemetry) figures = engine_.module().telemetry();
    figures.try_emplace("kv_allocated_pages", reserved_pages);
    const std::pair<const char*, std::uint64_t> own[] = {
        {"program_steps", counters_.program_steps},
        {"program_step_ns", counters_.program_step_ns},
        {"useful_tokens", counters_.useful_tokens},
        {"exact_decode_calls", counters_.exact_calls},
        {"exact_decode_positions", counters_.exact_positions},
        {"exact_decode_accepted_tokens", counters_.exact_accepted},
        {"cancelled_requests", counters_.cancelled},
        {"active_requests", requests_.size()},
        {"retained_sessions", 0U},
        {"parked_sessions", 0U},
        {"parked_pages", 0U},
        {"kv_reserved_pages", reserved_pages},
    };
    for (const auto& [name, value] : own) figures[name] = value;
    JsonLine reply("stats");
    for (const auto& [name, value] : figures) reply.number(name, value);
    reply.send(*out_);
  }

  void shutdown(FieldCursor& fields) {
    expect(fields.done() && requests_.empty(), "SHUTDOWN requires no retained state");
    JsonLine("shutdown").send(*out_);
    open_ = false;
  }

  const Engine& engine_;
  const LaunchOptions& options_;
  std::ostream* out_{};
  std::string_view verb_;
  std::map<std::uint64_t, std::unique_ptr<Request>> requests_;
  Counters counters_;
  bool open_{true};
};

int run(int argc, char** argv) {
  const auto options = parse_launch_options(argc, argv);
  auto artifact = std::make_shared<er::ModelArtifact>();
  expect_ok(er::ModelArtifact::load(std::filesystem::path(argv[1]), *artifact));
  if (options.mtp_draft_depth)
    expect_ok(artifact->configure_mtp_draft_depth(*options.mtp_draft_depth));
  const er::ModelDescriptor& model = artifact->model();
  require(model.schema_version >= 3U,
          "callable VM service requires a schema v3 artifact");
  // exactly one module must cover the program (moe_vm_runner.cpp:431-497);
  // this worker links one
  require(er::provider_supports_model(model,
                                      make_mi355_dense_fp4_provider().capabilities)
              .ok(),
          "no callable provider implements the artifact program");
  ArtifactProviderOptions provider_options;
  provider_options.max_context = options.max_context;
  provider_options.capacity = options.capacity;
  provider_options.kv_page_tokens = options.kv_page_tokens;
  provider_options.kv_cache_dtype = options.kv_cache_dtype;
  provider_options.vram_cache_bytes = options.vram_cache_gib << 30U;
  provider_options.routed_vram_policy = options.routed_vram_policy;
  provider_options.profile_gpu_phases = options.profile_gpu_phases;
  auto created = make_mi355_dense_fp4_module(artifact, provider_options);
  expect_ok(created.status);
  PreparedProgram prepared;
  expect_ok(prepare_program(model, created.module, prepared));
  if (created.module.finalize_service)
    expect_ok(created.module.finalize_service(created.module.service));
  check_service_contract(model, created.module, options);
  const Engine engine(model, created.module, prepared, options);
  return Service(engine, options).serve(std::cin, std::cout);
}

}  // namespace
}  // namespace qllm::worker

int main(int argc, char** argv) {
  if (argc < 3 || std::string_view(argv[2]) != "--worker") {
    std::cerr << "usage: qllm-worker <artifact> --worker <resource-options>\n";
    return 64;
  }
  try {
    return qllm::worker::run(argc, argv);
  } catch (const std::exception& error) {
    std::cerr << "qllm worker: " << error.what() << '\n';
    return 1;
  }
}
