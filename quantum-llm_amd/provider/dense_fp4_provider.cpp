#include "dense_fp4_provider.hpp"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <bit>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <stdexcept>

namespace qllm {
namespace {

constexpr std::uint32_t kMaximumGpuSamplingTopK = 64U;  // provider.cpp:8359
constexpr std::uint32_t kMaximumDraftDepth = 7U;

void hip_check(hipError_t error, const char* what) {
  if (error != hipSuccess)
    throw std::runtime_error(std::string(what) + ": " +
                             hipGetErrorString(error));
}

void status_check(std::int32_t status) {
  if (status != QLLM_OK) throw std::runtime_error(qllm_last_error());
}

std::uint32_t pad32(std::uint32_t value) { return (value + 31U) / 32U * 32U; }

// A device allocation that is freed unless release() hands it on.
class DeviceBuffer final {
 public:
  DeviceBuffer(std::size_t bytes, const char* what) {
    hip_check(hipMalloc(&pointer_, bytes), what);
  }
  ~DeviceBuffer() {
    if (pointer_) (void)hipFree(pointer_);
  }
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  [[nodiscard]] void* get() const noexcept { return pointer_; }
  [[nodiscard]] void* release() noexcept {
    void* pointer = pointer_;
    pointer_ = nullptr;
    return pointer;
  }

 private:
  void* pointer_{};
};

std::uint64_t request_parameter(const er::ProgramRequestContext& request,
                                std::string_view name) {
  const auto found = request.parameters.find(name);
  if (found == request.parameters.end())
    throw std::runtime_error("request parameter is absent: " +
                             std::string(name));
  return found->second;
}

// The penalty a request asks for: the parameter is biased by 2,000,000 ppm so
// that negative penalties travel as unsigned values
// (runtime/tools/moe_vm_runner.cpp:318-347, dense_fp4_provider.cpp:8336-8341).
double presence_penalty_of(const er::ProgramRequestContext& request) {
  const auto biased =
      request_parameter(request, "sampling_presence_penalty_biased_ppm");
  if (biased > 4'000'000U)
    throw std::runtime_error("sampling presence penalty is invalid");
  return (static_cast<double>(biased) - 2'000'000.0) / 1'000'000.0;
}

er::ExactDecodeExecutionHandle completed_exact(
    er::ExactDecodeExecutionResult result) {
  auto shared = std::make_shared<std::optional<er::ExactDecodeExecutionResult>>(
      std::move(result));
  return er::ExactDecodeExecutionHandle::from_callbacks(
      [shared]() {
        auto value = std::move(*shared);
        shared->reset();
        return value;
      },
      [shared]() { shared->reset(); });
}

const er::ImmutableModelTensor& tensor_for(
    std::span<const er::PreparedTensorBinding> tensors, std::string_view role) {
  for (const auto& binding : tensors)
    if (binding.role == role && binding.tensor) return *binding.tensor;
  throw std::runtime_error("tensor role is not bound: " + std::string(role));
}

const er::ImmutableModelTensor* optional_tensor(
    std::span<const er::PreparedTensorBinding> tensors, std::string_view role) {
  for (const auto& binding : tensors)
    if (binding.role == role && binding.tensor) return binding.tensor.get();
  return nullptr;
}

// The role the artifact compiler binds (compiler/expert_pack/adapters.py:
// 1422-1602: "weight", "input_norm", "norm"), or the longer name that hosts
// without an artifact use for the same tensor.
const er::ImmutableModelTensor& tensor_for_either(
    std::span<const er::PreparedTensorBinding> tensors, std::string_view role,
    std::string_view other_role) {
  if (const auto* tensor = optional_tensor(tensors, role)) return *tensor;
  if (const auto* tensor = optional_tensor(tensors, other_role)) return *tensor;
  throw std::runtime_error("tensor role is not bound: " + std::string(role));
}

// Value ABIs between operations as the artifact declares them
// (dense_fp4_provider.cpp:59-74).  The hidden-state ABI string names F32 rows
// in device memory; the memory domain says whose device.
constexpr std::string_view kHiddenAbi = "batch.hidden.f32.cuda.v1";
constexpr std::string_view kTokenAbi = "batch.token-id.u32.host.v1";
constexpr std::string_view kPositionAbi = "batch.position.u32.host.v1";
constexpr std::string_view kDeviceDomain = "hip.device";

// :550-564
std::span<const std::uint32_t> host_u32_batch(const er::ExecutionValue& value,
                                              std::string_view abi,
                                              std::string_view description) {
  if (!value.valid() || value.abi != abi || value.memory_domain != "host" ||
      value.bytes % sizeof(std::uint32_t) != 0U ||
      value.bytes / sizeof(std::uint32_t) > 1024U ||
      reinterpret_cast<std::uintptr_t>(value.data) % alignof(std::uint32_t) != 0U)
    throw std::runtime_error(std::string(description) + " ABI mismatch");
  return {reinterpret_cast<const std::uint32_t*>(value.data),
          static_cast<std::size_t>(value.bytes / sizeof(std::uint32_t))};
}

// :5605-5620
er::OperationExecutionHandle completed_operation(
    er::OperationExecutionResult result) {
  auto shared = std::make_shared<std::optional<er::OperationExecutionResult>>(
      std::move(result));
  return er::OperationExecutionHandle::from_callbacks(
      [shared]() {
        auto value = std::move(*shared);
        shared->reset();
        return value;
      },
      [shared]() { shared->reset(); });
}

er::Status validate_parameters(
    const std::map<std::string, std::uint64_t, std::less<>>& parameters) {
  for (const auto& [name, value] : parameters) {
    if (name.size() > 9 && name.ends_with("_f32_bits")) {
      const auto number =
          std::bit_cast<float>(static_cast<std::uint32_t>(value));
      if (!std::isfinite(number) || !(number > 0.0F))
        return {er::ErrorCode::invalid_argument,
                "float parameter is not finite and positive: " + name};
    }
  }
  return er::Status::success();
}

}  // namespace

// What prepare() leaves behind for execute() (PreparedOperation,
// dense_fp4_provider.cpp:2273-2291): which block this is, where its inputs sit
// in an invocation and which output ports, with which ABI, it must fill.
struct Mi355DenseFp4Provider::PreparedOperation final : er::IPreparedOperation {
  enum class Kind { embedding, attention, ffn, head, exact_decode };
  Kind kind{};
  std::string capability;
  std::uint32_t abi_version{};
  std::uint32_t logical_operation{};
  std::uint32_t layer{};   // attention / ffn: index among the blocks of its kind
  std::map<std::string, std::size_t, std::less<>> input_indices;
  std::vector<std::pair<std::string, std::string>> outputs;
};

er::WorkerProviderDefinition make_mi355_dense_fp4_provider() {
  const auto validator = [](const er::ModelDescriptor& model) {
    return validate_dense_fp4_descriptor(model);
  };
  // The capability strings the dense Qwen-style program requires
  // (dense_fp4_provider.cpp:996-1052; emitted by
  // compiler/expert_pack/adapters.py:1682-1697) plus the block-16 variants.
  return {"mi355-dense-fp4",
          200U,
          {{"embedding.lookup.fp4-block32.v1", 1U, 1U, validator},
           {"dense.activation-input.bfloat16.v1", 1U, 1U, validator},
           {"block.full-attention.output-gated.v1", 1U, 1U, validator},
           {"block.full-attention.standard-gqa.v1", 1U, 1U, validator},
           {"ffn.swiglu.dense.fp4-block32.v1", 1U, 1U, validator},
           {"head.rmsnorm.token-select.fp4-block32.v1", 1U, 1U, validator},
           {"decode.mtp.dense-full-attention.fp4-block32.exact.v2", 2U, 2U,
            validator},
           {"embedding.lookup.fp4-f16-block16.v1", 1U, 1U, validator},
           {"ffn.swiglu.dense.fp4-f16-block16.v1", 1U, 1U, validator},
           {"head.rmsnorm.token-select.fp4-f16-block16.v1", 1U, 1U, validator},
           {"decode.mtp.dense-full-attention.fp4-f16-block16.exact.v2", 2U, 2U,
            validator}},
          nullptr};
}

Mi355DenseFp4Provider::Mi355DenseFp4Provider(const DenseGeometry& geometry)
    : g_(geometry) {
  const bool bad =
      !g_.hidden || !g_.intermediate || !g_.layers || !g_.query_heads ||
      !g_.kv_heads || g_.query_heads % g_.kv_heads || !g_.vocabulary ||
      (g_.head_dim != 128U && g_.head_dim != 256U) || !g_.rotary_dim ||
      g_.rotary_dim > g_.head_dim || g_.rotary_dim % 2U ||
      !g_.kv_page_tokens || g_.kv_page_tokens % 64U || !g_.max_context ||
      g_.draft_depth == 0U || g_.draft_depth > kMaximumDraftDepth || g_.hidden % 64U ||
      g_.intermediate % 64U || (g_.query_heads * g_.head_dim) % 64U ||
      g_.scale_scheme > QLLM_SCALE_F16_BLOCK16 ||
      !(g_.norm_epsilon > 0.0F) || !(g_.rope_theta > 0.0F) ||
      g_.mtp_layers > 1U;
  if (bad) throw std::invalid_argument("dense FP4 geometry is not supported");
  if (g_.draft_vocabulary == 0U)
    g_.draft_vocabulary = std::min<std::uint32_t>(g_.vocabulary, 65536U);
  if (g_.mtp_layers &&
      (g_.draft_vocabulary > g_.vocabulary || g_.draft_vocabulary % 32U))
    throw std::invalid_argument(
        "draft vocabulary must be a multiple of 32 within the vocabulary");
  if (g_.kv_encoding == KvEncoding::fp16 &&
      g_.query_heads / g_.kv_heads > 16U)
    throw std::invalid_argument("exact F16 KV supports at most 16 grouped heads");
  // what one attention workgroup holds: three 16-row tiles of (row, grouped
  // query head) pairs, two at head_dim 256 - for every cache kind
  if ((g_.draft_depth + 1U) * (g_.query_heads / g_.kv_heads) >
      (g_.head_dim == 256U ? 32U : 48U))
    throw std::invalid_argument(
        "(draft_depth + 1) * (query_heads / kv_heads) exceeds the attention "
        "kernels' 48 rows (32 at head_dim 256)");
  hipStream_t stream{};
  hip_check(hipStreamCreate(&stream), "create provider stream");
  stream_ = stream;
  device_lifetime_ = std::make_shared<std::uint8_t>(std::uint8_t{0});
  layers_.resize(g_.layers);
  accepted_depth_calls_.assign(g_.draft_depth + 1U, 0U);
  max_rows_ = g_.draft_depth + 1U;
  try {
    allocate_workspaces();
  } catch (...) {
    release();
    throw;
  }
}

Mi355DenseFp4Provider::~Mi355DenseFp4Provider() { release(); }

void Mi355DenseFp4Provider::release() {
  for (void* graph : graphs_)
    if (graph) (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph));
  graphs_.clear();
  for (void* graph : mtp_graphs_)
    if (graph) (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph));
  mtp_graphs_.clear();
  if (stream_) (void)hipStreamSynchronize(static_cast<hipStream_t>(stream_));
  for (void* pointer : allocations_) (void)hipFree(pointer);
  allocations_.clear();
  for (void* pointer : prefill_allocations_) (void)hipFree(pointer);
  prefill_allocations_.clear();
  if (staging_) {
    (void)hipHostFree(staging_);
    staging_ = nullptr;
  }
  for (auto& slot : slots_)
    for (void* page : slot.pages)
      if (page) (void)hipFree(page);
  slots_.clear();
  for (auto& events : gpu_event_pool_) {
    (void)hipEventDestroy(static_cast<hipEvent_t>(events.start));
    (void)hipEventDestroy(static_cast<hipEvent_t>(events.stop));
  }
  gpu_event_pool_.clear();
  if (stream_) {
    (void)hipStreamDestroy(static_cast<hipStream_t>(stream_));
    stream_ = nullptr;
  }
}

std::uint64_t Mi355DenseFp4Provider::kv_bytes_per_token_layer() const noexcept {
  if (g_.kv_encoding == KvEncoding::fp16)
    return std::uint64_t{g_.kv_heads} * g_.head_dim * 2U * 2U;
  return std::uint64_t{g_.kv_heads} * 2U * (g_.head_dim / 2U + 2U);
}

void Mi355DenseFp4Provider::allocate_workspaces() {
  const auto device_alloc = [this](std::size_t bytes) {
    void* pointer{};
    hip_check(hipMalloc(&pointer, bytes), "allocate provider workspace");
    allocations_.push_back(pointer);
    return pointer;
  };
  const std::size_t rows = max_rows_;
  const std::size_t query_width =
      std::size_t{g_.query_heads} * g_.head_dim * (g_.output_gated ? 2U : 1U);
  const std::size_t kv_width = std::size_t{g_.kv_heads} * g_.head_dim;
  const std::size_t widest =
      std::max<std::size_t>({g_.hidden, g_.intermediate,
                             std::size_t{g_.query_heads} * g_.head_dim});
  // tokens (up to 8) and the four position words of a pass lie side by side,
  // so that one copy from pinned host memory uploads both
  tokens_ = static_cast<std::uint32_t*>(device_alloc((8U + 4U) * 4U));
  positions_ = tokens_ + 8U;
  {
    void* pinned = nullptr;
    hip_check(hipHostMalloc(&pinned, sizeof(HostStaging), hipHostMallocDefault),
              "allocate pinned staging");
    staging_ = static_cast<HostStaging*>(pinned);
    *staging_ = HostStaging{};
  }
  graphs_.assign(max_rows_ + 1U, nullptr);
  if (const char* eager = std::getenv("QLLM_PROVIDER_EAGER"))
    use_graphs_ = eager[0] == '0';
  if (g_.profile_gpu_phases) use_graphs_ = false;
  hidden_ = static_cast<float*>(device_alloc(rows * g_.hidden * 4U));
  // read by the proposer when a stream is synchronised before any target pass
  hip_check(hipMemset(hidden_, 0, rows * g_.hidden * 4U), "clear hidden state");
  normalized_ = static_cast<std::uint16_t*>(device_alloc(rows * widest * 2U));
  query_ = static_cast<float*>(device_alloc(rows * query_width * 4U));
  key_ = static_cast<float*>(device_alloc(rows * kv_width * 4U));
  value_ = static_cast<float*>(device_alloc(rows * kv_width * 4U));
  attention_ = static_cast<std::uint16_t*>(
      device_alloc(rows * g_.query_heads * g_.head_dim * 2U));
  activation_ =
      static_cast<std::uint16_t*>(device_alloc(rows * g_.intermediate * 2U));
  logits_ = static_cast<float*>(device_alloc(rows * g_.vocabulary * 4U));
  // The o and down projections have too few rows to occupy the GPU: K is cut
  // over projection_splits_ workgroups per tile and the norm that follows
  // adds the partials to the residual stream.
  if (const char* text = std::getenv("QLLM_PROVIDER_K_SPLITS"))
    projection_splits_ = static_cast<std::uint32_t>(
        std::clamp(std::atoi(text), 0, 16));
  if (g_.hidden % 4U != 0U || g_.hidden > 16384U) projection_splits_ = 0U;
  if (projection_splits_ > 1U)
    projection_partials_ = static_cast<float*>(
        device_alloc(projection_splits_ * rows * g_.hidden * 4U));

  if (g_.activation_q8) {
    if (g_.scale_scheme != QLLM_SCALE_UE8M0_BLOCK32 || g_.hidden % 64U != 0U ||
        g_.intermediate % 64U != 0U ||
        (std::size_t{g_.query_heads} * g_.head_dim) % 64U != 0U)
      throw std::invalid_argument(
          "Q8 activations need block-32 UE8M0 weights and projection widths "
          "that are multiples of 64");
    const std::size_t columns = std::max(widest, std::size_t{2U} * g_.hidden);
    q8_ = static_cast<std::int8_t*>(device_alloc(rows * columns));
    q8_scales_ = static_cast<float*>(device_alloc(rows * 4U));
    activation_f32_ = static_cast<float*>(device_alloc(rows * columns * 4U));
    if (g_.mtp_layers)
      mtp_fusion_f32_ =
          static_cast<float*>(device_alloc(rows * 2U * g_.hidden * 4U));
    // (q/k/v is never cut here: its rows go through the rotary as they are)
    qkv_splits_ = 0U;
  }
  // counters and partial sums of the balanced q/k/v and gate/up launches
  // (zeroed once; the kernels leave the counters at zero)
  gemm_workspace_bytes_ = qllm_fp4_gemm_balance_workspace_bytes();
  gemm_workspace_ = device_alloc(gemm_workspace_bytes_);
  hip_check(hipMemset(gemm_workspace_, 0, gemm_workspace_bytes_),
            "clear GEMM balance workspace");

  if (const char* text = std::getenv("QLLM_PROVIDER_QKV_SPLITS"))
    qkv_splits_ =
        static_cast<std::uint32_t>(std::clamp(std::atoi(text), 0, 16));
  if (g_.kv_encoding != KvEncoding::q4_f16_per_head || g_.activation_q8)
    qkv_splits_ = 0U;
  if (qkv_splits_ > 1U)
    qkv_partials_ = static_cast<float*>(device_alloc(
        qkv_splits_ * rows * (query_width + 2U * kv_width) * 4U));

  // Context splits: kv_heads * splits workgroups fill the 256 CUs; the
  // attention kernels deal the context's tiles evenly over them themselves
  // (split_tokens 0), whatever the context length.
  const std::uint32_t wanted_splits =
      std::max(1U, 256U / std::max(1U, g_.kv_heads));
  split_tokens_ = 0U;
  maximum_splits_ =
      std::min(wanted_splits, std::max(1U, (g_.max_context + 511U) / 512U));
  const std::size_t partials = rows * maximum_splits_ * g_.query_heads;
  partial_maxima_ = static_cast<float*>(device_alloc(partials * 4U));
  partial_sums_ = static_cast<float*>(device_alloc(partials * 4U));
  partial_outputs_ =
      static_cast<float*>(device_alloc(partials * g_.head_dim * 4U));
  if (g_.kv_encoding == KvEncoding::q4_f16_per_head) {
    // The rotary kernel hands the attention kernel its query operands (two
    // int8 planes in matrix-core order and the row scales).  Rows past the
    // batch are never written: they stay zero.
    const std::size_t operand_bytes = qllm_q4h_query_operand_bytes(
        max_rows_, g_.query_heads, g_.kv_heads, g_.head_dim);
    const std::size_t scale_bytes = std::size_t{g_.kv_heads} * 3U * 16U * 4U;
    query_operands_ = static_cast<std::int8_t*>(device_alloc(operand_bytes));
    query_operand_scales_ = static_cast<float*>(device_alloc(scale_bytes));
    hip_check(hipMemset(query_operands_, 0, operand_bytes),
              "clear query operands");
    hip_check(hipMemset(query_operand_scales_, 0, scale_bytes),
              "clear query operand scales");
    // (cos, sin) of a batch's rotary angles, computed once per pass
    rope_table_ = static_cast<float*>(
        device_alloc(std::size_t{max_rows_} * g_.rotary_dim * 4U));
  }

  // the heads' tile maxima: 32 vocabulary rows per tile
  const std::size_t head_maxima_bytes =
      (std::size_t{g_.vocabulary} + 31U) / 32U * max_rows_ * 8U;
  select_workspace_bytes_ = std::max(
      std::max(head_maxima_bytes,
               qllm_argmax_workspace_bytes(g_.vocabulary, max_rows_)),
      std::max(qllm_topk_workspace_bytes(g_.vocabulary, kMaximumGpuSamplingTopK),
               qllm_topk_batch_workspace_bytes(g_.vocabulary,
                                               kMaximumGpuSamplingTopK, max_rows_)));
  select_workspace_ = device_alloc(select_workspace_bytes_);
  argmax_tokens_ = static_cast<std::uint32_t*>(device_alloc(rows * 4U));
  presence_ = static_cast<std::uint8_t*>(device_alloc(g_.vocabulary));
  proposal_presence_ = static_cast<std::uint8_t*>(device_alloc(g_.vocabulary));
  hip_check(hipMemset(presence_, 0, g_.vocabulary), "clear presence bytes");
  hip_check(hipMemset(proposal_presence_, 0, g_.vocabulary),
            "clear presence bytes");
  mark_tokens_ = static_cast<std::uint32_t*>(device_alloc(8U * 4U));
  // top-k logits of up to 8 rows, then their tokens: one buffer, one readback
  top_logits_ = static_cast<float*>(
      device_alloc(8U * kMaximumGpuSamplingTopK * (4U + 4U)));
  top_tokens_ = reinterpret_cast<std::uint32_t*>(
      top_logits_ + 8U * kMaximumGpuSamplingTopK);

  if (g_.mtp_layers) {
    mtp_tokens_ = static_cast<std::uint32_t*>(device_alloc((8U + 4U) * 4U));
    mtp_positions_ = mtp_tokens_ + 8U;
    mtp_embedding_ = static_cast<float*>(device_alloc(rows * g_.hidden * 4U));
    mtp_fusion_input_ =
        static_cast<std::uint16_t*>(device_alloc(rows * 2U * g_.hidden * 2U));
    mtp_hidden_ = static_cast<float*>(device_alloc(rows * g_.hidden * 4U));
    mtp_last_hidden_ = static_cast<float*>(device_alloc(g_.hidden * 4U));
    hip_check(hipMemset(mtp_last_hidden_, 0, g_.hidden * 4U),
              "clear proposer hidden state");
    mtp_logits_ = static_cast<float*>(device_alloc(g_.draft_vocabulary * 4U));
    mtp_argmax_ = static_cast<std::uint32_t*>(device_alloc(4U));
    mtp_draft_tokens_ =
        static_cast<std::uint32_t*>(device_alloc(kMaximumDraftDepth * 4U));
    // a captured pass at 2 * rows + chained, then the captured greedy rollouts
    // (first pass of `rows` rows + drafts - 1 chained single-row passes) at
    // 2 * (max_rows + 1) + rows * (kMaximumDraftDepth + 1) + drafts
    mtp_graphs_.assign(2U * (max_rows_ + 1U) +
                           (max_rows_ + 1U) * (kMaximumDraftDepth + 1U),
                       nullptr);
  }

  // Page geometry: every page holds all target layers back to back, then the
  // proposer's Q8 layer (dense_fp4_provider.cpp:2582-2599, 2690-2759,
  // 6554-6588).
  kv_page_bytes_ = kv_bytes_per_token_layer() * g_.kv_page_tokens * g_.layers;
  mtp_page_offset_ = (kv_page_bytes_ + 15U) & ~std::uint64_t{15U};
  if (g_.mtp_layers)
    kv_page_bytes_ = mtp_page_offset_ +
                     qllm_q8_layer_bytes(g_.kv_page_tokens, g_.kv_heads, g_.head_dim);
  const std::size_t page_count =
      (g_.max_context + g_.kv_page_tokens - 1U) / g_.kv_page_tokens;
  slots_.resize(std::max(1U, g_.capacity));
  for (auto& slot : slots_) {
    slot.leased = std::make_shared<std::atomic<bool>>(false);
    slot.pages.assign(page_count, nullptr);
    if (slots_.size() > 1U) {
      slot.saved_presence = static_cast<std::uint8_t*>(device_alloc(g_.vocabulary));
      hip_check(hipMemset(slot.saved_presence, 0, g_.vocabulary),
                "clear slot presence bytes");
      if (g_.mtp_layers) {
        slot.saved_last_hidden = static_cast<float*>(device_alloc(g_.hidden * 4U));
        hip_check(hipMemset(slot.saved_last_hidden, 0, g_.hidden * 4U),
                  "clear slot proposer state");
      }
    }
  }
  device_page_table_ =
      static_cast<void**>(device_alloc(page_count * sizeof(void*)));
  hip_check(hipMemset(device_page_table_, 0, page_count * sizeof(void*)),
            "clear device page table");
}

// Makes `slot` the one whose pages, presence bytes and proposer state the
// kernels address.  Everything is ordered on the provider's stream, so work
// already enqueued for the outgoing slot still sees its own table.
void Mi355DenseFp4Provider::activate(std::uint32_t slot) {
  if (slot >= slots_.size()) throw std::runtime_error("request slot is invalid");
  if (slot == active_slot_) return;
  const auto stream = static_cast<hipStream_t>(stream_);
  auto& outgoing = slots_[active_slot_];
  auto& incoming = slots_[slot];
  hip_check(hipMemcpyAsync(outgoing.saved_presence, presence_, g_.vocabulary,
                           hipMemcpyDeviceToDevice, stream),
            "save request presence bytes");
  hip_check(hipMemcpyAsync(presence_, incoming.saved_presence, g_.vocabulary,
                           hipMemcpyDeviceToDevice, stream),
            "load request presence bytes");
  if (mtp_last_hidden_) {
    hip_check(hipMemcpyAsync(outgoing.saved_last_hidden, mtp_last_hidden_,
                             g_.hidden * 4U, hipMemcpyDeviceToDevice, stream),
              "save proposer state");
    hip_check(hipMemcpyAsync(mtp_last_hidden_, incoming.saved_last_hidden,
                             g_.hidden * 4U, hipMemcpyDeviceToDevice, stream),
              "load proposer state");
  }
  // a pageable source: the copy has read it when the call returns
  hip_check(hipMemcpyAsync(device_page_table_, incoming.pages.data(),
                           incoming.pages.size() * sizeof(void*),
                           hipMemcpyHostToDevice, stream),
            "load request page table");
  active_slot_ = slot;
}

// ---- GPU phase timing (dense_fp4_provider.cpp:5691-5738) ---------------------
// An event pair per operation of a pass, from a pool that grows on demand; the
// pass's last operation reads them all back and adds each to its phase's total.
std::size_t Mi355DenseFp4Provider::begin_gpu_phase(GpuPhase phase) {
  if (!g_.profile_gpu_phases) return ~std::size_t{0};
  if (active_gpu_events_ == gpu_event_pool_.size()) {
    hipEvent_t start{}, stop{};
    hip_check(hipEventCreate(&start), "create GPU phase start event");
    if (const auto status = hipEventCreate(&stop); status != hipSuccess) {
      (void)hipEventDestroy(start);
      hip_check(status, "create GPU phase stop event");
    }
    gpu_event_pool_.push_back({start, stop, phase});
  }
  auto& events = gpu_event_pool_[active_gpu_events_];
  events.phase = phase;
  hip_check(hipEventRecord(static_cast<hipEvent_t>(events.start),
                           static_cast<hipStream_t>(stream_)),
            "record GPU phase start");
  return active_gpu_events_++;
}

void Mi355DenseFp4Provider::end_gpu_phase(std::size_t index) {
  if (!g_.profile_gpu_phases) return;
  if (index >= active_gpu_events_)
    throw std::runtime_error("GPU phase event index is invalid");
  hip_check(hipEventRecord(static_cast<hipEvent_t>(gpu_event_pool_[index].stop),
                           static_cast<hipStream_t>(stream_)),
            "record GPU phase stop");
}

void Mi355DenseFp4Provider::collect_gpu_phases() {
  if (!g_.profile_gpu_phases || active_gpu_events_ == 0U) return;
  hip_check(hipEventSynchronize(static_cast<hipEvent_t>(
                gpu_event_pool_[active_gpu_events_ - 1U].stop)),
            "synchronize GPU phase events");
  for (std::size_t index = 0; index < active_gpu_events_; ++index) {
    const auto& events = gpu_event_pool_[index];
    float milliseconds{};
    hip_check(hipEventElapsedTime(&milliseconds,
                                  static_cast<hipEvent_t>(events.start),
                                  static_cast<hipEvent_t>(events.stop)),
              "read GPU phase elapsed time");
    gpu_phase_ns_[static_cast<std::size_t>(events.phase)] +=
        static_cast<std::uint64_t>(std::llround(double{milliseconds} * 1.0e6));
  }
  active_gpu_events_ = 0U;
  ++gpu_measured_batches_;
}

void Mi355DenseFp4Provider::ensure_pages(std::uint32_t last_position) {
  auto& pages = slots_[active_slot_].pages;
  const std::size_t last_page = last_position / g_.kv_page_tokens;
  if (last_page >= pages.size())
    throw std::runtime_error("KV position exceeds the configured context");
  for (std::size_t page = 0; page <= last_page; ++page) {
    if (pages[page]) continue;
    void* pointer{};
    hip_check(hipMalloc(&pointer, kv_page_bytes_), "allocate KV page");
    hip_check(hipMemset(pointer, 0, kv_page_bytes_), "clear KV page");
    pages[page] = pointer;
    hip_check(hipMemcpy(device_page_table_ + page, &pointer, sizeof(pointer),
                        hipMemcpyHostToDevice),
              "publish KV page");
  }
}

DeviceFp4Matrix Mi355DenseFp4Provider::upload_matrix(
    const er::ImmutableModelTensor& tensor, bool tiled) {
  if (tensor.encoding != "FP4_E2M1" || tensor.shape.size() != 2U ||
      !tensor.value.valid())
    throw std::runtime_error("FP4 tensor is invalid: " + tensor.name);
  const std::uint32_t rows = tensor.shape[0];
  const std::uint32_t columns = tensor.shape[1];
  const std::uint32_t padded = pad32(columns);
  const bool block16 = tensor.quant_abi == 16U;
  if (!block16 && tensor.quant_abi != 3U)
    throw std::runtime_error("FP4 tensor quant ABI is not supported: " +
                             tensor.name);
  const std::uint64_t code_bytes = std::uint64_t{rows} * padded / 2U;
  const std::uint64_t scale_bytes =
      block16 ? std::uint64_t{rows} * (padded / 16U) * 2U
              : std::uint64_t{rows} * (padded / 32U);
  // geometry check of dense_fp4_provider.cpp:3569-3580
  if (tensor.data_bytes != code_bytes || tensor.scale_bytes != scale_bytes ||
      tensor.data_offset + code_bytes > tensor.value.bytes ||
      tensor.scale_offset + scale_bytes > tensor.value.bytes)
    throw std::runtime_error("FP4 tensor geometry mismatch: " + tensor.name);

  DeviceBuffer staged_codes(code_bytes, "allocate FP4 weights");
  DeviceBuffer staged_scales(scale_bytes, "allocate FP4 scales");
  hip_check(hipMemcpy(staged_codes.get(), tensor.value.data + tensor.data_offset,
                      code_bytes, hipMemcpyHostToDevice),
            "upload FP4 weights");
  hip_check(hipMemcpy(staged_scales.get(),
                      tensor.value.data + tensor.scale_offset, scale_bytes,
                      hipMemcpyHostToDevice),
            "upload FP4 scales");
  DeviceFp4Matrix matrix;
  matrix.descriptor = {static_cast<const std::uint8_t*>(staged_codes.get()),
                       staged_scales.get(),
                       rows,
                       columns,
                       padded,
                       block16 ? std::uint32_t{QLLM_SCALE_F16_BLOCK16}
                               : std::uint32_t{QLLM_SCALE_UE8M0_BLOCK32},
                       QLLM_LAYOUT_ROW_MAJOR,
                       0U};
  const auto keep = [this, &matrix](DeviceBuffer& codes, DeviceBuffer& scales) {
    allocations_.reserve(allocations_.size() + 2U);
    matrix.weights = codes.get();
    matrix.scales = scales.get();
    allocations_.push_back(codes.release());
    allocations_.push_back(scales.release());
  };
  if (tiled && padded % 64U == 0U) {
    // tile height 0: full 32-row tiles
    DeviceBuffer packed_codes(qllm_fp4_packed_weight_bytes(rows, padded, 0U),
                              "allocate tiled FP4 weights");
    DeviceBuffer packed_scales(
        qllm_fp4_packed_scale_bytes(rows, padded,
                                    matrix.descriptor.scale_scheme, 0U),
        "allocate tiled FP4 scales");
    qllm_fp4_matrix packed{};
    status_check(qllm_fp4_prepack(&matrix.descriptor, 0U, packed_codes.get(),
                                  packed_scales.get(), &packed, stream_));
    hip_check(hipStreamSynchronize(static_cast<hipStream_t>(stream_)),
              "prepack FP4 weights");
    matrix.descriptor = packed;
    keep(packed_codes, packed_scales);   // the row-major copies are freed
  } else {
    keep(staged_codes, staged_scales);
  }
  weight_bytes_ += code_bytes + scale_bytes;
  return matrix;
}

DeviceFp4Matrix Mi355DenseFp4Provider::concatenate_rows(
    std::vector<DeviceFp4Matrix> parts) {
  const qllm_fp4_matrix& first = parts.front().descriptor;
  std::uint32_t rows = 0;
  for (const auto& part : parts) {
    const qllm_fp4_matrix& d = part.descriptor;
    if (d.layout != QLLM_LAYOUT_ROW_MAJOR || d.columns != first.columns ||
        d.padded_columns != first.padded_columns ||
        d.scale_scheme != first.scale_scheme)
      throw std::runtime_error("projections cannot be stored as one matrix");
    rows += d.rows;
  }
  const std::uint32_t padded = first.padded_columns;
  const bool block16 = first.scale_scheme == QLLM_SCALE_F16_BLOCK16;
  const std::size_t row_code_bytes = padded / 2U;
  const std::size_t row_scale_bytes =
      block16 ? std::size_t{padded / 16U} * 2U : padded / 32U;
  DeviceBuffer codes(rows * row_code_bytes, "allocate joined weights");
  DeviceBuffer scales(rows * row_scale_bytes, "allocate joined scales");
  std::size_t row = 0;
  for (const auto& part : parts) {
    const std::uint32_t part_rows = part.descriptor.rows;
    hip_check(hipMemcpy(static_cast<std::uint8_t*>(codes.get()) +
                            row * row_code_bytes,
                        part.weights, part_rows * row_code_bytes,
                        hipMemcpyDeviceToDevice),
              "join weights");
    hip_check(hipMemcpy(static_cast<std::uint8_t*>(scales.get()) +
                            row * row_scale_bytes,
                        part.scales, part_rows * row_scale_bytes,
                        hipMemcpyDeviceToDevice),
              "join scales");
    row += part_rows;
    for (void* pointer : {part.weights, part.scales}) {
      allocations_.erase(
          std::find(allocations_.begin(), allocations_.end(), pointer));
      (void)hipFree(pointer);
    }
  }
  DeviceFp4Matrix joined;
  joined.descriptor = first;
  joined.descriptor.weights = static_cast<const std::uint8_t*>(codes.get());
  joined.descriptor.scales = scales.get();
  joined.descriptor.rows = rows;
  const auto keep = [this, &joined](DeviceBuffer& kept_codes,
                                    DeviceBuffer& kept_scales) {
    allocations_.reserve(allocations_.size() + 2U);
    joined.weights = kept_codes.get();
    joined.scales = kept_scales.get();
    allocations_.push_back(kept_codes.release());
    allocations_.push_back(kept_scales.release());
  };
  if (padded % 64U == 0U) {
    DeviceBuffer packed_codes(qllm_fp4_packed_weight_bytes(rows, padded, 0U),
                              "allocate tiled FP4 weights");
    DeviceBuffer packed_scales(
        qllm_fp4_packed_scale_bytes(rows, padded, first.scale_scheme, 0U),
        "allocate tiled FP4 scales");
    qllm_fp4_matrix packed{};
    status_check(qllm_fp4_prepack(&joined.descriptor, 0U, packed_codes.get(),
                                  packed_scales.get(), &packed, stream_));
    hip_check(hipStreamSynchronize(static_cast<hipStream_t>(stream_)),
              "prepack joined FP4 weights");
    joined.descriptor = packed;
    keep(packed_codes, packed_scales);
  } else {
    keep(codes, scales);
  }
  return joined;
}

float* Mi355DenseFp4Provider::upload_f32(const er::ImmutableModelTensor& tensor,
                                         std::uint32_t elements) {
  if (tensor.encoding != "F32" || !tensor.value.valid() ||
      tensor.data_bytes != std::uint64_t{elements} * 4U ||
      tensor.data_offset + tensor.data_bytes > tensor.value.bytes)
    throw std::runtime_error("F32 tensor is invalid: " + tensor.name);
  void* pointer{};
  hip_check(hipMalloc(&pointer, tensor.data_bytes), "allocate F32 tensor");
  allocations_.push_back(pointer);
  hip_check(hipMemcpy(pointer, tensor.value.data + tensor.data_offset,
                      tensor.data_bytes, hipMemcpyHostToDevice),
            "upload F32 tensor");
  return static_cast<float*>(pointer);
}

er::PrepareOperationResult Mi355DenseFp4Provider::prepare(
    const er::OperationPreparationContext& context) {
  try {
    std::lock_guard lock(mutex_);
    auto status = validate_parameters(context.operation.parameters);
    if (!status.ok()) return {status, {}};
    const std::string& capability = context.operation.capability;
    auto prepared = std::make_shared<PreparedOperation>();
    prepared->capability = capability;
    prepared->abi_version = context.operation.abi_version;
    prepared->logical_operation = context.compiled.logical_operation;
    // ports: inputs arrive in the compiled order, outputs leave with the ABI
    // the artifact declares for the port (:2912-2923)
    for (std::size_t index = 0; index < context.compiled.input_values.size();
         ++index)
      prepared->input_indices.emplace(context.compiled.input_values[index].port,
                                      index);
    for (const auto& binding : context.compiled.output_values) {
      const auto output = context.operation.output_bindings.find(binding.port);
      if (output == context.operation.output_bindings.end())
        throw std::runtime_error("compiled output port is absent");
      prepared->outputs.emplace_back(binding.port, output->second.abi);
    }
    const auto query_rows =
        g_.query_heads * g_.head_dim * (g_.output_gated ? 2U : 1U);
    const auto require_shape = [](const DeviceFp4Matrix& matrix,
                                  std::uint32_t rows, std::uint32_t columns,
                                  const char* role) {
      if (matrix.descriptor.rows != rows || matrix.descriptor.columns != columns)
        throw std::runtime_error(std::string("tensor shape mismatch: ") + role);
    };
    if (capability.starts_with("embedding.lookup.")) {
      embedding_ = upload_matrix(
          tensor_for_either(context.tensors, "weight", "token_embedding"), false);
      require_shape(embedding_, g_.vocabulary, g_.hidden, "token_embedding");
      embedding_ready_ = true;
      prepared->kind = PreparedOperation::Kind::embedding;
    } else if (capability.starts_with("block.full-attention.")) {
      const bool gated = capability.find("output-gated") != std::string::npos;
      if (gated != g_.output_gated)
        throw std::runtime_error(
            "attention capability does not match the declared geometry");
      if (attention_ops_ >= g_.layers)
        throw std::runtime_error("more attention blocks than layers");
      auto& layer = layers_[attention_ops_];
      layer.input_norm =
          upload_f32(tensor_for(context.tensors, "input_norm"), g_.hidden);
      DeviceFp4Matrix query = upload_matrix(
          tensor_for(context.tensors, "query_projection"), false);
      DeviceFp4Matrix key =
          upload_matrix(tensor_for(context.tensors, "key_projection"), false);
      DeviceFp4Matrix value =
          upload_matrix(tensor_for(context.tensors, "value_projection"), false);
      layer.output = upload_matrix(
          tensor_for(context.tensors, "output_projection"), true);
      require_shape(query, query_rows, g_.hidden, "query_projection");
      require_shape(key, g_.kv_heads * g_.head_dim, g_.hidden,
                    "key_projection");
      require_shape(value, g_.kv_heads * g_.head_dim, g_.hidden,
                    "value_projection");
      layer.qkv = concatenate_rows({query, key, value});
      require_shape(layer.output, g_.hidden, g_.query_heads * g_.head_dim,
                    "output_projection");
      if (g_.qk_norm) {
        layer.query_norm =
            upload_f32(tensor_for(context.tensors, "query_norm"), g_.head_dim);
        layer.key_norm =
            upload_f32(tensor_for(context.tensors, "key_norm"), g_.head_dim);
      }
      prepared->kind = PreparedOperation::Kind::attention;
      prepared->layer = attention_ops_;
      ++attention_ops_;
    } else if (capability.starts_with("ffn.swiglu.dense.")) {
      if (ffn_ops_ >= g_.layers)
        throw std::runtime_error("more FFN blocks than layers");
      auto& layer = layers_[ffn_ops_];
      layer.post_attention_norm = upload_f32(
          tensor_for_either(context.tensors, "input_norm", "post_attention_norm"),
          g_.hidden);
      layer.gate =
          upload_matrix(tensor_for(context.tensors, "gate_projection"), true);
      layer.up =
          upload_matrix(tensor_for(context.tensors, "up_projection"), true);
      layer.down =
          upload_matrix(tensor_for(context.tensors, "down_projection"), true);
      require_shape(layer.gate, g_.intermediate, g_.hidden, "gate_projection");
      require_shape(layer.up, g_.intermediate, g_.hidden, "up_projection");
      require_shape(layer.down, g_.hidden, g_.intermediate, "down_projection");
      prepared->kind = PreparedOperation::Kind::ffn;
      prepared->layer = ffn_ops_;
      ++ffn_ops_;
    } else if (capability.starts_with("head.rmsnorm.token-select.")) {
      final_norm_ = upload_f32(
          tensor_for_either(context.tensors, "norm", "hidden_norm"), g_.hidden);
      head_ = upload_matrix(
          tensor_for_either(context.tensors, "weight", "output_head"), true);
      require_shape(head_, g_.vocabulary, g_.hidden, "output_head");
      head_ready_ = true;
      prepared->kind = PreparedOperation::Kind::head;
    } else {
      return {{er::ErrorCode::invalid_argument,
               "capability is not provided: " + capability},
              {}};
    }
    return {er::Status::success(), std::move(prepared)};
  } catch (const std::exception& error) {
    return {{er::ErrorCode::internal, error.what()}, {}};
  }
}

er::PrepareOperationResult Mi355DenseFp4Provider::prepare_exact_decode(
    const er::ExactDecodePreparationContext& context) {
  try {
    std::lock_guard lock(mutex_);
    if (!context.program.capability.starts_with(
            "decode.mtp.dense-full-attention.") ||
        context.program.abi_version != 2U)
      return {{er::ErrorCode::invalid_argument,
               "exact decode capability or ABI is not provided"},
              {}};
    // the artifact contract of the exact-decode program (:2934-2966)
    const auto& parameters = context.program.parameters;
    const auto depth = parameters.find("draft_depth");
    if (depth == parameters.end() || depth->second != g_.draft_depth ||
        context.program.maximum_emitted_tokens != g_.draft_depth + 1U)
      return {{er::ErrorCode::invalid_argument,
               "exact decode draft depth does not match the provider"},
              {}};
    if (!embedding_ready_ || !head_ready_ || attention_ops_ != g_.layers ||
        ffn_ops_ != g_.layers)
      return {{er::ErrorCode::invalid_argument,
               "target program is not fully prepared"},
              {}};
    if (g_.mtp_layers && !context.tensors.empty()) prepare_mtp(context.tensors);
    if (g_.mtp_layers && !mtp_.ready)
      return {{er::ErrorCode::invalid_argument,
               "exact decode with an MTP layer needs the proposer's tensors"},
              {}};
    auto prepared = std::make_shared<PreparedOperation>();
    prepared->kind = PreparedOperation::Kind::exact_decode;
    prepared->capability = context.program.capability;
    prepared->abi_version = context.program.abi_version;
    exact_ = prepared;
    return {er::Status::success(), exact_};
  } catch (const std::exception& error) {
    return {{er::ErrorCode::internal, error.what()}, {}};
  }
}

// Tensors of the exact-decode operation (validate_exact, :4730-4787).
void Mi355DenseFp4Provider::prepare_mtp(
    std::span<const er::PreparedTensorBinding> tensors) {
  const auto require_shape = [](const DeviceFp4Matrix& matrix, std::uint32_t rows,
                                std::uint32_t columns, const char* role) {
    if (matrix.descriptor.rows != rows || matrix.descriptor.columns != columns)
      throw std::runtime_error(std::string("tensor shape mismatch: ") + role);
  };
  const auto query_rows =
      g_.query_heads * g_.head_dim * (g_.output_gated ? 2U : 1U);
  mtp_.embedding_norm = upload_f32(tensor_for(tensors, "embedding_norm"), g_.hidden);
  mtp_.hidden_norm = upload_f32(tensor_for(tensors, "hidden_norm"), g_.hidden);
  mtp_.draft_norm = upload_f32(tensor_for(tensors, "draft_norm"), g_.hidden);
  mtp_.fusion = upload_matrix(tensor_for(tensors, "fusion_projection"), true);
  require_shape(mtp_.fusion, g_.hidden, 2U * g_.hidden, "fusion_projection");
  auto& layer = mtp_.layer;
  layer.input_norm =
      upload_f32(tensor_for(tensors, "layer.0.input_norm"), g_.hidden);
  DeviceFp4Matrix query =
      upload_matrix(tensor_for(tensors, "layer.0.query_projection"), false);
  DeviceFp4Matrix key =
      upload_matrix(tensor_for(tensors, "layer.0.key_projection"), false);
  DeviceFp4Matrix value =
      upload_matrix(tensor_for(tensors, "layer.0.value_projection"), false);
  require_shape(query, query_rows, g_.hidden, "layer.0.query_projection");
  require_shape(key, g_.kv_heads * g_.head_dim, g_.hidden, "layer.0.key_projection");
  require_shape(value, g_.kv_heads * g_.head_dim, g_.hidden,
                "layer.0.value_projection");
  layer.qkv = concatenate_rows({query, key, value});
  layer.output =
      upload_matrix(tensor_for(tensors, "layer.0.output_projection"), true);
  require_shape(layer.output, g_.hidden, g_.query_heads * g_.head_dim,
                "layer.0.output_projection");
  if (g_.qk_norm) {
    layer.query_norm =
        upload_f32(tensor_for(tensors, "layer.0.query_norm"), g_.head_dim);
    layer.key_norm =
        upload_f32(tensor_for(tensors, "layer.0.key_norm"), g_.head_dim);
  }
  layer.post_attention_norm =
      upload_f32(tensor_for(tensors, "layer.0.post_attention_norm"), g_.hidden);
  layer.gate = upload_matrix(tensor_for(tensors, "layer.0.gate_projection"), true);
  layer.up = upload_matrix(tensor_for(tensors, "layer.0.up_projection"), true);
  layer.down = upload_matrix(tensor_for(tensors, "layer.0.down_projection"), true);
  require_shape(layer.gate, g_.intermediate, g_.hidden, "layer.0.gate_projection");
  require_shape(layer.up, g_.intermediate, g_.hidden, "layer.0.up_projection");
  require_shape(layer.down, g_.hidden, g_.intermediate, "layer.0.down_projection");
  finish_mtp_weights();
}

// project_prefix (:6280-6308): the proposer scores the first draft_vocabulary
// rows of the output head; in either layout those are a leading byte range.
void Mi355DenseFp4Provider::finish_mtp_weights() {
  if (!head_ready_ && !head_.weights)
    throw std::runtime_error("the output head must be prepared before the proposer");
  mtp_.head_prefix = head_.descriptor;
  mtp_.head_prefix.rows = g_.draft_vocabulary;
  mtp_.ready = true;
}

er::CreateOperationRequestStateResult
Mi355DenseFp4Provider::create_request_state(
    const er::ProgramRequestContext& request) {
  try {
    std::lock_guard lock(mutex_);
    // the sampling profile check of dense_fp4_provider.cpp:5502-5513
    const auto temperature = request.parameters.find("sampling_temperature_ppm");
    if (temperature != request.parameters.end() && temperature->second != 0U) {
      const auto first = request.parameters.find("sampling_first_output_position");
      const auto presence =
          request.parameters.find("sampling_presence_penalty_biased_ppm");
      if (first == request.parameters.end() || first->second >= g_.max_context ||
          presence == request.parameters.end() || presence->second > 4'000'000U)
        throw std::runtime_error("request has an invalid sampling profile");
    }
    // a free slot, or the reference's answer when every slot is taken
    // (dense_fp4_provider.cpp:5514-5518)
    std::uint32_t slot = 0U;
    while (slot < slots_.size() &&
           slots_[slot].leased->load(std::memory_order_acquire))
      ++slot;
    if (slot == slots_.size())
      return {{er::ErrorCode::backpressure,
               "dense FP4 provider has no free request slot"},
              {}};
    activate(slot);
    hip_check(hipMemsetAsync(presence_, 0, g_.vocabulary,
                             static_cast<hipStream_t>(stream_)),
              "zero request sampling presence");
    // The KV pages of the request's reserved context are allocated and cleared
    // here, not page by page inside the decode loop (an allocation, a clearing
    // and a blocking copy at every page boundary).
    const auto reserved = request.parameters.find("reserved_context_tokens");
    if (reserved != request.parameters.end() && reserved->second != 0U)
      ensure_pages(static_cast<std::uint32_t>(
          std::min<std::uint64_t>(reserved->second, g_.max_context) - 1U));
    auto state = std::make_shared<DenseFp4RequestState>();
    state->slot = slot;
    state->lease = slots_[slot].leased;
    state->lease->store(true, std::memory_order_release);
    return {er::Status::success(), std::move(state)};
  } catch (const std::exception& error) {
    return {{er::ErrorCode::internal, error.what()}, {}};
  }
}

void Mi355DenseFp4Provider::mark_presence(
    std::uint8_t* emitted, std::span<const std::uint32_t> tokens) {
  if (tokens.empty()) return;
  if (tokens.size() > 8U) throw std::runtime_error("too many presence marks");
  const auto stream = static_cast<hipStream_t>(stream_);
  // the pinned words are free: every pass that used them ended with a wait
  std::copy(tokens.begin(), tokens.end(), staging_->marks);
  hip_check(hipMemcpyAsync(mark_tokens_, staging_->marks, tokens.size() * 4U,
                           hipMemcpyHostToDevice, stream),
            "upload presence marks");
  status_check(qllm_mark_presence(emitted, mark_tokens_,
                                  static_cast<std::uint32_t>(tokens.size()),
                                  g_.vocabulary, stream_));
}

er::Status Mi355DenseFp4Provider::rebind_request_state(
    const std::shared_ptr<er::IOperationProviderRequestState>& opaque_state,
    const er::ProgramRequestContext& request) {
  try {
    std::lock_guard lock(mutex_);
    const auto state =
        std::dynamic_pointer_cast<DenseFp4RequestState>(opaque_state);
    const auto first = request.parameters.find("sampling_first_output_position");
    const auto presence =
        request.parameters.find("sampling_presence_penalty_biased_ppm");
    if (!state || first == request.parameters.end() ||
        first->second >= g_.max_context ||
        presence == request.parameters.end() || presence->second > 4'000'000U)
      throw std::runtime_error("sampling request rebind is invalid");
    activate(state->slot);
    hip_check(hipMemsetAsync(presence_, 0, g_.vocabulary,
                             static_cast<hipStream_t>(stream_)),
              "reset request sampling presence");
    return er::Status::success();
  } catch (const std::exception& error) {
    return {er::ErrorCode::internal, error.what()};
  }
}

// :5579-5586
er::ExecutionValue Mi355DenseFp4Provider::device_hidden_value(
    std::uint32_t rows) const {
  if (!rows || rows > max_rows_)
    throw std::runtime_error("invalid FP4 hidden batch size");
  return {std::string(kHiddenAbi), std::string(kDeviceDomain), device_lifetime_,
          reinterpret_cast<const std::byte*>(hidden_),
          std::uint64_t{rows} * g_.hidden * sizeof(float)};
}

// :5649-5660
std::uint32_t Mi355DenseFp4Provider::require_hidden_value(
    const er::ExecutionValue& value) const {
  const auto row_bytes = std::uint64_t{g_.hidden} * sizeof(float);
  if (value.abi != kHiddenAbi || value.memory_domain != kDeviceDomain ||
      value.data != reinterpret_cast<const std::byte*>(hidden_) ||
      value.bytes % row_bytes != 0U || value.bytes / row_bytes == 0U ||
      value.bytes / row_bytes > max_rows_)
    throw std::runtime_error("hidden-state execution ABI mismatch");
  return static_cast<std::uint32_t>(value.bytes / row_bytes);
}

// The head's token for a request (run_head with a request, :8433-8517): the
// presence penalty from the first output position on, arg-max at temperature
// zero, otherwise top-k or whole-row candidates ordered on the host and one
// draw from stream 0; an output token is marked as emitted.  logits_ row 0.
std::uint32_t Mi355DenseFp4Provider::select_head_token(
    const er::ProgramRequestContext& request, std::uint32_t sample_position) {
  const auto stream = static_cast<hipStream_t>(stream_);
  const auto first_output =
      request_parameter(request, "sampling_first_output_position");
  const bool output_sampling = sample_position >= first_output;
  const auto penalty = presence_penalty_of(request);
  if (output_sampling && penalty != 0.0) {
    status_check(qllm_apply_presence_penalty(logits_, presence_, g_.vocabulary,
                                             static_cast<float>(penalty),
                                             stream_));
    status_check(qllm_argmax_batch(logits_, g_.vocabulary, 1U, argmax_tokens_,
                                   select_workspace_, select_workspace_bytes_,
                                   stream_));
  }
  const auto temperature = request_parameter(request, "sampling_temperature_ppm");
  std::uint32_t selected{};
  if (temperature == 0U) {
    hip_check(hipMemcpyAsync(&selected, argmax_tokens_, sizeof(selected),
                             hipMemcpyDeviceToHost, stream),
              "copy dense FP4 greedy token");
    hip_check(hipStreamSynchronize(stream), "copy dense FP4 greedy token");
    // a row without a finite logit selects nothing (0xffffffff): reported
    // before the presence bytes or the caller's state change
    if (selected >= g_.vocabulary)
      throw std::runtime_error("head logits have no finite maximum");
  } else {
    // the penalty, if any, has been applied: the distribution is taken from
    // the row as it stands
    er::ProgramRequestContext unpenalised = request;
    unpenalised.parameters["sampling_presence_penalty_biased_ppm"] = 2'000'000U;
    const auto top_k = request_parameter(request, "sampling_top_k");
    if (top_k > kMaximumGpuSamplingTopK) {
      // the scalar sampler orders that many candidates on the host
      // (sample_token, :773-799)
      std::vector<float> row(g_.vocabulary);
      hip_check(hipMemcpyAsync(row.data(), logits_, row.size() * 4U,
                               hipMemcpyDeviceToHost, stream),
                "copy dense FP4 sampling logits");
      hip_check(hipStreamSynchronize(stream), "copy dense FP4 sampling logits");
      if (top_k > row.size())
        throw std::runtime_error("invalid token sampling contract");
      std::vector<std::uint32_t> candidates(row.size());
      std::iota(candidates.begin(), candidates.end(), 0U);
      const auto before = [&](std::uint32_t left, std::uint32_t right) {
        const float a = row[left];
        const float b = row[right];
        if (std::isnan(a)) return false;
        if (std::isnan(b)) return true;
        return a == b ? left < right : a > b;
      };
      std::partial_sort(candidates.begin(), candidates.begin() + top_k,
                        candidates.end(), before);
      candidates.resize(top_k);
      std::vector<float> ordered;
      for (const auto candidate : candidates) ordered.push_back(row[candidate]);
      sampling_logit_transfer_bytes_ += row.size() * 4U;
      const auto distribution = er::make_sampling_distribution(
          ordered, candidates, static_cast<std::uint32_t>(temperature),
          static_cast<std::uint32_t>(
              request_parameter(request, "sampling_top_p_ppm")),
          static_cast<std::uint32_t>(
              request_parameter(request, "sampling_min_p_ppm")));
      selected = er::sample_distribution(
          distribution,
          er::counter_uniform(request_parameter(request, "sampling_seed"),
                              sample_position, 0U));
    } else {
      const auto distribution = distribution_from_logits(
          logits_, g_.vocabulary, argmax_tokens_, unpenalised, nullptr);
      selected = er::sample_distribution(
          distribution,
          er::counter_uniform(request_parameter(request, "sampling_seed"),
                              sample_position, 0U));
    }
  }
  if (output_sampling) {
    const std::uint32_t token[1] = {selected};
    mark_presence(presence_, token);
  }
  return selected;
}

// One operation of the artifact's program (execute, :10680-10992).
er::OperationExecutionHandle Mi355DenseFp4Provider::execute(
    const er::IPreparedOperation& opaque_operation,
    const std::shared_ptr<er::IOperationProviderRequestState>& opaque_state,
    const er::OperationInvocation& invocation) {
  try {
    std::lock_guard lock(mutex_);
    const auto* operation =
        dynamic_cast<const PreparedOperation*>(&opaque_operation);
    const auto state =
        std::dynamic_pointer_cast<DenseFp4RequestState>(opaque_state);
    if (!operation || !state ||
        operation->kind == PreparedOperation::Kind::exact_decode)
      throw std::runtime_error("dense FP4 invocation state is invalid");
    activate(state->slot);
    const auto input = [&](std::string_view port) -> const er::ExecutionValue& {
      const auto found = operation->input_indices.find(port);
      if (found == operation->input_indices.end() ||
          found->second >= invocation.inputs.size())
        throw std::runtime_error("operation input port is absent");
      return invocation.inputs[found->second];
    };
    const auto stream = static_cast<hipStream_t>(stream_);
    std::map<std::string, er::ExecutionValue, std::less<>> outputs;
    const auto phase_of = [](PreparedOperation::Kind kind) {
      switch (kind) {
        case PreparedOperation::Kind::embedding: return GpuPhase::embedding;
        case PreparedOperation::Kind::attention: return GpuPhase::full_attention;
        case PreparedOperation::Kind::ffn: return GpuPhase::ffn;
        case PreparedOperation::Kind::head: return GpuPhase::head;
        default: return GpuPhase::mtp;
      }
    };
    const auto phase_events = begin_gpu_phase(phase_of(operation->kind));
    switch (operation->kind) {
      case PreparedOperation::Kind::embedding: {
        state->exact_decode_enabled =
            exact_ &&
            request_parameter(invocation.request, "exact_decode_enabled") != 0U;
        if (state->synchronization_rows != 0U)
          throw std::runtime_error("previous target batch was not synchronized");
        const auto tokens =
            host_u32_batch(input("token_ids"), kTokenAbi, "embedding token batch");
        if (tokens.empty() || tokens.size() > max_rows_)
          throw std::runtime_error("invalid FP4 hidden batch size");
        for (const auto token : tokens)
          if (token >= g_.vocabulary)
            throw std::runtime_error("embedding token exceeds vocabulary");
        const auto rows = static_cast<std::uint32_t>(tokens.size());
        // a pageable source: the copy has read it when the call returns
        hip_check(hipMemcpyAsync(tokens_, tokens.data(), rows * 4U,
                                 hipMemcpyHostToDevice, stream),
                  "upload target tokens");
        status_check(qllm_fp4_embedding_batch(&embedding_.descriptor, tokens_,
                                              hidden_, rows, stream_));
        pending_partials_ = 0U;
        state->current_batch_rows = rows;
        outputs.emplace("hidden", device_hidden_value(rows));
        break;
      }
      case PreparedOperation::Kind::attention: {
        const auto rows = require_hidden_value(input("hidden"));
        const auto positions = host_u32_batch(input("positions"), kPositionAbi,
                                              "attention position batch");
        if (positions.size() != rows || rows != state->current_batch_rows)
          throw std::runtime_error("attention batch width changed in program");
        for (std::uint32_t row = 0; row < rows; ++row)
          if (positions[row] >= g_.max_context ||
              (row != 0U && positions[row] != positions[0] + row))
            throw std::runtime_error("attention position batch is not contiguous");
        state->current_batch_first = positions.front();
        state->current_position = positions.back();
        ensure_pages(positions.back());
        enqueue_rope_table(rows, positions.front(), false);
        enqueue_attention_block(operation->layer, rows, positions.front(), false,
                                false);
        outputs.emplace("hidden", device_hidden_value(rows));
        break;
      }
      case PreparedOperation::Kind::ffn: {
        const auto rows = require_hidden_value(input("hidden"));
        if (rows != state->current_batch_rows)
          throw std::runtime_error("FFN batch width changed in program");
        enqueue_ffn_block(operation->layer, rows, false);
        outputs.emplace("hidden", device_hidden_value(rows));
        break;
      }
      case PreparedOperation::Kind::head: {
        const auto rows = require_hidden_value(input("hidden"));
        if (rows != state->current_batch_rows)
          throw std::runtime_error("head batch width changed in program");
        // hidden_ keeps the batch: the proposer is synchronised from it
        if (state->exact_decode_enabled) {
          state->synchronization_first = state->current_batch_first;
          state->synchronization_rows = rows;
          state->synchronization_consumed = 0U;
        } else {
          state->synchronization_first = 0U;
          state->synchronization_rows = 0U;
          state->synchronization_consumed = 0U;
          state->mtp_length = state->current_position + 1U;
          state->draft_valid = false;
          state->draft_predictions.clear();
        }
        // a batch selects for its last row only (terminal_only, :8397-8402)
        enqueue_head(rows - 1U, 1U);
        end_gpu_phase(phase_events);
        collect_gpu_phases();
        auto owner = std::make_shared<std::vector<std::uint32_t>>(
            1U, select_head_token(invocation.request, state->current_position));
        outputs.emplace(
            "token_ids",
            er::ExecutionValue{std::string(kTokenAbi), "host", owner,
                               reinterpret_cast<const std::byte*>(owner->data()),
                               owner->size() * sizeof(std::uint32_t)});
        program_steps_ += rows;
        if (rows > 1U) prefill_tokens_total_ += rows;
        break;
      }
      case PreparedOperation::Kind::exact_decode:
        throw std::runtime_error("exact decode entered scalar execution");
    }
    if (operation->kind != PreparedOperation::Kind::head)
      end_gpu_phase(phase_events);
    er::OperationExecutionResult result;
    result.status = er::Status::success();
    result.outputs.reserve(operation->outputs.size());
    for (const auto& [port, abi] : operation->outputs) {
      const auto found = outputs.find(port);
      if (found == outputs.end() || found->second.abi != abi)
        throw std::runtime_error("dense FP4 output ABI mismatch");
      result.outputs.push_back(std::move(found->second));
    }
    return completed_operation(std::move(result));
  } catch (const std::exception& error) {
    return completed_operation({{er::ErrorCode::internal, error.what()}, {}});
  }
}

// :10994-11009
er::Status Mi355DenseFp4Provider::synchronize_exact_decode(
    const er::IPreparedOperation& operation,
    const std::shared_ptr<er::IOperationProviderRequestState>& state,
    const er::ExactDecodeSynchronization& synchronization) {
  const std::uint32_t tokens[1] = {synchronization.next_token};
  return synchronize_exact_decode_batch(
      operation, state,
      er::ExactDecodeSynchronizationBatch{synchronization.request, tokens,
                                          synchronization.target_position,
                                          synchronization.produce_draft});
}

// Records where the verified stream stands after prefill / a previous step
// (dense_fp4_provider.cpp:11011-11130).  Producing the drafts themselves is
// the proposer's job; they arrive through set_draft_predictions().
er::Status Mi355DenseFp4Provider::synchronize_exact_decode_batch(
    const er::IPreparedOperation& operation,
    const std::shared_ptr<er::IOperationProviderRequestState>& opaque_state,
    const er::ExactDecodeSynchronizationBatch& synchronization) {
  try {
    std::lock_guard lock(mutex_);
    const auto state =
        std::dynamic_pointer_cast<DenseFp4RequestState>(opaque_state);
    if (&operation != exact_.get() || !state ||
        synchronization.next_tokens.empty())
      return {er::ErrorCode::invalid_argument,
              "exact decode synchronization is invalid"};
    for (const auto token : synchronization.next_tokens)
      if (token >= g_.vocabulary)
        return {er::ErrorCode::invalid_argument,
                "synchronized token is outside the vocabulary"};
    activate(state->slot);
    const auto rows =
        static_cast<std::uint32_t>(synchronization.next_tokens.size());
    if (rows > max_rows_ ||
        synchronization.first_target_position > g_.max_context - rows)
      return {er::ErrorCode::invalid_argument,
              "exact decode synchronization is invalid"};
    // Rows of the last head execute() ran are consumed in order (:11020-11036);
    // a host that runs the target through run_target() has no such window and
    // synchronises from row 0 of that pass.
    const float* previous_hidden = hidden_;
    if (state->synchronization_rows != 0U) {
      if (state->synchronization_consumed >= state->synchronization_rows ||
          rows > state->synchronization_rows - state->synchronization_consumed ||
          state->mtp_length != synchronization.first_target_position ||
          synchronization.first_target_position !=
              state->synchronization_first + state->synchronization_consumed)
        throw std::runtime_error("MTP synchronization stream is invalid");
      previous_hidden =
          hidden_ + std::size_t{state->synchronization_consumed} * g_.hidden;
      state->synchronization_consumed += rows;
      if (state->synchronization_consumed == state->synchronization_rows)
        state->synchronization_rows = state->synchronization_consumed = 0U;
    }
    state->synchronized_token = synchronization.next_tokens.back();
    state->draft_valid = false;
    state->draft_predictions.clear();
    // next_tokens[r] sits at position first_target_position + r + 1 and was
    // chosen from the target's hidden state at first_target_position + r; the
    // proposer is fed exactly these pairs (its cache lags the target's by one
    // token), after which the guaranteed token stands at mtp_length.
    state->mtp_length = synchronization.first_target_position;
    if (mtp_.ready) {
      const auto sample_position = synchronization.first_target_position + rows;
      if (synchronization.produce_final_draft)
        hip_check(hipMemcpyAsync(proposal_presence_, presence_, g_.vocabulary,
                                 hipMemcpyDeviceToDevice,
                                 static_cast<hipStream_t>(stream_)),
                  "initialize speculative proposal presence");
      auto draft = run_mtp(*state, synchronization.next_tokens, previous_hidden,
                           synchronization.produce_final_draft,
                           synchronization.produce_final_draft
                               ? &synchronization.request
                               : nullptr,
                           synchronization.produce_final_draft
                               ? proposal_presence_
                               : nullptr,
                           sample_position, 1U);
      if (synchronization.produce_final_draft) {
        if (!draft)
          throw std::runtime_error("MTP synchronization produced no draft");
        const auto reserved = synchronization.request.parameters.find(
            "reserved_context_tokens");
        const auto context_limit =
            reserved == synchronization.request.parameters.end()
                ? g_.max_context
                : static_cast<std::uint32_t>(reserved->second);
        extend_mtp_rollout(*state, synchronization.request, std::move(*draft),
                           context_limit);
      }
    } else {
      state->mtp_length += rows;
    }
    return er::Status::success();
  } catch (const std::exception& error) {
    return {er::ErrorCode::internal, error.what()};
  }
}

er::Status Mi355DenseFp4Provider::begin_stream(
    const std::shared_ptr<er::IOperationProviderRequestState>& opaque_state,
    std::uint32_t token) {
  std::lock_guard lock(mutex_);
  const auto state =
      std::dynamic_pointer_cast<DenseFp4RequestState>(opaque_state);
  if (!state || token >= g_.vocabulary)
    return {er::ErrorCode::invalid_argument, "stream start is invalid"};
  state->synchronized_token = token;
  state->mtp_length = 0U;
  state->draft_valid = false;
  state->draft_predictions.clear();
  return er::Status::success();
}

er::Status Mi355DenseFp4Provider::set_draft_predictions(
    const std::shared_ptr<er::IOperationProviderRequestState>& opaque_state,
    std::vector<DraftPrediction> drafts) {
  std::lock_guard lock(mutex_);
  const auto state =
      std::dynamic_pointer_cast<DenseFp4RequestState>(opaque_state);
  if (!state || drafts.empty() || drafts.size() > g_.draft_depth)
    return {er::ErrorCode::invalid_argument, "draft predictions are invalid"};
  for (const auto& draft : drafts)
    if (draft.token >= g_.vocabulary)
      return {er::ErrorCode::invalid_argument,
              "draft token is outside the vocabulary"};
  state->draft_predictions = std::move(drafts);
  state->draft_valid = true;
  return er::Status::success();
}

// ---- target pass ------------------------------------------------------------

// Rotary + per-head norm of the new rows' q and k, their K/V records into the
// layer's cache and the rows' attention over everything cached so far
// (run_full_attention, :6892-7960).  `query`, `key`, `value` hold `rows` rows
// starting at `first_position`; the result goes to `attention_out` in bf16.
void Mi355DenseFp4Provider::enqueue_attention(
    std::uint32_t index, std::uint32_t rows, std::uint32_t first_position,
    bool deferred_positions, float* query, float* key, float* value,
    std::uint16_t* attention_out, const float* qkv_partials,
    std::uint32_t qkv_partial_count) {
  void* const stream = stream_;
  const auto& layer = layers_[index];
  const std::uint32_t query_stride = g_.head_dim * (g_.output_gated ? 2U : 1U);
  if (g_.kv_encoding == KvEncoding::q4_f16_per_head) {
    // With the projection in one piece the attention kernel does the rotary
    // and the K/V store itself (cos / sin from rope_table_, see
    // enqueue_rope_table); K-split partials go through the rotary kernel,
    // which sums them and leaves the queries as the attention kernel's int8
    // operands.
    const bool fused = qkv_partials == nullptr;
    if (!fused)
      status_check(qllm_qkv_rope_cache_paged_q4h_prepared(
          qkv_partials, qkv_partial_count, query, query_stride, key, value,
          layer.query_norm, layer.key_norm,
          const_cast<const void* const*>(device_page_table_), index,
          g_.kv_page_tokens, first_position, first_position,
          deferred_positions ? positions_ : nullptr, rows, g_.query_heads,
          g_.kv_heads, g_.head_dim, g_.rotary_dim, g_.norm_epsilon,
          g_.rope_theta, 0, query_operands_, query_operand_scales_, stream));
    qllm_q4h_attention_launch launch{};
    launch.query = query;
    launch.q8_queries = fused ? nullptr : query_operands_;
    launch.query_scales = fused ? nullptr : query_operand_scales_;
    launch.page_table = const_cast<const void* const*>(device_page_table_);
    launch.output = attention_out;
    launch.partial_maxima = partial_maxima_;
    launch.partial_sums = partial_sums_;
    launch.partial_outputs = partial_outputs_;
    launch.first_context_tokens = first_position + 1U;  // :7915
    launch.rows = rows;
    launch.full_attention_layer = index;
    launch.page_tokens = g_.kv_page_tokens;
    launch.query_heads = g_.query_heads;
    launch.kv_heads = g_.kv_heads;
    launch.head_dim = g_.head_dim;
    launch.split_tokens = split_tokens_;
    launch.maximum_splits = maximum_splits_;
    launch.query_stride = query_stride;
    launch.output_gated = g_.output_gated;
    launch.output_kind = g_.activation_q8 ? QLLM_OUT_F32 : QLLM_OUT_BF16;
    launch.stream = stream;
    launch.device_positions = deferred_positions ? positions_ : nullptr;
    if (fused) {
      qllm_q4h_fused_rope rope{};
      rope.key = key;
      rope.value = value;
      rope.q_norm_weight = layer.query_norm;
      rope.k_norm_weight = layer.key_norm;
      rope.rope_table = rope_table_;
      rope.rotary_dim = g_.rotary_dim;
      rope.epsilon = g_.norm_epsilon;
      rope.first_cache_position = first_position;
      rope.bf16_activations = 0;
      status_check(qllm_attention_paged_q4h_fused(&launch, &rope));
    } else {
      status_check(qllm_attention_paged_q4h(&launch));
    }
  } else {
    status_check(qllm_qkv_rope_batch(
        query, query_stride, key, layer.query_norm, layer.key_norm,
        first_position, rows, g_.query_heads, g_.kv_heads, g_.head_dim,
        g_.rotary_dim, g_.norm_epsilon, g_.rope_theta, 0, stream));
    status_check(qllm_store_kv_paged_f16_batch(
        key, value, const_cast<const void* const*>(device_page_table_),
        index, g_.kv_page_tokens, first_position, rows, g_.kv_heads,
        g_.head_dim, stream));
    qllm_f16_attention_launch launch{};
    launch.query = query;
    launch.device_pages = const_cast<const void* const*>(device_page_table_);
    launch.output = attention_out;
    launch.partial_maxima = partial_maxima_;
    launch.partial_sums = partial_sums_;
    launch.partial_outputs = partial_outputs_;
    launch.first_context_tokens = first_position + 1U;
    launch.rows = rows;
    launch.device_page_layer = index;
    launch.device_page_tokens = g_.kv_page_tokens;
    launch.query_heads = g_.query_heads;
    launch.kv_heads = g_.kv_heads;
    launch.head_dim = g_.head_dim;
    launch.split_tokens = split_tokens_;
    launch.maximum_splits = maximum_splits_;
    launch.query_stride = query_stride;
    launch.output_gated = g_.output_gated;
    launch.output_kind = g_.activation_q8 ? QLLM_OUT_F32 : QLLM_OUT_BF16;
    launch.stream = stream;
    status_check(qllm_attention_paged_f16(&launch));
  }
}

// Context splits of a batched (prompt) attention launch.  Every workgroup pays
// a prologue and a merge of its eight wave states whatever its share of the
// context, so the context is cut only as far as it takes to give every CU a
// workgroup: a full chunk's row batches need no cut at all (a 32768-token
// prompt: 5.50 s with eight splits, 5.09 / 4.91 / 4.79 s with four / two / one).
std::uint32_t Mi355DenseFp4Provider::prefill_splits_for(
    std::uint32_t rows, std::uint32_t attention_batch) const noexcept {
  const std::uint32_t batches = (rows + attention_batch - 1U) / attention_batch;
  const std::uint32_t workgroups = std::max(1U, batches * g_.kv_heads);
  return std::clamp((256U + workgroups - 1U) / workgroups, 1U, prefill_splits_);
}

// Context splits of the shared-tile prompt attention (eight row batches per
// workgroup), or 0 where the batched launch of the verify step's kernel serves:
// fewer than 32 row batches, head_dim 256.
std::uint32_t Mi355DenseFp4Provider::prompt_attention_splits(
    std::uint32_t rows, std::uint32_t attention_batch) const noexcept {
  const std::uint32_t batches = (rows + attention_batch - 1U) / attention_batch;
  if (g_.head_dim != 128U || batches < 32U) return 0U;
  const std::uint32_t workgroups = (batches + 7U) / 8U * g_.kv_heads;
  return std::clamp((256U + workgroups - 1U) / workgroups, 1U, prefill_splits_);
}

// (cos, sin) of the rotary angles of a batch at first_position .. + rows - 1
// (or at the device-side positions), for the attention launches of a pass.
void Mi355DenseFp4Provider::enqueue_rope_table(std::uint32_t rows,
                                               std::uint32_t first_position,
                                               bool deferred_positions) {
  if (!rope_table_) return;
  status_check(qllm_rope_table(rope_table_, rows, g_.rotary_dim, first_position,
                               g_.rope_theta, 0,
                               deferred_positions ? positions_ : nullptr,
                               stream_));
}

// RMSNorm of hidden_ into normalized_ (bf16), first adding the partials a
// K-split residual projection left behind.
// Per-row Q8 of `rows` F32 rows (quantize_rows, dense_fp4_provider.cpp:5983-
// 5992) into q8_ / q8_scales_, what the next projection reads.
void Mi355DenseFp4Provider::enqueue_quantise(const float* input,
                                             std::uint32_t rows,
                                             std::uint32_t columns) {
  status_check(qllm_quantize_q8_batch(input, q8_, q8_scales_, rows, columns,
                                      columns, 0, stream_));
}

// RMSNorm of `rows` rows of `input` into q8_ / q8_scales_: one launch where the
// fused kernel takes the row length, otherwise the norm and the quantisation.
void Mi355DenseFp4Provider::enqueue_normalise_q8(const float* input,
                                                 const float* weight,
                                                 std::uint32_t rows) {
  if (g_.hidden % 4U == 0U && g_.hidden <= 16384U) {
    status_check(qllm_rms_norm_q8_batch(input, weight, q8_, q8_scales_, rows,
                                        g_.hidden, g_.norm_epsilon,
                                        g_.zero_centered_norm, stream_));
    return;
  }
  status_check(qllm_rms_norm_batch(input, weight, activation_f32_, nullptr, 0U, rows,
                                   g_.hidden, g_.norm_epsilon,
                                   g_.zero_centered_norm, stream_));
  enqueue_quantise(activation_f32_, rows, g_.hidden);
}

void Mi355DenseFp4Provider::enqueue_normalise(const float* weight,
                                              std::uint32_t rows) {
  if (g_.activation_q8) {
    // normalize_rows then quantize_rows (:5740-5778, :5983-5992)
    if (pending_partials_)
      status_check(qllm_rms_norm_partials_q8_batch(
          hidden_, hidden_, projection_partials_, pending_partials_, weight, q8_,
          q8_scales_, rows, g_.hidden, g_.norm_epsilon, g_.zero_centered_norm,
          stream_));
    else
      enqueue_normalise_q8(hidden_, weight, rows);
    pending_partials_ = 0U;
    return;
  }
  if (pending_partials_)
    status_check(qllm_rms_norm_residual_batch(
        hidden_, projection_partials_, pending_partials_, weight, normalized_,
        rows, g_.hidden, g_.norm_epsilon, g_.zero_centered_norm, stream_));
  else
    status_check(qllm_rms_norm_batch(hidden_, weight, nullptr, normalized_,
                                     g_.hidden, rows, g_.hidden, g_.norm_epsilon,
                                     g_.zero_centered_norm, stream_));
  pending_partials_ = 0U;
}

// hidden_ += matrix * input, in the projection's epilogue or - when the
// caller lets the next norm finish the sum - as K-split partials.
void Mi355DenseFp4Provider::enqueue_residual_projection(
    const qllm_fp4_matrix& matrix, const std::uint16_t* input,
    std::size_t input_bytes, std::uint32_t rows, bool leave_partials) {
  const bool cut = leave_partials && projection_splits_ > 1U &&
                   matrix.layout == QLLM_LAYOUT_TILED &&
                   matrix.padded_columns / 64U >= projection_splits_;
  if (g_.activation_q8) {
    // the projection's input was quantised into q8_ by the caller
    if (cut && g_.hidden % 4U == 0U && g_.hidden <= 16384U) {
      status_check(qllm_fp4_gemm_q8_partial(&matrix, q8_, q8_scales_,
                                            projection_partials_, projection_splits_,
                                            rows, stream_));
      pending_partials_ = projection_splits_;
    } else {
      status_check(qllm_fp4_gemm_q8(&matrix, q8_, q8_scales_, hidden_, QLLM_OUT_F32,
                                    hidden_, rows, stream_));
    }
    return;
  }
  if (cut) {
    status_check(qllm_fp4_gemm_bf16_partial(&matrix, input, input_bytes,
                                            projection_partials_,
                                            projection_splits_, rows, stream_));
    pending_partials_ = projection_splits_;
  } else {
    status_check(qllm_fp4_gemm_bf16(&matrix, input, input_bytes, hidden_,
                                    QLLM_OUT_F32, hidden_, rows, stream_));
  }
}

// full attention block (run_full_attention, :6892)
void Mi355DenseFp4Provider::enqueue_attention_block(std::uint32_t index,
                                                    std::uint32_t rows,
                                                    std::uint32_t first_position,
                                                    bool deferred_positions,
                                                    bool leave_partials) {
  const auto& layer = layers_[index];
  const std::size_t hidden_bytes = std::size_t{rows} * g_.hidden * 2U;
  const std::size_t attention_bytes =
      std::size_t{rows} * g_.query_heads * g_.head_dim * 2U;
  enqueue_normalise(layer.input_norm, rows);
  // query, key and value projections (:7004-7011) in one launch
  const std::uint32_t kv_rows = g_.kv_heads * g_.head_dim;
  if (g_.activation_q8) {
    const qllm_gemm_segment projections[3] = {
        {query_, layer.qkv.descriptor.rows - 2U * kv_rows, QLLM_OUT_F32},
        {key_, kv_rows, QLLM_OUT_F32},
        {value_, kv_rows, QLLM_OUT_F32}};
    status_check(qllm_fp4_gemm_q8_split(&layer.qkv.descriptor, q8_, q8_scales_,
                                        projections, 3U, rows, gemm_workspace_,
                                        gemm_workspace_bytes_, stream_));
    // F32 attention output, quantised for the output projection (:7996)
    enqueue_attention(index, rows, first_position, deferred_positions, query_,
                      key_, value_,
                      reinterpret_cast<std::uint16_t*>(activation_f32_));
    enqueue_quantise(activation_f32_, rows, g_.query_heads * g_.head_dim);
    enqueue_residual_projection(layer.output.descriptor, nullptr, 0U, rows,
                                leave_partials);
    return;
  }
  const bool cut_qkv = qkv_splits_ > 1U &&
                       layer.qkv.descriptor.layout == QLLM_LAYOUT_TILED &&
                       layer.qkv.descriptor.padded_columns / 64U >= qkv_splits_;
  if (cut_qkv) {
    status_check(qllm_fp4_gemm_bf16_partial(&layer.qkv.descriptor, normalized_,
                                            hidden_bytes, qkv_partials_,
                                            qkv_splits_, rows, stream_));
    enqueue_attention(index, rows, first_position, deferred_positions, query_,
                      key_, value_, attention_, qkv_partials_, qkv_splits_);
  } else {
    const qllm_gemm_segment projections[3] = {
        {query_, layer.qkv.descriptor.rows - 2U * kv_rows, QLLM_OUT_F32},
        {key_, kv_rows, QLLM_OUT_F32},
        {value_, kv_rows, QLLM_OUT_F32}};
    status_check(qllm_fp4_gemm_bf16_split_balanced(
        &layer.qkv.descriptor, normalized_, hidden_bytes, projections, 3U, rows,
        gemm_workspace_, gemm_workspace_bytes_, stream_));
    enqueue_attention(index, rows, first_position, deferred_positions, query_,
                      key_, value_, attention_);
  }
  enqueue_residual_projection(layer.output.descriptor, attention_,
                              attention_bytes, rows, leave_partials);
}

// dense SwiGLU block (run_ffn, :8250-8293)
void Mi355DenseFp4Provider::enqueue_ffn_block(std::uint32_t index,
                                              std::uint32_t rows,
                                              bool leave_partials) {
  const auto& layer = layers_[index];
  enqueue_normalise(layer.post_attention_norm, rows);
  if (g_.activation_q8) {
    // one quantisation shared by gate and up, the F32 SiLU product quantised
    // again for the down projection (run_ffn, :8258-8290)
    status_check(qllm_fp4_swiglu_q8(&layer.gate.descriptor, &layer.up.descriptor,
                                    q8_, q8_scales_, activation_f32_, rows,
                                    gemm_workspace_, gemm_workspace_bytes_,
                                    stream_));
    enqueue_quantise(activation_f32_, rows, g_.intermediate);
    enqueue_residual_projection(layer.down.descriptor, nullptr, 0U, rows,
                                leave_partials);
    return;
  }
  status_check(qllm_fp4_swiglu_bf16_balanced(
      &layer.gate.descriptor, &layer.up.descriptor, normalized_,
      std::size_t{rows} * g_.hidden * 2U, activation_, rows, gemm_workspace_,
      gemm_workspace_bytes_, stream_));
  enqueue_residual_projection(layer.down.descriptor, activation_,
                              std::size_t{rows} * g_.intermediate * 2U, rows,
                              leave_partials);
}

// head (run_head, :8393-8432) on rows [first_row, first_row + rows) of
// hidden_: logits_ [rows, vocabulary] and their arg-max tokens.  The norm
// also completes hidden_ when partials are pending, which is only so for a
// head over all rows.
void Mi355DenseFp4Provider::enqueue_head(std::uint32_t first_row,
                                         std::uint32_t rows) {
  if (pending_partials_ && first_row != 0U)
    throw std::runtime_error("head over a row range needs a complete hidden state");
  if (g_.activation_q8) {
    if (first_row == 0U)
      enqueue_normalise(final_norm_, rows);   // finishes a cut projection too
    else
      enqueue_normalise_q8(hidden_ + std::size_t{first_row} * g_.hidden, final_norm_,
                           rows);
    status_check(qllm_fp4_gemm_q8(&head_.descriptor, q8_, q8_scales_, logits_,
                                  QLLM_OUT_F32, nullptr, rows, stream_));
    status_check(qllm_argmax_batch(logits_, g_.vocabulary, rows, argmax_tokens_,
                                   select_workspace_, select_workspace_bytes_,
                                   stream_));
    return;
  }
  if (first_row == 0U) {
    enqueue_normalise(final_norm_, rows);
  } else {
    status_check(qllm_rms_norm_batch(
        hidden_ + std::size_t{first_row} * g_.hidden, final_norm_, nullptr,
        normalized_, g_.hidden, rows, g_.hidden, g_.norm_epsilon,
        g_.zero_centered_norm, stream_));
  }
  enqueue_head_projection(head_.descriptor, normalized_, logits_, rows,
                          argmax_tokens_, nullptr);
}

// logits = head . normalized_ and their arg-max tokens: the projection's
// epilogue leaves the tiles' maxima for a one-block launch to finish (with
// `advance`, which also hands the winner to the next proposer pass); matrices
// the matrix-core kernel does not take go through the plain arg-max.
void Mi355DenseFp4Provider::enqueue_head_projection(
    const qllm_fp4_matrix& head, const std::uint16_t* input, float* logits,
    std::uint32_t rows, std::uint32_t* tokens, const qllm_rollout_step* advance) {
  const std::size_t input_bytes = std::size_t{rows} * g_.hidden * 2U;
  if (head.padded_columns % 64U == 0U &&
      qllm_fp4_head_workspace_bytes(&head, rows) <= select_workspace_bytes_) {
    status_check(qllm_fp4_head_argmax(&head, input, input_bytes, logits, rows,
                                      tokens, select_workspace_,
                                      select_workspace_bytes_, advance, stream_));
    return;
  }
  status_check(qllm_fp4_gemm_bf16(&head, input, input_bytes, logits,
                                  QLLM_OUT_F32, nullptr, rows, stream_));
  status_check(qllm_argmax_batch(logits, head.rows, rows, tokens, select_workspace_,
                                 select_workspace_bytes_, stream_));
  if (advance)
    status_check(qllm_rollout_advance(tokens, advance->next_token,
                                      advance->draft_tokens, advance->capacity,
                                      advance->rows, advance->device_positions,
                                      stream_));
}

void Mi355DenseFp4Provider::enqueue_target(const std::uint32_t* device_tokens,
                                           std::uint32_t rows,
                                           std::uint32_t first_position,
                                           bool deferred_positions) {
  // with phase timing on, an event pair around every operation (nothing is
  // recorded otherwise, and never into a captured graph: profiling passes run
  // uncaptured)
  const auto timed = [this](GpuPhase phase, auto&& enqueue) {
    const auto events = begin_gpu_phase(phase);
    enqueue();
    end_gpu_phase(events);
  };
  timed(GpuPhase::embedding, [&] {
    status_check(qllm_fp4_embedding_batch(&embedding_.descriptor, device_tokens,
                                          hidden_, rows, stream_));
    enqueue_rope_table(rows, first_position, deferred_positions);
  });
  pending_partials_ = 0U;
  for (std::uint32_t index = 0; index < g_.layers; ++index) {
    timed(GpuPhase::full_attention, [&] {
      enqueue_attention_block(index, rows, first_position, deferred_positions,
                              true);
    });
    timed(GpuPhase::ffn, [&] { enqueue_ffn_block(index, rows, true); });
  }
  timed(GpuPhase::head, [&] { enqueue_head(0U, rows); });
}

// The proposer's pass over a prompt chunk: row r pairs tokens[r] (the token
// after prompt position `position` + r) with the target's hidden state of that
// position, which prefill() left in prefill_hidden_.  The operations of
// enqueue_mtp up to the key / value store, on the tall-batch GEMM and the
// Q8 cache store; writes the proposer's cache records position .. position +
// rows - 1 and reuses the prefill buffers (prefill_hidden_ becomes the
// proposer's residual stream).
void Mi355DenseFp4Provider::enqueue_mtp_prefill(
    std::span<const std::uint32_t> tokens, std::uint32_t position) {
  void* const stream = stream_;
  const auto hip_stream = static_cast<hipStream_t>(stream_);
  const auto rows = static_cast<std::uint32_t>(tokens.size());
  const auto& layer = mtp_.layer;
  const std::size_t hidden_bytes = std::size_t{rows} * g_.hidden * 2U;
  const std::uint32_t query_stride = g_.head_dim * (g_.output_gated ? 2U : 1U);
  float* const embedding = prefill_embedding_;            // f32 [rows, hidden]
  std::uint16_t* const fusion_input = prefill_activation_;  // bf16 [rows, 2 hidden]
  hip_check(hipMemcpyAsync(prefill_tokens_, tokens.data(), rows * 4U,
                           hipMemcpyHostToDevice, hip_stream),
            "upload the proposer's prompt tokens");
  status_check(qllm_fp4_embedding_batch(&embedding_.descriptor, prefill_tokens_,
                                        embedding, rows, stream));
  status_check(qllm_rms_norm_concat_batch(
      embedding, mtp_.embedding_norm, prefill_hidden_, mtp_.hidden_norm,
      fusion_input, rows, g_.hidden, g_.norm_epsilon, g_.zero_centered_norm,
      stream));
  status_check(qllm_fp4_gemm_bf16_tall(&mtp_.fusion.descriptor, fusion_input,
                                       2U * hidden_bytes, prefill_hidden_,
                                       QLLM_OUT_F32, nullptr, rows, stream));
  status_check(qllm_rms_norm_batch(prefill_hidden_, layer.input_norm, nullptr,
                                   prefill_normalized_, g_.hidden, rows,
                                   g_.hidden, g_.norm_epsilon,
                                   g_.zero_centered_norm, stream));
  const std::uint32_t kv_rows = g_.kv_heads * g_.head_dim;
  const qllm_gemm_segment projections[3] = {
      {prefill_query_, layer.qkv.descriptor.rows - 2U * kv_rows, QLLM_OUT_F32},
      {prefill_key_, kv_rows, QLLM_OUT_F32},
      {prefill_value_, kv_rows, QLLM_OUT_F32}};
  status_check(qllm_fp4_gemm_bf16_tall_split(&layer.qkv.descriptor,
                                             prefill_normalized_, hidden_bytes,
                                             projections, 3U, rows, stream));
  const auto pages = const_cast<const void* const*>(device_page_table_);
  // the proposer's cache lags the target's by one token: record `position`
  // carries rotary position `position` + 1 (enqueue_mtp)
  status_check(qllm_qkv_rope_batch(
      prefill_query_, query_stride, prefill_key_, layer.query_norm,
      layer.key_norm, position + 1U, rows, g_.query_heads, g_.kv_heads,
      g_.head_dim, g_.rotary_dim, g_.norm_epsilon, g_.rope_theta, 0, stream));
  status_check(qllm_store_kv_paged_q8_batch(
      prefill_key_, prefill_value_, pages, mtp_page_offset_, g_.kv_page_tokens,
      position, rows, g_.kv_heads, g_.head_dim, stream));
  // The pass ends with the cache records: the proposer has one layer and a
  // prompt pass asks for no draft, so nothing reads what its attention and
  // MLP would compute.
}

// The buffers of a prompt pass of up to `rows` rows.  A longer prompt than any
// before replaces them by larger ones (the stream is idle between prefills).
void Mi355DenseFp4Provider::ensure_prefill_workspace(std::uint32_t rows) {
  if (rows <= prefill_rows_) return;
  const auto release = [this] {
    for (void* pointer : prefill_allocations_) (void)hipFree(pointer);
    prefill_allocations_.clear();
    prefill_rows_ = 0U;
  };
  if (prefill_rows_) {
    hip_check(hipStreamSynchronize(static_cast<hipStream_t>(stream_)),
              "drain the stream before the prefill workspace grows");
    release();
  }
  // an allocation that fails part-way leaves no workspace at all rather than
  // a mix of new and dangling buffers: the next prompt starts over
  const auto allocate = [this, &release](std::size_t bytes) {
    void* pointer{};
    if (const auto error = hipMalloc(&pointer, bytes); error != hipSuccess) {
      release();
      hip_check(error, "allocate prefill workspace");
    }
    prefill_allocations_.push_back(pointer);
    return pointer;
  };
  const std::size_t n = rows;
  const std::size_t query_width =
      std::size_t{g_.query_heads} * g_.head_dim * (g_.output_gated ? 2U : 1U);
  const std::size_t kv_width = std::size_t{g_.kv_heads} * g_.head_dim;
  prefill_tokens_ = static_cast<std::uint32_t*>(allocate(n * 4U));
  prefill_hidden_ = static_cast<float*>(allocate(n * g_.hidden * 4U));
  prefill_normalized_ =
      static_cast<std::uint16_t*>(allocate(n * g_.hidden * 2U));
  prefill_query_ = static_cast<float*>(allocate(n * query_width * 4U));
  prefill_key_ = static_cast<float*>(allocate(n * kv_width * 4U));
  prefill_value_ = static_cast<float*>(allocate(n * kv_width * 4U));
  prefill_attention_ = static_cast<std::uint16_t*>(
      allocate(n * g_.query_heads * g_.head_dim * 2U));
  prefill_embedding_ = static_cast<float*>(allocate(n * g_.hidden * 4U));
  // the MLP's activation; the proposer's fusion input [rows, 2 hidden] too
  prefill_activation_ = static_cast<std::uint16_t*>(allocate(
      n * std::max<std::size_t>(g_.intermediate, 2U * g_.hidden) * 2U));
  {
    // fewer splits than the verify step: the row batches of a chunk already
    // fill the GPU, and the partials are per row
    prefill_splits_ = std::min<std::uint32_t>(maximum_splits_, 8U);
    // partial rows: the most rows x splits any chunk of up to n rows asks for
    // (long chunks are not cut, short ones have few rows)
    const std::uint32_t attention_batch = std::max(
        1U, (g_.head_dim == 256U ? 32U : 48U) / (g_.query_heads / g_.kv_heads));
    std::size_t partial_rows = 0;
    for (std::uint32_t chunk = 1; chunk <= rows; ++chunk)
      partial_rows = std::max<std::size_t>(
          partial_rows,
          std::size_t{chunk} *
              std::max(prefill_splits_for(chunk, attention_batch),
                       prompt_attention_splits(chunk, attention_batch)));
    const std::size_t partials = partial_rows * g_.query_heads;
    prefill_partial_maxima_ = static_cast<float*>(allocate(partials * 4U));
    prefill_partial_sums_ = static_cast<float*>(allocate(partials * 4U));
    prefill_partial_outputs_ =
        static_cast<float*>(allocate(partials * g_.head_dim * 4U));
  }
  prefill_rows_ = rows;
}

Mi355DenseFp4Provider::PrefillResult Mi355DenseFp4Provider::prefill(
    const std::shared_ptr<er::IOperationProviderRequestState>& opaque_state,
    std::span<const std::uint32_t> tokens, std::uint32_t first_position,
    const er::ProgramRequestContext& request) {
  try {
    std::lock_guard lock(mutex_);
    const auto state =
        std::dynamic_pointer_cast<DenseFp4RequestState>(opaque_state);
    if (tokens.empty() || tokens.size() > g_.max_context ||
        first_position > g_.max_context - tokens.size() ||
        (opaque_state && !state))
      return {{er::ErrorCode::invalid_argument, "prompt rows are invalid"}, 0U};
    if (!embedding_ready_ || !head_ready_ || attention_ops_ != g_.layers ||
        ffn_ops_ != g_.layers)
      return {{er::ErrorCode::invalid_argument, "target program is not prepared"},
              0U};
    if (g_.activation_q8)
      return {{er::ErrorCode::invalid_argument,
               "the tall prompt path takes bf16 activation input; with Q8 "
               "activations a prompt goes through the program in row batches"},
              0U};
    for (const auto token : tokens)
      if (token >= g_.vocabulary)
        return {{er::ErrorCode::invalid_argument,
                 "prompt token is outside the vocabulary"},
                0U};
    if (state) activate(state->slot);
    const auto count = static_cast<std::uint32_t>(tokens.size());
    // sized for the pass this prompt needs, in steps of 4096 rows
    ensure_prefill_workspace(std::min(
        std::min(prefill_chunk_rows(), g_.max_context),
        (std::min(count, prefill_chunk_rows()) + 4095U) / 4096U * 4096U));
    ensure_pages(first_position + count - 1U);
    void* const stream = stream_;
    const auto hip_stream = static_cast<hipStream_t>(stream_);
    const std::size_t query_width =
        std::size_t{g_.query_heads} * g_.head_dim * (g_.output_gated ? 2U : 1U);
    const std::size_t kv_width = std::size_t{g_.kv_heads} * g_.head_dim;
    const std::size_t attention_width = std::size_t{g_.query_heads} * g_.head_dim;
    // a request that will not be decoded speculatively keeps the proposer out
    // (the runner synchronises only exact-eligible requests,
    // runtime/tools/moe_vm_runner.cpp:735-745)
    const auto exact_enabled = request.parameters.find("exact_decode_enabled");
    const bool feed_proposer =
        state && mtp_.ready &&
        (exact_enabled == request.parameters.end() || exact_enabled->second != 0U);
    // query rows per attention workgroup: as many as the kernels' three (two at
    // head_dim 256) 16-row tiles hold for one KV head's group of query heads
    const std::uint32_t attention_batch = std::max(
        1U, (g_.head_dim == 256U ? 32U : 48U) / (g_.query_heads / g_.kv_heads));
    if (state) {
      state->draft_valid = false;
      state->draft_predictions.clear();
      state->mtp_length = first_position;
    }

    for (std::uint32_t done = 0; done < count;) {
      const std::uint32_t rows = std::min(prefill_rows_, count - done);
      const std::uint32_t position = first_position + done;
      hip_check(hipMemcpyAsync(prefill_tokens_, tokens.data() + done, rows * 4U,
                               hipMemcpyHostToDevice, hip_stream),
                "upload prompt tokens");
      status_check(qllm_fp4_embedding_batch(&embedding_.descriptor,
                                            prefill_tokens_, prefill_hidden_,
                                            rows, stream));
      const std::size_t hidden_bytes = std::size_t{rows} * g_.hidden * 2U;
      for (std::uint32_t index = 0; index < g_.layers; ++index) {
        const auto& layer = layers_[index];
        status_check(qllm_rms_norm_batch(
            prefill_hidden_, layer.input_norm, nullptr, prefill_normalized_,
            g_.hidden, rows, g_.hidden, g_.norm_epsilon, g_.zero_centered_norm,
            stream));
        const std::uint32_t kv_rows = g_.kv_heads * g_.head_dim;
        const qllm_gemm_segment projections[3] = {
            {prefill_query_, layer.qkv.descriptor.rows - 2U * kv_rows, QLLM_OUT_F32},
            {prefill_key_, kv_rows, QLLM_OUT_F32},
            {prefill_value_, kv_rows, QLLM_OUT_F32}};
        status_check(qllm_fp4_gemm_bf16_tall_split(
            &layer.qkv.descriptor, prefill_normalized_, hidden_bytes,
            projections, 3U, rows, stream));
        // attention in row batches of the verify step's size: each batch sees
        // the cache up to and including its own rows
        if (g_.kv_encoding == KvEncoding::q4_f16_per_head) {
          // every row's K/V record first, then all batches in one launch
          const std::uint32_t query_stride =
              g_.head_dim * (g_.output_gated ? 2U : 1U);
          const auto pages = const_cast<const void* const*>(device_page_table_);
          status_check(qllm_qkv_rope_cache_paged_q4h_batch(
              prefill_query_, query_stride, prefill_key_, prefill_value_,
              layer.query_norm, layer.key_norm, pages, index, g_.kv_page_tokens,
              position, position, rows, g_.query_heads, g_.kv_heads, g_.head_dim,
              g_.rotary_dim, g_.norm_epsilon, g_.rope_theta, 0, stream));
          qllm_q4h_attention_launch launch{};
          launch.query = prefill_query_;
          launch.page_table = pages;
          launch.output = prefill_attention_;
          launch.partial_maxima = prefill_partial_maxima_;
          launch.partial_sums = prefill_partial_sums_;
          launch.partial_outputs = prefill_partial_outputs_;
          launch.first_context_tokens = position + 1U;
          launch.rows = rows;
          launch.full_attention_layer = index;
          launch.page_tokens = g_.kv_page_tokens;
          launch.query_heads = g_.query_heads;
          launch.kv_heads = g_.kv_heads;
          launch.head_dim = g_.head_dim;
          launch.split_tokens = 0U;
          launch.query_stride = query_stride;
          launch.output_gated = g_.output_gated;
          launch.output_kind = QLLM_OUT_BF16;
          launch.stream = stream;
          // From 32 row batches on, eight batches share a workgroup and every
          // cache tile it fetches and converts; the context is then cut as far
          // as it takes to give every CU one of those workgroups.
          if (const std::uint32_t splits =
                  prompt_attention_splits(rows, attention_batch)) {
            launch.maximum_splits = splits;
            status_check(qllm_attention_paged_q4h_prompt(&launch, attention_batch));
          } else {
            launch.maximum_splits = prefill_splits_for(rows, attention_batch);
            status_check(
                qllm_attention_paged_q4h_batched(&launch, attention_batch));
          }
        } else {
          const std::uint32_t query_stride =
              g_.head_dim * (g_.output_gated ? 2U : 1U);
          const auto pages = const_cast<const void* const*>(device_page_table_);
          status_check(qllm_qkv_rope_batch(
              prefill_query_, query_stride, prefill_key_, layer.query_norm,
              layer.key_norm, position, rows, g_.query_heads, g_.kv_heads,
              g_.head_dim, g_.rotary_dim, g_.norm_epsilon, g_.rope_theta, 0,
              stream));
          status_check(qllm_store_kv_paged_f16_batch(
              prefill_key_, prefill_value_, pages, index, g_.kv_page_tokens,
              position, rows, g_.kv_heads, g_.head_dim, stream));
          qllm_f16_attention_launch launch{};
          launch.query = prefill_query_;
          launch.device_pages = pages;
          launch.output = prefill_attention_;
          launch.partial_maxima = prefill_partial_maxima_;
          launch.partial_sums = prefill_partial_sums_;
          launch.partial_outputs = prefill_partial_outputs_;
          launch.first_context_tokens = position + 1U;
          launch.rows = rows;
          launch.device_page_layer = index;
          launch.device_page_tokens = g_.kv_page_tokens;
          launch.query_heads = g_.query_heads;
          launch.kv_heads = g_.kv_heads;
          launch.head_dim = g_.head_dim;
          launch.split_tokens = 0U;
          launch.maximum_splits = prefill_splits_for(rows, attention_batch);
          launch.query_stride = query_stride;
          launch.output_gated = g_.output_gated;
          launch.output_kind = QLLM_OUT_BF16;
          launch.stream = stream;
          status_check(qllm_attention_paged_f16_batched(&launch, attention_batch));
        }
        status_check(qllm_fp4_gemm_bf16_tall(
            &layer.output.descriptor, prefill_attention_,
            std::size_t{rows} * attention_width * 2U, prefill_hidden_,
            QLLM_OUT_F32, prefill_hidden_, rows, stream));
        status_check(qllm_rms_norm_batch(
            prefill_hidden_, layer.post_attention_norm, nullptr,
            prefill_normalized_, g_.hidden, rows, g_.hidden, g_.norm_epsilon,
            g_.zero_centered_norm, stream));
        // gate and up in one launch; silu(gate) * up leaves it in bf16 with
        // the verify step's rounding points
        status_check(qllm_fp4_swiglu_bf16_tall(
            &layer.gate.descriptor, &layer.up.descriptor, prefill_normalized_,
            hidden_bytes, prefill_activation_, rows, stream));
        status_check(qllm_fp4_gemm_bf16_tall(
            &layer.down.descriptor, prefill_activation_,
            std::size_t{rows} * g_.intermediate * 2U, prefill_hidden_,
            QLLM_OUT_F32, prefill_hidden_, rows, stream));
      }
      if (done + rows == count) {
        // last row -> the verify step's buffers, then the head on that row
        hip_check(hipMemcpyAsync(
                      hidden_, prefill_hidden_ + std::size_t{rows - 1U} * g_.hidden,
                      g_.hidden * 4U, hipMemcpyDeviceToDevice, hip_stream),
                  "retain the prompt's last hidden state");
      }
      // the proposer sees (token at p + 1, target hidden at p) for every prompt
      // position but the last, whose successor is not known yet
      if (feed_proposer) {
        const std::uint32_t pairs = done + rows == count ? rows - 1U : rows;
        const bool tall = g_.hidden <= 16384U &&
                          mtp_.fusion.descriptor.layout == QLLM_LAYOUT_TILED;
        if (pairs && tall) {
          enqueue_mtp_prefill(tokens.subspan(done + 1U, pairs), position);
          state->mtp_length += pairs;
          ++mtp_passes_;
          mtp_rows_ += pairs;
        } else {
          for (std::uint32_t row = 0; row < pairs; row += max_rows_) {
            const std::uint32_t batch = std::min(max_rows_, pairs - row);
            (void)run_mtp(*state, tokens.subspan(done + row + 1U, batch),
                          prefill_hidden_ + std::size_t{row} * g_.hidden, false,
                          nullptr, nullptr, 0U, 0U);
          }
        }
      }
      done += rows;
    }
    status_check(qllm_rms_norm_batch(hidden_, final_norm_, nullptr, normalized_,
                                     g_.hidden, 1U, g_.hidden, g_.norm_epsilon,
                                     g_.zero_centered_norm, stream));
    status_check(qllm_fp4_gemm_bf16(&head_.descriptor, normalized_,
                                    std::size_t{g_.hidden} * 2U, logits_,
                                    QLLM_OUT_F32, nullptr, 1U, stream));
    status_check(qllm_argmax_batch(logits_, g_.vocabulary, 1U, argmax_tokens_,
                                   select_workspace_, select_workspace_bytes_,
                                   stream));
    std::uint32_t predicted{};
    if (request.parameters.contains("sampling_temperature_ppm")) {
      // the head under the request's sampling profile, at the position of the
      // prompt's last token (run_head with a request, :8433-8517)
      predicted = select_head_token(request, first_position + count - 1U);
    } else {
      hip_check(hipMemcpyAsync(&predicted, argmax_tokens_, sizeof(predicted),
                               hipMemcpyDeviceToHost, hip_stream),
                "copy the prompt's prediction");
      hip_check(hipStreamSynchronize(hip_stream), "prompt prefill");
    }
    prefill_tokens_total_ += count;
    if (state) {
      state->synchronized_token = predicted;
      if (feed_proposer) {
        // the last pair, then the first drafts (as synchronize does)
        const std::uint32_t last[1] = {predicted};
        const auto sample_position = first_position + count;
        hip_check(hipMemcpyAsync(proposal_presence_, presence_, g_.vocabulary,
                                 hipMemcpyDeviceToDevice, hip_stream),
                  "initialize speculative proposal presence");
        auto draft = run_mtp(*state, last, hidden_, true, &request,
                             proposal_presence_, sample_position, 1U);
        if (!draft) throw std::runtime_error("prompt prefill produced no draft");
        const auto reserved = request.parameters.find("reserved_context_tokens");
        const auto context_limit =
            reserved == request.parameters.end()
                ? g_.max_context
                : static_cast<std::uint32_t>(reserved->second);
        if (state->mtp_length + 1U < context_limit)
          extend_mtp_rollout(*state, request, std::move(*draft), context_limit);
      } else {
        state->mtp_length = first_position + count;
      }
    }
    return {er::Status::success(), predicted};
  } catch (const std::exception& error) {
    return {{er::ErrorCode::internal, error.what()}, 0U};
  }
}

er::Status Mi355DenseFp4Provider::run_target(const std::uint32_t* tokens,
                                             std::uint32_t rows,
                                             std::uint32_t first_position) {
  try {
    if (!tokens || !rows || rows > max_rows_ ||
        first_position > g_.max_context - rows)
      return {er::ErrorCode::invalid_argument, "target rows are invalid"};
    if (!embedding_ready_ || !head_ready_)
      return {er::ErrorCode::invalid_argument, "target program is not prepared"};
    ensure_pages(first_position + rows - 1U);
    hip_check(hipMemcpyAsync(tokens_, tokens, rows * sizeof(std::uint32_t),
                             hipMemcpyHostToDevice,
                             static_cast<hipStream_t>(stream_)),
              "upload target tokens");
    enqueue_target(tokens_, rows, first_position, false);
    collect_gpu_phases();
    return er::Status::success();
  } catch (const std::exception& error) {
    return {er::ErrorCode::internal, error.what()};
  }
}

er::Status Mi355DenseFp4Provider::run_target_graph(const std::uint32_t* tokens,
                                                   std::uint32_t rows,
                                                   std::uint32_t first_position) {
  if (g_.kv_encoding != KvEncoding::q4_f16_per_head)
    return run_target(tokens, rows, first_position);
  try {
    if (!tokens || !rows || rows > max_rows_ ||
        first_position > g_.max_context - rows)
      return {er::ErrorCode::invalid_argument, "target rows are invalid"};
    if (!embedding_ready_ || !head_ready_)
      return {er::ErrorCode::invalid_argument, "target program is not prepared"};
    ensure_pages(first_position + rows - 1U);
    const auto stream = static_cast<hipStream_t>(stream_);
    // The stream is idle here (every pass ends with a wait), so the pinned
    // words of the previous pass have been read.
    std::copy(tokens, tokens + rows, staging_->target);
    const std::uint32_t positions[4] = {first_position, first_position,
                                        first_position + 1U, rows};
    std::copy(positions, positions + 4, staging_->target + 8);
    hip_check(hipMemcpyAsync(tokens_, staging_->target, sizeof(staging_->target),
                             hipMemcpyHostToDevice, stream),
              "upload target tokens and positions");
    if (!graphs_[rows]) {
      hip_check(hipStreamSynchronize(stream), "drain stream before capture");
      hipGraph_t graph{};
      hip_check(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal),
                "begin target capture");
      try {
        enqueue_target(tokens_, rows, first_position, true);
      } catch (...) {
        (void)hipStreamEndCapture(stream, &graph);
        if (graph) (void)hipGraphDestroy(graph);
        throw;
      }
      hip_check(hipStreamEndCapture(stream, &graph), "end target capture");
      hipGraphExec_t exec{};
      const auto status = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
      (void)hipGraphDestroy(graph);
      hip_check(status, "instantiate target graph");
      graphs_[rows] = exec;
    }
    hip_check(hipGraphLaunch(static_cast<hipGraphExec_t>(graphs_[rows]), stream),
              "launch target graph");
    last_graph_rows_ = rows;
    return er::Status::success();
  } catch (const std::exception& error) {
    return {er::ErrorCode::internal, error.what()};
  }
}

er::Status Mi355DenseFp4Provider::capture_target_graph(
    const std::uint32_t* tokens, std::uint32_t rows,
    std::uint32_t first_position) {
  return run_target_graph(tokens, rows, first_position);
}

er::Status Mi355DenseFp4Provider::replay_target_graph() {
  if (!last_graph_rows_ || !graphs_[last_graph_rows_])
    return {er::ErrorCode::invalid_argument, "no target graph was captured"};
  const auto status =
      hipGraphLaunch(static_cast<hipGraphExec_t>(graphs_[last_graph_rows_]),
                     static_cast<hipStream_t>(stream_));
  if (status != hipSuccess)
    return {er::ErrorCode::internal, hipGetErrorString(status)};
  return er::Status::success();
}

er::Status Mi355DenseFp4Provider::time_kernel(const std::string& which,
                                              std::uint32_t rounds,
                                              std::uint32_t context_tokens,
                                              double* microseconds,
                                              std::uint64_t* launches) {
  try {
    std::lock_guard lock(mutex_);
    if (!microseconds || !launches || !rounds || !head_ready_)
      return {er::ErrorCode::invalid_argument, "kernel timing request is invalid"};
    const auto stream = static_cast<hipStream_t>(stream_);
    const std::uint32_t rows = max_rows_;
    const std::size_t hidden_bytes = std::size_t{rows} * g_.hidden * 2U;
    const std::uint32_t query_stride = g_.head_dim * (g_.output_gated ? 2U : 1U);
    if (which == "attention") {
      if (!context_tokens || context_tokens + rows > g_.max_context)
        return {er::ErrorCode::invalid_argument, "timing context is invalid"};
      ensure_pages(context_tokens + rows - 1U);
      // the attention launches rotate and store the batch themselves
      enqueue_rope_table(rows, context_tokens, false);
    }
    const auto launch_one = [&](std::uint32_t index) {
      const auto& layer = layers_[index % g_.layers];
      if (g_.activation_q8 && which != "attention") {
        // the Q8 forms of the same launches (inputs: whatever q8_ holds)
        const std::uint32_t kv_rows = g_.kv_heads * g_.head_dim;
        if (which == "ffn_gate_up") {
          status_check(qllm_fp4_swiglu_q8(&layer.gate.descriptor,
                                          &layer.up.descriptor, q8_, q8_scales_,
                                          activation_f32_, rows, gemm_workspace_,
                                          gemm_workspace_bytes_, stream_));
        } else if (which == "ffn_down") {
          // as the target pass launches it
          if (projection_splits_ > 1U &&
              layer.down.descriptor.padded_columns / 64U >= projection_splits_)
            status_check(qllm_fp4_gemm_q8_partial(
                &layer.down.descriptor, q8_, q8_scales_, projection_partials_,
                projection_splits_, rows, stream_));
          else
            status_check(qllm_fp4_gemm_q8(&layer.down.descriptor, q8_, q8_scales_,
                                          query_, QLLM_OUT_F32, nullptr, rows,
                                          stream_));
        } else if (which == "qkv") {
          const qllm_gemm_segment projections[3] = {
              {query_, layer.qkv.descriptor.rows - 2U * kv_rows, QLLM_OUT_F32},
              {key_, kv_rows, QLLM_OUT_F32},
              {value_, kv_rows, QLLM_OUT_F32}};
          status_check(qllm_fp4_gemm_q8_split(&layer.qkv.descriptor, q8_, q8_scales_,
                                              projections, 3U, rows, gemm_workspace_,
                                              gemm_workspace_bytes_, stream_));
        } else if (which == "attention_output") {
          if (projection_splits_ > 1U &&
              layer.output.descriptor.padded_columns / 64U >= projection_splits_)
            status_check(qllm_fp4_gemm_q8_partial(
                &layer.output.descriptor, q8_, q8_scales_, projection_partials_,
                projection_splits_, rows, stream_));
          else
            status_check(qllm_fp4_gemm_q8(&layer.output.descriptor, q8_, q8_scales_,
                                          query_, QLLM_OUT_F32, nullptr, rows,
                                          stream_));
        } else if (which == "lm_head") {
          status_check(qllm_fp4_gemm_q8(&head_.descriptor, q8_, q8_scales_, logits_,
                                        QLLM_OUT_F32, nullptr, rows, stream_));
        } else {
          throw std::runtime_error("unknown kernel name: " + which);
        }
      } else if (which == "ffn_gate_up") {
        status_check(qllm_fp4_swiglu_bf16_balanced(
            &layer.gate.descriptor, &layer.up.descriptor, normalized_, hidden_bytes,
            activation_, rows, gemm_workspace_, gemm_workspace_bytes_, stream_));
      } else if (which == "ffn_down") {
        // as the target pass launches it
        const auto& down = layer.down.descriptor;
        if (projection_splits_ > 1U && down.layout == QLLM_LAYOUT_TILED &&
            down.padded_columns / 64U >= projection_splits_)
          status_check(qllm_fp4_gemm_bf16_partial(
              &down, activation_, std::size_t{rows} * g_.intermediate * 2U,
              projection_partials_, projection_splits_, rows, stream_));
        else
          status_check(qllm_fp4_gemm_bf16(
              &down, activation_, std::size_t{rows} * g_.intermediate * 2U,
              query_, QLLM_OUT_F32, nullptr, rows, stream_));
      } else if (which == "qkv") {
        // as the target pass launches it
        const auto& qkv = layer.qkv.descriptor;
        const std::uint32_t kv_rows = g_.kv_heads * g_.head_dim;
        if (qkv_splits_ > 1U && qkv.layout == QLLM_LAYOUT_TILED &&
            qkv.padded_columns / 64U >= qkv_splits_) {
          status_check(qllm_fp4_gemm_bf16_partial(&qkv, normalized_, hidden_bytes,
                                                  qkv_partials_, qkv_splits_,
                                                  rows, stream_));
        } else {
          const qllm_gemm_segment projections[3] = {
              {query_, qkv.rows - 2U * kv_rows, QLLM_OUT_F32},
              {key_, kv_rows, QLLM_OUT_F32},
              {value_, kv_rows, QLLM_OUT_F32}};
          status_check(qllm_fp4_gemm_bf16_split_balanced(
              &qkv, normalized_, hidden_bytes, projections, 3U, rows,
              gemm_workspace_, gemm_workspace_bytes_, stream_));
        }
      } else if (which == "attention_output") {
        const auto& output = layer.output.descriptor;
        const std::size_t bytes =
            std::size_t{rows} * g_.query_heads * g_.head_dim * 2U;
        if (projection_splits_ > 1U && output.layout == QLLM_LAYOUT_TILED &&
            output.padded_columns / 64U >= projection_splits_)
          status_check(qllm_fp4_gemm_bf16_partial(&output, attention_, bytes,
                                                  projection_partials_,
                                                  projection_splits_, rows,
                                                  stream_));
        else
          status_check(qllm_fp4_gemm_bf16(&output, attention_, bytes, query_,
                                          QLLM_OUT_F32, nullptr, rows, stream_));
      } else if (which == "lm_head") {
        status_check(qllm_fp4_gemm_bf16(&head_.descriptor, normalized_,
                                        hidden_bytes, logits_, QLLM_OUT_F32,
                                        nullptr, rows, stream_));
      } else if (which == "attention" && g_.kv_encoding == KvEncoding::fp16) {
        qllm_f16_attention_launch launch{};
        launch.query = query_;
        launch.device_pages = const_cast<const void* const*>(device_page_table_);
        launch.output = attention_;
        launch.partial_maxima = partial_maxima_;
        launch.partial_sums = partial_sums_;
        launch.partial_outputs = partial_outputs_;
        launch.first_context_tokens = context_tokens + 1U;
        launch.rows = rows;
        launch.device_page_layer = index % g_.layers;
        launch.device_page_tokens = g_.kv_page_tokens;
        launch.query_heads = g_.query_heads;
        launch.kv_heads = g_.kv_heads;
        launch.head_dim = g_.head_dim;
        launch.split_tokens = split_tokens_;
        launch.maximum_splits = maximum_splits_;
        launch.query_stride = query_stride;
        launch.output_gated = g_.output_gated;
        launch.output_kind = QLLM_OUT_BF16;
        launch.stream = stream_;
        status_check(qllm_attention_paged_f16(&launch));
      } else if (which == "attention") {
        qllm_q4h_attention_launch launch{};
        launch.query = query_;
        launch.page_table = const_cast<const void* const*>(device_page_table_);
        launch.output = attention_;
        launch.partial_maxima = partial_maxima_;
        launch.partial_sums = partial_sums_;
        launch.partial_outputs = partial_outputs_;
        launch.first_context_tokens = context_tokens + 1U;
        launch.rows = rows;
        launch.full_attention_layer = index % g_.layers;
        launch.page_tokens = g_.kv_page_tokens;
        launch.query_heads = g_.query_heads;
        launch.kv_heads = g_.kv_heads;
        launch.head_dim = g_.head_dim;
        launch.split_tokens = split_tokens_;
        launch.maximum_splits = maximum_splits_;
        launch.query_stride = query_stride;
        launch.output_gated = g_.output_gated;
        launch.output_kind = QLLM_OUT_BF16;
        launch.stream = stream_;
        // as the target pass launches it
        qllm_q4h_fused_rope rope{};
        rope.key = key_;
        rope.value = value_;
        rope.q_norm_weight = layer.query_norm;
        rope.k_norm_weight = layer.key_norm;
        rope.rope_table = rope_table_;
        rope.rotary_dim = g_.rotary_dim;
        rope.epsilon = g_.norm_epsilon;
        rope.first_cache_position = context_tokens;
        status_check(qllm_attention_paged_q4h_fused(&launch, &rope));
      } else {
        throw std::runtime_error("unknown kernel name: " + which);
      }
    };
    hipEvent_t begin{};
    hipEvent_t end{};
    hip_check(hipEventCreate(&begin), "create timing event");
    hip_check(hipEventCreate(&end), "create timing event");
    const auto timed = [&](const auto& body) {
      hip_check(hipEventRecord(begin, stream), "record timing event");
      body();
      hip_check(hipEventRecord(end, stream), "record timing event");
      hip_check(hipEventSynchronize(end), "wait for timing event");
      float milliseconds{};
      hip_check(hipEventElapsedTime(&milliseconds, begin, end), "read timing");
      return static_cast<double>(milliseconds);
    };
    if (which == "lm_head") {
      // There is one head, and it nearly fits the last-level cache: launched
      // back to back it would be timed on cached weights.  Every timed launch
      // therefore follows the gate/up launches of several layers - more than
      // twice the cache's size of other weights, as in a step - and the time of
      // those launches alone is taken off.
      const std::uint64_t filler_bytes =
          2U * qllm_fp4_packed_weight_bytes(g_.intermediate, pad32(g_.hidden), 0U);
      const std::uint32_t fillers = std::min<std::uint32_t>(
          g_.layers, static_cast<std::uint32_t>(
                         (std::uint64_t{640} << 20U) / std::max<std::uint64_t>(
                                                           filler_bytes, 1U) + 1U));
      const auto filler = [&](std::uint32_t round) {
        for (std::uint32_t index = 0; index < fillers; ++index) {
          const auto& layer = layers_[(round * fillers + index) % g_.layers];
          status_check(qllm_fp4_swiglu_bf16_balanced(
              &layer.gate.descriptor, &layer.up.descriptor, normalized_,
              hidden_bytes, activation_, rows, gemm_workspace_,
              gemm_workspace_bytes_, stream_));
        }
      };
      filler(0U);
      launch_one(0U);
      const double with_head = timed([&] {
        for (std::uint32_t round = 0; round < rounds; ++round) {
          filler(round);
          launch_one(0U);
        }
      });
      const double without = timed([&] {
        for (std::uint32_t round = 0; round < rounds; ++round) filler(round);
      });
      *launches = rounds;
      *microseconds = 1000.0 * (with_head - without) / static_cast<double>(rounds);
    } else {
      const std::uint32_t per_round = g_.layers;
      for (std::uint32_t index = 0; index < per_round; ++index) launch_one(index);
      const double milliseconds = timed([&] {
        for (std::uint32_t round = 0; round < rounds; ++round)
          for (std::uint32_t index = 0; index < per_round; ++index)
            launch_one(index);
      });
      *launches = std::uint64_t{rounds} * per_round;
      *microseconds = 1000.0 * milliseconds / static_cast<double>(*launches);
    }
    (void)hipEventDestroy(begin);
    (void)hipEventDestroy(end);
    return er::Status::success();
  } catch (const std::exception& error) {
    return {er::ErrorCode::internal, error.what()};
  }
}

er::Status Mi355DenseFp4Provider::synchronize() {
  const auto status = hipStreamSynchronize(static_cast<hipStream_t>(stream_));
  if (status != hipSuccess)
    return {er::ErrorCode::internal, hipGetErrorString(status)};
  return er::Status::success();
}

// ---- sampling ---------------------------------------------------------------

// distribution_from_logits, dense_fp4_provider.cpp:8331-8391.  top_k == 0
// selects the whole-vocabulary path of the scalar sampler (sample_token,
// :773-799): the row is copied to the host and ordered there.
er::SamplingDistribution Mi355DenseFp4Provider::distribution_from_logits(
    float* row_logits, std::uint32_t vocabulary, std::uint32_t* device_argmax,
    const er::ProgramRequestContext& request, const std::uint8_t* presence) {
  const auto stream = static_cast<hipStream_t>(stream_);
  const auto penalty = presence_penalty_of(request);
  const auto temperature = request_parameter(request, "sampling_temperature_ppm");
  if (penalty != 0.0) {
    if (!presence) throw std::runtime_error("sampling presence state is absent");
    status_check(qllm_apply_presence_penalty(row_logits, presence, vocabulary,
                                             static_cast<float>(penalty),
                                             stream_));
    // the arg-max the pass left behind was taken before the penalty
    if (temperature == 0U)
      status_check(qllm_argmax_batch(row_logits, vocabulary, 1U, device_argmax,
                                     select_workspace_, select_workspace_bytes_,
                                     stream_));
  }
  if (temperature == 0U) {
    std::uint32_t token{};
    hip_check(hipMemcpyAsync(&token, device_argmax, sizeof(token),
                             hipMemcpyDeviceToHost, stream),
              "copy exact greedy token");
    hip_check(hipStreamSynchronize(stream), "copy exact greedy token");
    return {{{token, 1.0}}};
  }
  const auto top_p = static_cast<std::uint32_t>(
      request_parameter(request, "sampling_top_p_ppm"));
  const auto min_p = static_cast<std::uint32_t>(
      request_parameter(request, "sampling_min_p_ppm"));
  const auto top_k = request_parameter(request, "sampling_top_k");
  if (top_k > kMaximumGpuSamplingTopK || top_k > vocabulary)
    throw std::runtime_error(
        "sampled exact decode requires top-k of at most 64 (0 = whole row)");
  std::vector<float> host_logits;
  std::vector<std::uint32_t> host_tokens;
  if (top_k == 0U) {
    std::vector<float> full(vocabulary);
    hip_check(hipMemcpyAsync(full.data(), row_logits, full.size() * 4U,
                             hipMemcpyDeviceToHost, stream),
              "copy logit row");
    hip_check(hipStreamSynchronize(stream), "copy logit row");
    host_tokens.resize(vocabulary);
    std::iota(host_tokens.begin(), host_tokens.end(), 0U);
    std::sort(host_tokens.begin(), host_tokens.end(),
              [&](std::uint32_t left, std::uint32_t right) {
                const float a = full[left];
                const float b = full[right];
                if (std::isnan(a)) return false;
                if (std::isnan(b)) return true;
                return a == b ? left < right : a > b;
              });
    host_logits.reserve(vocabulary);
    for (const auto token : host_tokens) host_logits.push_back(full[token]);
    sampling_logit_transfer_bytes_ += full.size() * 4U;
  } else {
    return std::move(distributions_from_top_k(row_logits, vocabulary, vocabulary,
                                              1U, request)
                         .front());
  }
  return er::make_sampling_distribution(
      host_logits, host_tokens, static_cast<std::uint32_t>(temperature), top_p,
      min_p);
}

// The distributions of `rows` rows of logits (row r at logits + r * stride)
// for a sampled request with 1 <= top_k <= 64: one selection launch for all
// rows, one readback, then make_sampling_distribution per row
// (distribution_from_logits, dense_fp4_provider.cpp:8331-8391, which selects
// and reads back row by row).
std::vector<er::SamplingDistribution>
Mi355DenseFp4Provider::distributions_from_top_k(
    const float* logits, std::uint32_t vocabulary, std::size_t stride,
    std::uint32_t rows, const er::ProgramRequestContext& request) {
  const auto stream = static_cast<hipStream_t>(stream_);
  const auto temperature = request_parameter(request, "sampling_temperature_ppm");
  const auto top_p = static_cast<std::uint32_t>(
      request_parameter(request, "sampling_top_p_ppm"));
  const auto min_p = static_cast<std::uint32_t>(
      request_parameter(request, "sampling_min_p_ppm"));
  const auto top_k =
      static_cast<std::uint32_t>(request_parameter(request, "sampling_top_k"));
  if (!rows || rows > 8U || !top_k || top_k > kMaximumGpuSamplingTopK ||
      top_k > vocabulary)
    throw std::runtime_error(
        "sampled exact decode requires top-k of at most 64 (0 = whole row)");
  status_check(qllm_topk_logits_batch(logits, vocabulary, stride, top_k, rows,
                                      top_logits_, top_tokens_, select_workspace_,
                                      select_workspace_bytes_, stream_));
  // logits of all rows, then tokens of all rows (the device buffers are
  // adjacent with room for 8 rows of 64)
  constexpr std::size_t kCapacity = 8U * kMaximumGpuSamplingTopK;
  hip_check(hipMemcpyAsync(staging_->top_logits, top_logits_,
                           kCapacity * 4U + std::size_t{rows} * top_k * 4U,
                           hipMemcpyDeviceToHost, stream),
            "copy speculative top-k");
  hip_check(hipStreamSynchronize(stream), "copy speculative top-k");
  ++sampling_gpu_calls_;
  sampling_logit_transfer_bytes_ += std::size_t{rows} * top_k * 8U;
  std::vector<er::SamplingDistribution> result;
  result.reserve(rows);
  for (std::uint32_t row = 0; row < rows; ++row) {
    const std::span<const float> row_logits(
        staging_->top_logits + std::size_t{row} * top_k, top_k);
    const std::span<const std::uint32_t> row_tokens(
        staging_->top_tokens + std::size_t{row} * top_k, top_k);
    result.push_back(er::make_sampling_distribution(
        row_logits, row_tokens, static_cast<std::uint32_t>(temperature), top_p,
        min_p));
  }
  return result;
}

// ---- the proposer (run_mtp / extend_mtp_rollout, :8681-8852) -----------------

// The kernels of one proposer pass over the tokens in mtp_tokens_, through the
// draft head's argmax when `produce_logits`.  With `deferred_positions` the
// positions come from mtp_positions_ when the kernels run and the pass ends by
// advancing them (qllm_rollout_advance), so that a captured pass can be
// replayed, and greedy passes chained, without the host in between.
void Mi355DenseFp4Provider::enqueue_mtp(std::uint32_t rows,
                                        const float* previous_hidden,
                                        bool produce_logits,
                                        std::uint32_t cache_position,
                                        bool deferred_positions,
                                        std::uint8_t* mark_emitted) {
  void* const stream = stream_;
  const auto hip_stream = static_cast<hipStream_t>(stream_);
  const std::uint32_t rotary_position = cache_position + 1U;  // row 0
  // the lookup is part of the input norms' launch where that kernel serves
  const bool fused_lookup = !g_.activation_q8 && g_.hidden <= 16384U &&
                            g_.hidden % 4U == 0U &&
                            embedding_.descriptor.layout == QLLM_LAYOUT_ROW_MAJOR;
  if (!fused_lookup) {
    status_check(qllm_fp4_embedding_batch(&embedding_.descriptor, mtp_tokens_,
                                          mtp_embedding_, rows, stream));
    if (mark_emitted)
      status_check(qllm_mark_presence(mark_emitted, mtp_tokens_, rows,
                                      g_.vocabulary, stream));
  }
  // [RMSNorm(embedding) | RMSNorm(previous target hidden)] -> fusion projection
  const std::size_t half_bytes = std::size_t{g_.hidden} * 2U;
  const bool q8 = g_.activation_q8;
  // RMSNorm of `count` rows as the input of the projection that follows: bf16
  // rows in normalized_, or Q8 rows in q8_
  const auto normalise = [&](const float* rows_in, const float* weight,
                             std::uint32_t count) {
    if (q8) {
      enqueue_normalise_q8(rows_in, weight, count);
    } else {
      status_check(qllm_rms_norm_batch(rows_in, weight, nullptr, normalized_,
                                       g_.hidden, count, g_.hidden, g_.norm_epsilon,
                                       g_.zero_centered_norm, stream));
    }
  };
  // a projection of the rows prepared above (or of bf16 rows elsewhere)
  const auto project = [&](const qllm_fp4_matrix& matrix, const std::uint16_t* bf16,
                           std::size_t bf16_bytes, float* out, const float* residual,
                           std::uint32_t count) {
    if (q8)
      status_check(qllm_fp4_gemm_q8(&matrix, q8_, q8_scales_, out, QLLM_OUT_F32,
                                    residual, count, stream));
    else
      status_check(qllm_fp4_gemm_bf16(&matrix, bf16, bf16_bytes, out, QLLM_OUT_F32,
                                      residual, count, stream));
  };
  if (q8) {
    // both norms in F32 side by side, one quantisation of the 2 * hidden row
    // (the fusion projection's input is one activation row, :8716-8735)
    const std::size_t half_f32 = std::size_t{g_.hidden} * 4U;
    status_check(qllm_rms_norm_batch(mtp_embedding_, mtp_.embedding_norm,
                                     activation_f32_, nullptr, 0U, rows, g_.hidden,
                                     g_.norm_epsilon, g_.zero_centered_norm, stream));
    hip_check(hipMemcpy2DAsync(mtp_fusion_f32_, 2U * half_f32, activation_f32_,
                               half_f32, half_f32, rows, hipMemcpyDeviceToDevice,
                               hip_stream),
              "assemble MTP normalized embedding batch");
    status_check(qllm_rms_norm_batch(previous_hidden, mtp_.hidden_norm,
                                     activation_f32_, nullptr, 0U, rows, g_.hidden,
                                     g_.norm_epsilon, g_.zero_centered_norm, stream));
    hip_check(hipMemcpy2DAsync(mtp_fusion_f32_ + g_.hidden, 2U * half_f32,
                               activation_f32_, half_f32, half_f32, rows,
                               hipMemcpyDeviceToDevice, hip_stream),
              "assemble MTP target hidden batch");
    enqueue_quantise(mtp_fusion_f32_, rows, 2U * g_.hidden);
  } else if (fused_lookup) {
    status_check(qllm_rms_norm_concat_embedding_batch(
        &embedding_.descriptor, mtp_tokens_, mtp_.embedding_norm, previous_hidden,
        mtp_.hidden_norm, mtp_fusion_input_, rows, g_.norm_epsilon,
        g_.zero_centered_norm, mark_emitted, stream));
  } else if (g_.hidden <= 16384U) {
    status_check(qllm_rms_norm_concat_batch(
        mtp_embedding_, mtp_.embedding_norm, previous_hidden, mtp_.hidden_norm,
        mtp_fusion_input_, rows, g_.hidden, g_.norm_epsilon,
        g_.zero_centered_norm, stream));
  } else {
    status_check(qllm_rms_norm_batch(mtp_embedding_, mtp_.embedding_norm, nullptr,
                                     normalized_, g_.hidden, rows, g_.hidden,
                                     g_.norm_epsilon, g_.zero_centered_norm, stream));
    hip_check(hipMemcpy2DAsync(mtp_fusion_input_, 2U * half_bytes, normalized_,
                               half_bytes, half_bytes, rows,
                               hipMemcpyDeviceToDevice, hip_stream),
              "assemble MTP normalized embedding batch");
    status_check(qllm_rms_norm_batch(previous_hidden, mtp_.hidden_norm, nullptr,
                                     normalized_, g_.hidden, rows, g_.hidden,
                                     g_.norm_epsilon, g_.zero_centered_norm, stream));
    hip_check(hipMemcpy2DAsync(mtp_fusion_input_ + g_.hidden, 2U * half_bytes,
                               normalized_, half_bytes, half_bytes, rows,
                               hipMemcpyDeviceToDevice, hip_stream),
              "assemble MTP target hidden batch");
  }
  // The projections onto the hidden width have few rows for the GPU: with bf16
  // activations their K is cut over workgroups and the norm that follows adds
  // the partial sums to the residual stream (as in the target's layers).
  // sum = residual + matrix * input, normalized_ = RMSNorm(sum) under `weight`.
  const auto project_and_normalise =
      [&](const qllm_fp4_matrix& matrix, const std::uint16_t* bf16,
          std::size_t bf16_bytes, const float* residual, float* sum,
          const float* weight) {
        if (!q8 && projection_splits_ > 1U && matrix.layout == QLLM_LAYOUT_TILED &&
            matrix.padded_columns / 64U >= projection_splits_ &&
            g_.hidden <= 16384U && g_.hidden % 4U == 0U) {
          status_check(qllm_fp4_gemm_bf16_partial(&matrix, bf16, bf16_bytes,
                                                  projection_partials_,
                                                  projection_splits_, rows, stream));
          status_check(qllm_rms_norm_partials_batch(
              residual, sum, projection_partials_, projection_splits_, weight,
              normalized_, rows, g_.hidden, g_.norm_epsilon, g_.zero_centered_norm,
              stream));
          return;
        }
        project(matrix, bf16, bf16_bytes, sum, residual, rows);
        normalise(sum, weight, rows);
      };
  // one transformer block over its own Q8 cache (run_full_attention + run_ffn)
  const auto& layer = mtp_.layer;
  const std::uint32_t query_stride = g_.head_dim * (g_.output_gated ? 2U : 1U);
  const std::size_t hidden_bytes = std::size_t{rows} * g_.hidden * 2U;
  const std::uint32_t kv_rows = g_.kv_heads * g_.head_dim;
  project_and_normalise(mtp_.fusion.descriptor, mtp_fusion_input_,
                        std::size_t{rows} * 2U * half_bytes, nullptr, mtp_hidden_,
                        layer.input_norm);
  const qllm_gemm_segment projections[3] = {
      {query_, layer.qkv.descriptor.rows - 2U * kv_rows, QLLM_OUT_F32},
      {key_, kv_rows, QLLM_OUT_F32},
      {value_, kv_rows, QLLM_OUT_F32}};
  if (q8)
    status_check(qllm_fp4_gemm_q8_split(&layer.qkv.descriptor, q8_, q8_scales_,
                                        projections, 3U, rows, gemm_workspace_,
                                        gemm_workspace_bytes_, stream));
  else
    status_check(qllm_fp4_gemm_bf16_split_balanced(
        &layer.qkv.descriptor, normalized_, hidden_bytes, projections, 3U, rows,
        gemm_workspace_, gemm_workspace_bytes_, stream));
  const auto pages = const_cast<const void* const*>(device_page_table_);
  // rotary of q and k and the rows' Q8 K/V records in one launch
  status_check(qllm_qkv_rope_store_q8_batch(
      query_, query_stride, key_, value_, layer.query_norm, layer.key_norm, pages,
      mtp_page_offset_, g_.kv_page_tokens, cache_position, rotary_position,
      deferred_positions ? mtp_positions_ : nullptr, rows, g_.query_heads,
      g_.kv_heads, g_.head_dim, g_.rotary_dim, g_.norm_epsilon, g_.rope_theta, 0,
      stream));
  if (!produce_logits) {
    // A pass that only feeds the proposer's cache ends here: the layer has no
    // successor, so nothing reads its attention or FFN output (the reference
    // computes them all the same, run_mtp :8737-8766).
    if (deferred_positions)
      status_check(qllm_rollout_advance(mtp_argmax_, mtp_tokens_,
                                        mtp_draft_tokens_, g_.draft_depth, rows,
                                        mtp_positions_, stream));
    return;
  }
  qllm_q8_attention_launch launch{};
  launch.query = query_;
  launch.device_pages = pages;
  launch.output = q8 ? static_cast<void*>(activation_f32_) : attention_;
  launch.partial_maxima = partial_maxima_;
  launch.partial_sums = partial_sums_;
  launch.partial_outputs = partial_outputs_;
  launch.page_offset_bytes = mtp_page_offset_;
  launch.first_context_tokens = cache_position + 1U;
  launch.rows = rows;
  launch.page_tokens = g_.kv_page_tokens;
  launch.query_heads = g_.query_heads;
  launch.kv_heads = g_.kv_heads;
  launch.head_dim = g_.head_dim;
  launch.split_tokens = split_tokens_;
  launch.maximum_splits = maximum_splits_;
  launch.query_stride = query_stride;
  launch.output_gated = g_.output_gated;
  launch.output_kind = g_.activation_q8 ? QLLM_OUT_F32 : QLLM_OUT_BF16;
  launch.stream = stream;
  launch.device_positions = deferred_positions ? mtp_positions_ : nullptr;
  status_check(qllm_attention_paged_q8(&launch));
  if (q8) enqueue_quantise(activation_f32_, rows, g_.query_heads * g_.head_dim);
  project_and_normalise(layer.output.descriptor, attention_,
                        std::size_t{rows} * g_.query_heads * g_.head_dim * 2U,
                        mtp_hidden_, mtp_hidden_, layer.post_attention_norm);
  if (q8) {
    status_check(qllm_fp4_swiglu_q8(&layer.gate.descriptor, &layer.up.descriptor,
                                    q8_, q8_scales_, activation_f32_, rows,
                                    gemm_workspace_, gemm_workspace_bytes_, stream));
    enqueue_quantise(activation_f32_, rows, g_.intermediate);
  } else {
    status_check(qllm_fp4_swiglu_bf16_balanced(
        &layer.gate.descriptor, &layer.up.descriptor, normalized_, hidden_bytes,
        activation_, rows, gemm_workspace_, gemm_workspace_bytes_, stream));
  }
  // a single-row pass leaves its hidden state where the next pass reads it
  const bool retain_in_place = rows == 1U;
  float* const last_sum = retain_in_place ? mtp_last_hidden_ : mtp_hidden_;
  const auto retain_last_row = [&] {
    if (!retain_in_place)
      hip_check(hipMemcpyAsync(mtp_last_hidden_,
                               mtp_hidden_ + std::size_t{rows - 1U} * g_.hidden,
                               g_.hidden * 4U, hipMemcpyDeviceToDevice, hip_stream),
                "retain final MTP hidden state");
  };
  // draft head: the last row, draft norm, the head's first draft_vocabulary rows
  if (q8) {
    project(layer.down.descriptor, activation_,
            std::size_t{rows} * g_.intermediate * 2U, last_sum, mtp_hidden_, rows);
    retain_last_row();
    normalise(mtp_last_hidden_, mtp_.draft_norm, 1U);
    project(mtp_.head_prefix, normalized_, std::size_t{g_.hidden} * 2U, mtp_logits_,
            nullptr, 1U);
    status_check(qllm_argmax_batch(mtp_logits_, g_.draft_vocabulary, 1U, mtp_argmax_,
                                   select_workspace_, select_workspace_bytes_,
                                   stream));
    if (deferred_positions)
      status_check(qllm_rollout_advance(mtp_argmax_, mtp_tokens_, mtp_draft_tokens_,
                                        g_.draft_depth, rows, mtp_positions_, stream));
    return;
  }
  // (every row goes through the norm that finishes the down projection; the
  // head reads the last)
  project_and_normalise(layer.down.descriptor, activation_,
                        std::size_t{rows} * g_.intermediate * 2U, mtp_hidden_,
                        last_sum, mtp_.draft_norm);
  retain_last_row();
  // the draft head, its arg-max and the hand-over to the next pass
  const qllm_rollout_step advance{mtp_tokens_, mtp_draft_tokens_, g_.draft_depth, rows,
                                  mtp_positions_};
  enqueue_head_projection(mtp_.head_prefix,
                          normalized_ + std::size_t{rows - 1U} * g_.hidden,
                          mtp_logits_, 1U, mtp_argmax_,
                          deferred_positions ? &advance : nullptr);
}

// Replays the proposer pass captured for (rows, source of the previous hidden
// state); the first use captures it.  `chained` passes read the proposer's own
// last hidden state, the others the target's.
// `drafts` == 0: one pass of `rows` rows (on the target's hidden state, or
// `chained` on the proposer's own).  `drafts` >= 1: a whole greedy rollout in
// one graph - the pass of `rows` rows on the target's hidden state followed by
// drafts - 1 chained single-row passes.
void Mi355DenseFp4Provider::launch_mtp_graph(std::uint32_t rows, bool chained,
                                             std::uint32_t drafts) {
  const auto stream = static_cast<hipStream_t>(stream_);
  void*& slot = mtp_graphs_.at(
      drafts ? 2U * (max_rows_ + 1U) + rows * (kMaximumDraftDepth + 1U) + drafts
             : 2U * rows + (chained ? 1U : 0U));
  if (!slot) {
    hip_check(hipStreamSynchronize(stream), "drain stream before capture");
    hipGraph_t graph{};
    hip_check(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal),
              "begin proposer capture");
    try {
      // the pass over the target's hidden rows takes the tokens the verify
      // step emitted: it also marks them present
      enqueue_mtp(rows, chained ? mtp_last_hidden_ : hidden_, true, 0U, true,
                  chained ? nullptr : presence_);
      for (std::uint32_t pass = 1; pass < drafts; ++pass)
        enqueue_mtp(1U, mtp_last_hidden_, true, 0U, true);
    } catch (...) {
      (void)hipStreamEndCapture(stream, &graph);
      if (graph) (void)hipGraphDestroy(graph);
      throw;
    }
    hip_check(hipStreamEndCapture(stream, &graph), "end proposer capture");
    hipGraphExec_t exec{};
    const auto status = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    hip_check(status, "instantiate proposer graph");
    slot = exec;
  }
  hip_check(hipGraphLaunch(static_cast<hipGraphExec_t>(slot), stream),
            "launch proposer graph");
}

std::optional<DraftPrediction> Mi355DenseFp4Provider::run_mtp(
    DenseFp4RequestState& state, std::span<const std::uint32_t> tokens,
    const float* previous_hidden, bool produce_logits,
    const er::ProgramRequestContext* request, const std::uint8_t* presence,
    std::uint32_t sample_position, std::uint32_t random_stream) {
  if (!mtp_.ready || tokens.empty() || tokens.size() > max_rows_ ||
      !previous_hidden || state.mtp_length + tokens.size() > g_.max_context)
    throw std::runtime_error("invalid MTP microbatch");
  const auto rows = static_cast<std::uint32_t>(tokens.size());
  for (const auto token : tokens)
    if (token >= g_.vocabulary)
      throw std::runtime_error("MTP token is outside the vocabulary");
  const auto hip_stream = static_cast<hipStream_t>(stream_);
  const std::uint32_t cache_position = state.mtp_length;  // row 0
  ensure_pages(cache_position + rows - 1U);
  hip_check(hipMemcpyAsync(mtp_tokens_, tokens.data(), rows * 4U,
                           hipMemcpyHostToDevice, hip_stream),
            "upload MTP token batch");
  {
    const auto events = begin_gpu_phase(GpuPhase::mtp);
    enqueue_mtp(rows, previous_hidden, produce_logits, cache_position, false);
    end_gpu_phase(events);
    collect_gpu_phases();
  }
  state.mtp_length += rows;
  ++mtp_passes_;
  mtp_rows_ += rows;
  if (!produce_logits) return std::nullopt;

  DraftPrediction result;
  if (request) {
    result.distribution = distribution_from_logits(
        mtp_logits_, g_.draft_vocabulary, mtp_argmax_, *request, presence);
    result.token = er::sample_distribution(
        result.distribution,
        er::counter_uniform(request_parameter(*request, "sampling_seed"),
                            sample_position, random_stream));
  } else {
    hip_check(hipMemcpyAsync(&result.token, mtp_argmax_, sizeof(result.token),
                             hipMemcpyDeviceToHost, hip_stream),
              "copy final MTP draft token");
    hip_check(hipStreamSynchronize(hip_stream), "copy final MTP draft token");
    result.distribution.entries.push_back({result.token, 1.0});
  }
  // logits without a finite maximum select no token
  if (result.token >= g_.draft_vocabulary)
    throw std::runtime_error("MTP draft token is outside the draft vocabulary");
  return result;
}

// run_mtp over the accepted tokens followed by extend_mtp_rollout, as captured
// graphs: the first pass pairs `tokens` with the target's hidden rows, every
// further pass feeds the proposer its own draft and hidden state.  A greedy
// request runs all passes back to back and reads the drafts once; a sampled
// one returns to the host after each pass for its distribution.  Positions,
// sampling positions and streams are those of the two functions it replaces.
void Mi355DenseFp4Provider::propose_with_graphs(
    DenseFp4RequestState& state, std::span<const std::uint32_t> tokens,
    const er::ProgramRequestContext& request, std::uint32_t context_limit) {
  if (!mtp_.ready || tokens.empty() || tokens.size() > max_rows_ ||
      context_limit > g_.max_context ||
      state.mtp_length + tokens.size() + 1U >= context_limit)
    throw std::runtime_error("invalid MTP proposal");
  for (const auto token : tokens)
    if (token >= g_.vocabulary)
      throw std::runtime_error("MTP token is outside the vocabulary");
  const auto rows = static_cast<std::uint32_t>(tokens.size());
  const auto stream = static_cast<hipStream_t>(stream_);
  const std::uint32_t first_position = state.mtp_length;
  const std::uint32_t committed_length = first_position + rows;
  // drafts: the root, then as many as depth and context allow
  // (extend_mtp_rollout's loop, :8794-8852)
  std::uint32_t drafts = 1U;
  while (drafts < g_.draft_depth &&
         committed_length + (drafts - 1U) + 2U < context_limit)
    ++drafts;
  // rollout pass i writes the proposer's cache at committed_length + i - 1
  ensure_pages(committed_length + drafts - 2U);
  const std::uint32_t positions[4] = {first_position, first_position + 1U,
                                      first_position + 1U, 0U};
  std::copy(tokens.begin(), tokens.end(), staging_->proposer);
  std::copy(positions, positions + 4, staging_->proposer + 8);
  hip_check(hipMemcpyAsync(mtp_tokens_, staging_->proposer,
                           sizeof(staging_->proposer), hipMemcpyHostToDevice,
                           stream),
            "upload MTP tokens and positions");
  state.draft_predictions.clear();
  state.draft_predictions.reserve(drafts);
  const bool greedy =
      request_parameter(request, "sampling_temperature_ppm") == 0U;
  if (greedy) {
    launch_mtp_graph(rows, false, drafts);
    std::uint32_t* const chosen = staging_->download;
    hip_check(hipMemcpyAsync(chosen, mtp_draft_tokens_, drafts * 4U,
                             hipMemcpyDeviceToHost, stream),
              "copy MTP draft tokens");
    hip_check(hipStreamSynchronize(stream), "copy MTP draft tokens");
    for (std::uint32_t depth = 0; depth < drafts; ++depth) {
      // logits without a finite maximum select no token (0xffffffff); the
      // chained pass embedded a row of zeros for it and every kernel ran
      if (chosen[depth] >= g_.draft_vocabulary)
        throw std::runtime_error(
            "MTP draft token is outside the draft vocabulary");
      DraftPrediction prediction;
      prediction.token = chosen[depth];
      prediction.distribution.entries.push_back({chosen[depth], 1.0});
      state.draft_predictions.push_back(std::move(prediction));
    }
  } else {
    const auto seed = request_parameter(request, "sampling_seed");
    for (std::uint32_t depth = 0; depth < drafts; ++depth) {
      if (depth) {
        // the device chained its own argmax; the sampled draft replaces it
        // (pinned word: the previous pass ended with a wait, and the copy is
        // ordered before the pass launched next)
        staging_->proposer[0] = state.draft_predictions.back().token;
        hip_check(hipMemcpyAsync(mtp_tokens_, staging_->proposer,
                                 sizeof(std::uint32_t), hipMemcpyHostToDevice,
                                 stream),
                  "upload sampled MTP draft");
      }
      launch_mtp_graph(depth ? 1U : rows, depth != 0U);
      DraftPrediction prediction;
      // a request with a presence penalty takes the uncaptured passes
      prediction.distribution = distribution_from_logits(
          mtp_logits_, g_.draft_vocabulary, mtp_argmax_, request, nullptr);
      prediction.token = er::sample_distribution(
          prediction.distribution,
          er::counter_uniform(seed, committed_length + (depth ? depth - 1U : 0U),
                              1U + depth));
      if (!(prediction.distribution.probability(prediction.token) > 0.0))
        throw std::runtime_error("invalid MTP rollout root");
      state.draft_predictions.push_back(std::move(prediction));
    }
  }
  mtp_passes_ += drafts;
  mtp_rows_ += rows + drafts - 1U;
  state.draft_valid = true;
  // speculative rows of the proposer's cache are overwritten by the next pass
  state.mtp_length = committed_length;
}

void Mi355DenseFp4Provider::extend_mtp_rollout(
    DenseFp4RequestState& state, const er::ProgramRequestContext& request,
    DraftPrediction first, std::uint32_t context_limit) {
  if (context_limit > g_.max_context || state.mtp_length >= context_limit ||
      !(first.distribution.probability(first.token) > 0.0))
    throw std::runtime_error("invalid MTP rollout root");
  state.draft_predictions.clear();
  state.draft_predictions.reserve(g_.draft_depth);
  const auto committed_length = state.mtp_length;
  if (committed_length + 1U >= context_limit)
    throw std::runtime_error("MTP rollout root exceeds context");
  state.draft_predictions.push_back(std::move(first));
  // every draft is present for the drafts after it (:8822-8847)
  const std::uint32_t root[1] = {state.draft_predictions.back().token};
  mark_presence(proposal_presence_, root);
  while (state.draft_predictions.size() < g_.draft_depth &&
         state.mtp_length + 2U < context_limit) {
    // the next pass reads the proposer's own last hidden state before it
    // replaces it (both on the provider's stream, in order)
    const auto sample_position = state.mtp_length;
    const std::uint32_t token[1] = {state.draft_predictions.back().token};
    auto prediction = run_mtp(
        state, token, mtp_last_hidden_, true, &request, proposal_presence_,
        sample_position,
        1U + static_cast<std::uint32_t>(state.draft_predictions.size()));
    if (!prediction) throw std::runtime_error("MTP rollout produced no proposal");
    state.draft_predictions.push_back(std::move(*prediction));
    const std::uint32_t drafted[1] = {state.draft_predictions.back().token};
    mark_presence(proposal_presence_, drafted);
  }
  state.draft_valid = !state.draft_predictions.empty();
  // speculative rows of the proposer's cache are overwritten by the next pass
  state.mtp_length = committed_length;
}

// ---- the verify step (execute_exact_decode ABI 2, :11156-11318) -------------

er::ExactDecodeExecutionHandle Mi355DenseFp4Provider::execute_exact_decode(
    const er::IPreparedOperation& operation,
    const std::shared_ptr<er::IOperationProviderRequestState>& opaque_state,
    const er::ExactDecodeInvocation& invocation) {
  try {
    std::lock_guard lock(mutex_);
    const auto state =
        std::dynamic_pointer_cast<DenseFp4RequestState>(opaque_state);
    if (&operation != exact_.get() || !state || !state->draft_valid ||
        invocation.guaranteed_token != state->synchronized_token ||
        invocation.position != state->mtp_length ||
        invocation.position + 1U >= invocation.context_limit ||
        invocation.context_limit > g_.max_context)
      throw std::runtime_error("exact MTP invocation stream is invalid");
    activate(state->slot);
    const auto proposal_count = state->draft_predictions.size();
    if (proposal_count == 0U || proposal_count > g_.draft_depth ||
        invocation.position + proposal_count >= invocation.context_limit)
      throw std::runtime_error("multi-draft MTP state is invalid");

    std::vector<std::uint32_t> target_tokens{invocation.guaranteed_token};
    for (const auto& proposal : state->draft_predictions) {
      if (!(proposal.distribution.probability(proposal.token) > 0.0))
        throw std::runtime_error("MTP proposal has zero draft mass");
      target_tokens.push_back(proposal.token);
    }
    const auto rows = static_cast<std::uint32_t>(target_tokens.size());
    auto status = use_graphs_ ? run_target_graph(target_tokens.data(), rows,
                                                 invocation.position)
                              : run_target(target_tokens.data(), rows,
                                           invocation.position);
    if (!status.ok()) throw std::runtime_error(std::string(status.message()));

    // Row r is penalised at the tokens emitted before this step and at the
    // drafts of the rows before it (:11182-11202); tokens_[1..] are the drafts.
    const auto penalty = presence_penalty_of(invocation.request);
    const bool greedy =
        request_parameter(invocation.request, "sampling_temperature_ppm") == 0U;
    if (penalty != 0.0) {
      status_check(qllm_apply_presence_penalty_rows(
          logits_, g_.vocabulary, presence_, tokens_ + 1, rows, g_.vocabulary,
          static_cast<float>(penalty), stream_));
      if (greedy)
        status_check(qllm_argmax_batch(logits_, g_.vocabulary, rows,
                                       argmax_tokens_, select_workspace_,
                                       select_workspace_bytes_, stream_));
    }
    std::vector<er::SamplingDistribution> target_distributions;
    target_distributions.reserve(rows);
    if (greedy) {
      // greedy: the rows' arg-max tokens in one copy and one wait
      const auto stream = static_cast<hipStream_t>(stream_);
      hip_check(hipMemcpyAsync(staging_->download, argmax_tokens_,
                               rows * sizeof(std::uint32_t),
                               hipMemcpyDeviceToHost, stream),
                "copy exact greedy tokens");
      hip_check(hipStreamSynchronize(stream), "copy exact greedy tokens");
      // a row without a finite logit selects nothing (0xffffffff): reported
      // here, before the proposer or the request state is touched
      for (std::uint32_t row = 0; row < rows; ++row)
        if (staging_->download[row] >= g_.vocabulary)
          throw std::runtime_error("target logits have no finite maximum");
      for (std::uint32_t row = 0; row < rows; ++row)
        target_distributions.push_back({{{staging_->download[row], 1.0}}});
    } else if (request_parameter(invocation.request, "sampling_top_k") != 0U) {
      target_distributions = distributions_from_top_k(
          logits_, g_.vocabulary, g_.vocabulary, rows, invocation.request);
    } else {
      // whole-vocabulary candidates; the penalty has been applied above
      er::ProgramRequestContext unpenalised = invocation.request;
      unpenalised.parameters["sampling_presence_penalty_biased_ppm"] = 2'000'000U;
      for (std::uint32_t row = 0; row < rows; ++row)
        target_distributions.push_back(distribution_from_logits(
            logits_ + std::size_t{row} * g_.vocabulary, g_.vocabulary,
            argmax_tokens_ + row, unpenalised, nullptr));
    }

    const auto seed = request_parameter(invocation.request, "sampling_seed");
    std::size_t accepted{};
    std::uint32_t next_token{};
    bool rejected{};
    for (; accepted < proposal_count; ++accepted) {
      const auto& proposal = state->draft_predictions[accepted];
      const auto depth = static_cast<std::uint32_t>(accepted);
      const auto decision = er::rejection_sample(
          proposal.token, target_distributions[accepted], proposal.distribution,
          er::counter_uniform(seed, invocation.position + depth, 100U, depth),
          er::counter_uniform(seed, invocation.position + depth, 200U, depth));
      if (!decision.accepted) {
        next_token = decision.token;
        rejected = true;
        break;
      }
    }
    if (!rejected)
      next_token = er::sample_distribution(
          target_distributions.back(),
          er::counter_uniform(
              seed, invocation.position + static_cast<std::uint32_t>(accepted),
              300U));

    const auto positions_advanced = static_cast<std::uint32_t>(accepted + 1U);
    const bool future_exact =
        invocation.position + positions_advanced + 1U < invocation.context_limit;
    // The captured passes select their drafts on the device without the
    // presence bytes; a request with a penalty takes the uncaptured ones.
    const bool captured_proposal =
        mtp_.ready && future_exact && use_graphs_ && penalty == 0.0;
    if (!captured_proposal) {
      // accepted drafts and the next token are emitted tokens from here on
      // (:11261-11270); the captured proposer pass marks them itself
      std::vector<std::uint32_t> emitted_now;
      for (std::size_t index = 0; index < accepted; ++index)
        emitted_now.push_back(state->draft_predictions[index].token);
      emitted_now.push_back(next_token);
      mark_presence(presence_, emitted_now);
    }
    if (mtp_.ready) {
      // advance the proposer over the accepted drafts and the next token (row r
      // pairs the token at position + r + 1 with the target's hidden state at
      // position + r), then roll the next drafts out (:11262-11288)
      std::vector<std::uint32_t> mtp_tokens;
      for (std::size_t index = 0; index < accepted; ++index)
        mtp_tokens.push_back(state->draft_predictions[index].token);
      mtp_tokens.push_back(next_token);
      state->mtp_length = invocation.position;
      state->draft_valid = false;
      state->draft_predictions.clear();
      if (captured_proposal) {
        propose_with_graphs(*state, mtp_tokens, invocation.request,
                            invocation.context_limit);
      } else {
        hip_check(hipMemcpyAsync(proposal_presence_, presence_, g_.vocabulary,
                                 hipMemcpyDeviceToDevice,
                                 static_cast<hipStream_t>(stream_)),
                  "initialize next MTP rollout presence");
        auto first = run_mtp(*state, mtp_tokens, hidden_, future_exact,
                             future_exact ? &invocation.request : nullptr,
                             future_exact ? proposal_presence_ : nullptr,
                             invocation.position + positions_advanced, 1U);
        if (future_exact) {
          if (!first)
            throw std::runtime_error("next MTP rollout produced no root");
          extend_mtp_rollout(*state, invocation.request, std::move(*first),
                             invocation.context_limit);
        }
      }
    } else {
      state->mtp_length = invocation.position + positions_advanced;
      state->draft_valid = false;
      state->draft_predictions.clear();
    }
    state->synchronized_token = next_token;

    er::ExactDecodeExecutionResult result;
    result.status = er::Status::success();
    result.emitted_tokens.push_back(invocation.guaranteed_token);
    for (std::size_t index = 0; index < accepted; ++index)
      result.emitted_tokens.push_back(target_tokens[index + 1U]);
    result.next_token = next_token;
    result.positions_advanced = positions_advanced;
    ++exact_calls_;
    accepted_drafts_ += accepted;
    ++accepted_depth_calls_.at(accepted);
    program_steps_ += positions_advanced;
    return completed_exact(std::move(result));
  } catch (const std::exception& error) {
    er::ExactDecodeExecutionResult failure;
    failure.status = {er::ErrorCode::internal, error.what()};
    return completed_exact(std::move(failure));
  }
}

// ---- synthetic model / cache ---------------------------------------------------

DeviceFp4Matrix Mi355DenseFp4Provider::synthetic_matrix(std::uint32_t rows,
                                                        std::uint32_t columns,
                                                        std::uint64_t seed,
                                                        bool tiled) {
  const std::uint32_t padded = pad32(columns);
  const bool block16 = g_.scale_scheme == QLLM_SCALE_F16_BLOCK16;
  // the row-major and the tiled layout hold the same multiset of bytes per
  // matrix; a random-init model may be generated in either directly
  const bool use_tiles = tiled && padded % 64U == 0U;
  const std::uint32_t tile_rows = use_tiles ? 32U : 0U;
  const std::size_t padded_rows =
      use_tiles ? std::size_t{(rows + tile_rows - 1U) / tile_rows} * tile_rows
                : rows;
  const std::size_t code_bytes = padded_rows * padded / 2U;
  const std::size_t scale_count = padded_rows * (padded / (block16 ? 16U : 32U));
  const std::size_t scale_bytes = scale_count * (block16 ? 2U : 1U);
  void* codes{};
  void* scales{};
  hip_check(hipMalloc(&codes, code_bytes), "allocate synthetic weights");
  hip_check(hipMalloc(&scales, scale_bytes), "allocate synthetic scales");
  allocations_.push_back(codes);
  allocations_.push_back(scales);
  status_check(qllm_fill_random(codes, code_bytes, 0U, seed, stream_));
  status_check(qllm_fill_random(scales, scale_count, block16 ? 3U : 5U,
                                seed ^ 0x5ca1eULL, stream_));
  DeviceFp4Matrix matrix;
  matrix.weights = codes;
  matrix.scales = scales;
  matrix.descriptor = {static_cast<const std::uint8_t*>(codes),
                       scales,
                       rows,
                       columns,
                       padded,
                       g_.scale_scheme,
                       use_tiles ? std::uint32_t{QLLM_LAYOUT_TILED}
                                 : std::uint32_t{QLLM_LAYOUT_ROW_MAJOR},
                       tile_rows};
  weight_bytes_ += std::uint64_t{rows} * padded / 2U +
                   std::uint64_t{rows} * (padded / (block16 ? 16U : 32U)) *
                       (block16 ? 2U : 1U);
  return matrix;
}

er::Status Mi355DenseFp4Provider::load_synthetic_weights(std::uint64_t seed) {
  try {
    std::lock_guard lock(mutex_);
    const auto ones = [this](std::uint32_t elements, float value) {
      std::vector<float> host(elements, value);
      void* pointer{};
      hip_check(hipMalloc(&pointer, elements * 4U), "allocate norm weight");
      allocations_.push_back(pointer);
      hip_check(hipMemcpy(pointer, host.data(), elements * 4U,
                          hipMemcpyHostToDevice),
                "upload norm weight");
      return static_cast<float*>(pointer);
    };
    const float unit = g_.zero_centered_norm ? 0.0F : 1.0F;
    const auto query_rows =
        g_.query_heads * g_.head_dim * (g_.output_gated ? 2U : 1U);
    std::uint64_t stream_seed = seed;
    const auto next_seed = [&stream_seed]() {
      stream_seed += 0x9e3779b97f4a7c15ULL;
      return stream_seed;
    };
    embedding_ = synthetic_matrix(g_.vocabulary, g_.hidden, next_seed(), false);
    for (auto& layer : layers_) {
      layer.input_norm = ones(g_.hidden, unit);
      layer.post_attention_norm = ones(g_.hidden, unit);
      if (g_.qk_norm) {
        layer.query_norm = ones(g_.head_dim, 0.0F);
        layer.key_norm = ones(g_.head_dim, 0.0F);
      }
      layer.qkv =
          synthetic_matrix(query_rows + 2U * g_.kv_heads * g_.head_dim,
                           g_.hidden, next_seed(), true);
      layer.output = synthetic_matrix(g_.hidden, g_.query_heads * g_.head_dim,
                                      next_seed(), true);
      layer.gate = synthetic_matrix(g_.intermediate, g_.hidden, next_seed(), true);
      layer.up = synthetic_matrix(g_.intermediate, g_.hidden, next_seed(), true);
      layer.down = synthetic_matrix(g_.hidden, g_.intermediate, next_seed(), true);
    }
    final_norm_ = ones(g_.hidden, unit);
    head_ = synthetic_matrix(g_.vocabulary, g_.hidden, next_seed(), true);
    if (g_.mtp_layers) {
      mtp_.embedding_norm = ones(g_.hidden, unit);
      mtp_.hidden_norm = ones(g_.hidden, unit);
      mtp_.draft_norm = ones(g_.hidden, unit);
      mtp_.fusion = synthetic_matrix(g_.hidden, 2U * g_.hidden, next_seed(), true);
      auto& layer = mtp_.layer;
      layer.input_norm = ones(g_.hidden, unit);
      layer.post_attention_norm = ones(g_.hidden, unit);
      if (g_.qk_norm) {
        layer.query_norm = ones(g_.head_dim, 0.0F);
        layer.key_norm = ones(g_.head_dim, 0.0F);
      }
      layer.qkv = synthetic_matrix(query_rows + 2U * g_.kv_heads * g_.head_dim,
                                   g_.hidden, next_seed(), true);
      layer.output = synthetic_matrix(g_.hidden, g_.query_heads * g_.head_dim,
                                      next_seed(), true);
      layer.gate = synthetic_matrix(g_.intermediate, g_.hidden, next_seed(), true);
      layer.up = synthetic_matrix(g_.intermediate, g_.hidden, next_seed(), true);
      layer.down = synthetic_matrix(g_.hidden, g_.intermediate, next_seed(), true);
      finish_mtp_weights();
    }
    attention_ops_ = ffn_ops_ = g_.layers;
    embedding_ready_ = head_ready_ = true;
    hip_check(hipStreamSynchronize(static_cast<hipStream_t>(stream_)),
              "generate synthetic weights");
    return er::Status::success();
  } catch (const std::exception& error) {
    return {er::ErrorCode::internal, error.what()};
  }
}

er::Status Mi355DenseFp4Provider::prefill_synthetic_kv(std::uint32_t tokens,
                                                       std::uint64_t seed) {
  try {
    std::lock_guard lock(mutex_);
    if (!tokens || tokens > g_.max_context)
      return {er::ErrorCode::invalid_argument, "prefill length is invalid"};
    ensure_pages(tokens - 1U);
    const std::uint32_t chunk = 4096U;
    const std::size_t width = std::size_t{g_.kv_heads} * g_.head_dim;
    float* keys{};
    float* values{};
    hip_check(hipMalloc(&keys, chunk * width * 4U), "allocate prefill keys");
    hip_check(hipMalloc(&values, chunk * width * 4U), "allocate prefill values");
    for (std::uint32_t layer = 0; layer < g_.layers; ++layer) {
      for (std::uint32_t first = 0; first < tokens; first += chunk) {
        const std::uint32_t count = std::min(chunk, tokens - first);
        const std::uint64_t salt =
            seed + (std::uint64_t{layer} << 32U) + first;
        status_check(qllm_fill_random(keys, count * width, 1U, salt, stream_));
        status_check(qllm_fill_random(values, count * width, 1U,
                                      salt ^ 0xabcdef12345ULL, stream_));
        if (g_.kv_encoding == KvEncoding::q4_f16_per_head)
          status_check(qllm_store_kv_paged_q4h_batch(
              keys, values, const_cast<const void* const*>(device_page_table_),
              layer, g_.kv_page_tokens, first, count, g_.kv_heads, g_.head_dim,
              stream_));
        else
          status_check(qllm_store_kv_paged_f16_batch(
              keys, values, const_cast<const void* const*>(device_page_table_),
              layer, g_.kv_page_tokens, first, count, g_.kv_heads, g_.head_dim,
              stream_));
      }
    }
    if (g_.mtp_layers) {
      for (std::uint32_t first = 0; first < tokens; first += chunk) {
        const std::uint32_t count = std::min(chunk, tokens - first);
        const std::uint64_t salt = seed + (std::uint64_t{0xffffU} << 32U) + first;
        status_check(qllm_fill_random(keys, count * width, 1U, salt, stream_));
        status_check(qllm_fill_random(values, count * width, 1U,
                                      salt ^ 0xabcdef12345ULL, stream_));
        status_check(qllm_store_kv_paged_q8_batch(
            keys, values, const_cast<const void* const*>(device_page_table_),
            mtp_page_offset_, g_.kv_page_tokens, first, count, g_.kv_heads,
            g_.head_dim, stream_));
      }
    }
    hip_check(hipStreamSynchronize(static_cast<hipStream_t>(stream_)),
              "prefill synthetic KV");
    (void)hipFree(keys);
    (void)hipFree(values);
    return er::Status::success();
  } catch (const std::exception& error) {
    return {er::ErrorCode::internal, error.what()};
  }
}

er::Status Mi355DenseFp4Provider::copy_mtp_state(float* host_last_hidden,
                                                 float* host_draft_logits) {
  std::lock_guard lock(mutex_);
  if (!mtp_.ready)
    return {er::ErrorCode::invalid_argument, "the provider has no MTP layer"};
  auto status = hipStreamSynchronize(static_cast<hipStream_t>(stream_));
  if (status == hipSuccess && host_last_hidden)
    status = hipMemcpy(host_last_hidden, mtp_last_hidden_, g_.hidden * 4U,
                       hipMemcpyDeviceToHost);
  if (status == hipSuccess && host_draft_logits)
    status = hipMemcpy(host_draft_logits, mtp_logits_, g_.draft_vocabulary * 4U,
                       hipMemcpyDeviceToHost);
  if (status != hipSuccess)
    return {er::ErrorCode::internal, hipGetErrorString(status)};
  return er::Status::success();
}

er::Status Mi355DenseFp4Provider::copy_kv_page(std::uint32_t page_index,
                                               void* host_output) {
  std::lock_guard lock(mutex_);
  const auto& pages_ = slots_[active_slot_].pages;
  if (!host_output || page_index >= pages_.size())
    return {er::ErrorCode::invalid_argument, "KV page index is invalid"};
  auto status = hipStreamSynchronize(static_cast<hipStream_t>(stream_));
  if (status == hipSuccess) {
    if (pages_[page_index])
      status = hipMemcpy(host_output, pages_[page_index], kv_page_bytes_,
                         hipMemcpyDeviceToHost);
    else
      std::memset(host_output, 0, kv_page_bytes_);
  }
  if (status != hipSuccess)
    return {er::ErrorCode::internal, hipGetErrorString(status)};
  return er::Status::success();
}

std::map<std::string, std::uint64_t, std::less<>>
Mi355DenseFp4Provider::telemetry() const {
  std::lock_guard lock(mutex_);
  std::map<std::string, std::uint64_t, std::less<>> values;
  values["provider_exact_calls"] = exact_calls_;
  values["provider_accepted_drafts"] = accepted_drafts_;
  values["provider_program_steps"] = program_steps_;
  values["provider_sampling_gpu_calls"] = sampling_gpu_calls_;
  values["provider_sampling_logit_transfer_bytes"] =
      sampling_logit_transfer_bytes_;
  for (std::size_t depth = 0; depth < accepted_depth_calls_.size(); ++depth)
    values["provider_accepted_depth_" + std::to_string(depth)] =
        accepted_depth_calls_[depth];
  values["provider_mtp_passes"] = mtp_passes_;
  values["provider_mtp_rows"] = mtp_rows_;
  values["provider_mtp_kv_page_offset"] = mtp_page_offset_;
  values["provider_weight_bytes"] = weight_bytes_;
  values["provider_kv_page_bytes"] = kv_page_bytes_;
  // dense_fp4_provider.cpp:3117-3119
  values["provider_dense_activation_input_bf16"] = g_.activation_q8 ? 0U : 1U;
  // dense_fp4_provider.cpp:3170-3200
  if (g_.profile_gpu_phases) {
    const auto phase = [this](GpuPhase which) {
      return gpu_phase_ns_[static_cast<std::size_t>(which)];
    };
    values["provider_gpu_embedding_ns"] = phase(GpuPhase::embedding);
    values["provider_gpu_full_attention_ns"] = phase(GpuPhase::full_attention);
    values["provider_gpu_ffn_ns"] = phase(GpuPhase::ffn);
    values["provider_gpu_head_ns"] = phase(GpuPhase::head);
    values["provider_gpu_mtp_ns"] = phase(GpuPhase::mtp);
    values["provider_gpu_measured_batches"] = gpu_measured_batches_;
  }
  return values;
}

er::Status Mi355DenseFp4Provider::copy_matrix_rows(std::string_view name,
                                                   std::uint32_t first_row,
                                                   std::uint32_t rows,
                                                   void* host_codes,
                                                   void* host_scales) {
  try {
    std::lock_guard lock(mutex_);
    const auto of_layer = [](const LayerWeights& layer,
                             std::string_view which) -> const DeviceFp4Matrix* {
      if (which == "qkv") return &layer.qkv;
      if (which == "output") return &layer.output;
      if (which == "gate") return &layer.gate;
      if (which == "up") return &layer.up;
      if (which == "down") return &layer.down;
      return nullptr;
    };
    const DeviceFp4Matrix* matrix = nullptr;
    if (name == "token_embedding") {
      matrix = &embedding_;
    } else if (name == "output_head") {
      matrix = &head_;
    } else if (name == "mtp.fusion") {
      matrix = &mtp_.fusion;
    } else if (name.starts_with("mtp.layer.")) {
      matrix = of_layer(mtp_.layer, name.substr(10));
    } else if (name.starts_with("layer.")) {
      const auto rest = name.substr(6);
      const auto dot = rest.find('.');
      if (dot != std::string_view::npos) {
        const auto index = std::stoul(std::string(rest.substr(0, dot)));
        if (index < layers_.size())
          matrix = of_layer(layers_[index], rest.substr(dot + 1U));
      }
    }
    if (!matrix || !matrix->weights || !host_codes || !host_scales || !rows ||
        first_row >= matrix->descriptor.rows ||
        rows > matrix->descriptor.rows - first_row)
      return {er::ErrorCode::invalid_argument,
              "matrix name or row range is invalid: " + std::string(name)};
    const auto& d = matrix->descriptor;
    const std::size_t code_bytes = std::size_t{rows} * d.padded_columns / 2U;
    const std::size_t scale_bytes =
        d.scale_scheme == QLLM_SCALE_F16_BLOCK16
            ? std::size_t{rows} * (d.padded_columns / 16U) * 2U
            : std::size_t{rows} * (d.padded_columns / 32U);
    DeviceBuffer codes(code_bytes, "allocate row read-back");
    DeviceBuffer scales(scale_bytes, "allocate row read-back");
    status_check(qllm_fp4_unpack_rows(&d, first_row, rows, codes.get(),
                                      scales.get(), stream_));
    const auto stream = static_cast<hipStream_t>(stream_);
    hip_check(hipMemcpyAsync(host_codes, codes.get(), code_bytes,
                             hipMemcpyDeviceToHost, stream),
              "copy matrix rows");
    hip_check(hipMemcpyAsync(host_scales, scales.get(), scale_bytes,
                             hipMemcpyDeviceToHost, stream),
              "copy matrix row scales");
    hip_check(hipStreamSynchronize(stream), "copy matrix rows");
    return er::Status::success();
  } catch (const std::exception& error) {
    return {er::ErrorCode::internal, error.what()};
  }
}

// The contract the runner validates and publishes (values of
// dense_fp4_provider.cpp:11447-11486 for a dense resident model).
er::ExecutionProviderModule::ServiceContract
Mi355DenseFp4Provider::service_contract() const {
  er::ExecutionProviderModule::ServiceContract contract;
  contract.prefill_mode = "causal_layer_major";
  contract.prefill_chunk_tokens = max_rows_;   // rows one execute() batch holds
  contract.session_retention = false;
  contract.request_stream_mode = "per_request_nonblocking";
  contract.rope_mode = "artifact";
  contract.kv_dtype = g_.kv_encoding == KvEncoding::fp16 ? "fp16"
                                                          : "q4-f16-per-head";
  contract.kv_allocation = "paged_on_demand";
  contract.kv_page_tokens = g_.kv_page_tokens;
  contract.kv_page_bytes = kv_page_bytes_;
  contract.kv_page_capacity = slots_.size() * slots_.front().pages.size();
  contract.placement_mode = "resident";
  contract.placement_profile = "resident";
  contract.ram_cache_bytes = 0U;
  contract.vram_cache_bytes = std::max<std::uint64_t>(weight_bytes_, 1U);
  contract.placement_prefetch_enabled = false;
  contract.placement_prefetch_state = "disabled";
  contract.placement_minimum_observations = 0U;
  contract.mtp_resource_available = static_cast<bool>(exact_);
  contract.mtp_runtime_ready = static_cast<bool>(exact_);
  contract.mtp_enabled = static_cast<bool>(exact_);
  contract.retain_previous_route = false;
  contract.cpu_hybrid_enabled = false;
  contract.sampling_supported = true;
  return contract;
}

}  // namespace qllm
