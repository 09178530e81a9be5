// MI355X provider for the dense FP4 decoder's speculative verify step.
//
// Plays the role of the reference's "sm86-dense-fp4" provider
// (runtime/tools/dense_fp4_provider.cpp): it implements IOperationProvider,
// advertises the same capability strings, owns the device copies of the
// weights, the paged KV cache and the step workspaces, and runs
// execute_exact_decode (:11139-11318) - target pass over 1+drafts rows, target
// distributions, accept-longest-prefix, residual/bonus token - by enqueueing
// the gfx950 kernels of include/qllm_kernels.h on one HIP stream.
#pragma once

#include <atomic>
#include <cstdint>
#include <map>
#include <memory>
#include <mutex>
#include <optional>
#include <span>
#include <string>
#include <vector>

#include "qllm_kernels.h"
#include "expert/runtime/program_executor.hpp"
#include "expert/runtime/worker_provider.hpp"
#include "expert/runtime/speculative_sampling.hpp"

namespace qllm {

namespace er = expert::runtime;

enum class KvEncoding : std::uint32_t { q4_f16_per_head = 0, fp16 = 1 };

// Geometry the artifact declares for the dense decoder
// (validate_dense_fp4_descriptor, dense_fp4_provider.cpp:804-994).
struct DenseGeometry final {
  std::uint32_t hidden{};
  std::uint32_t intermediate{};
  std::uint32_t layers{};
  std::uint32_t query_heads{};
  std::uint32_t kv_heads{};
  std::uint32_t head_dim{};
  std::uint32_t rotary_dim{};
  std::uint32_t vocabulary{};
  float rope_theta{1.0e6F};
  float norm_epsilon{1.0e-6F};
  bool output_gated{};        // q projection emits [query, gate] per head
  bool qk_norm{};             // per-head RMSNorm(1+w) on q and k
  bool zero_centered_norm{};  // block norms use (1 + w)
  std::uint32_t scale_scheme{QLLM_SCALE_F16_BLOCK16};
  KvEncoding kv_encoding{KvEncoding::q4_f16_per_head};
  std::uint32_t kv_page_tokens{256};
  std::uint32_t max_context{};
  std::uint32_t draft_depth{4};
  // The proposer (one MTP layer with its own Q8 KV cache): 0 = drafts come
  // from outside through set_draft_predictions(), 1 = this provider runs it.
  std::uint32_t mtp_layers{0};
  // Rows of the output head the proposer scores (project_prefix); 0 stands
  // for min(vocabulary, 65536).  A multiple of 32.
  std::uint32_t draft_vocabulary{0};
  // Prompt rows per pass of the tall linears; 0 stands for 32768 (measured on
  // a 27B-class model over a 32768-token prompt: 3.42 s in one pass, 3.64 s in
  // passes of 4096 rows, whose o and down projections load the CUs unevenly;
  // the workspace of a pass is about 200 KB per row).
  std::uint32_t prefill_chunk_rows{0};
  // The artifact's activation contract (prepare_dense_activation,
  // dense_fp4_provider.cpp:5983-6003): true = every projection takes per-row
  // Q8 activations and runs the reference's integer statement (the default of
  // an artifact that does not declare dense_activation_input_bf16), false =
  // bf16 activations.  Q8 needs block-32 UE8M0 weights and K % 64 == 0.
  bool activation_q8{};
  // Requests that may be open at once (request slots,
  // dense_fp4_provider.cpp:5514-5518, 6554-6588): each owns its KV pages, its
  // presence bytes and its proposer state.
  std::uint32_t capacity{1};
  // Opt-in hipEvent pairs around every operation kind, accumulated into the
  // provider_gpu_*_ns telemetry (dense_fp4_provider.cpp:5661-5738).  Passes run
  // one launch at a time then: a captured graph has no place for the events.
  bool profile_gpu_phases{};
};

// Defined with the artifact factory: the descriptor check behind every
// capability (validate_dense_fp4_descriptor, dense_fp4_provider.cpp:804-994).
[[nodiscard]] er::Status validate_dense_fp4_descriptor(
    const er::ModelDescriptor& model);

struct DraftPrediction final {
  std::uint32_t token{};
  er::SamplingDistribution distribution;
};

class DenseFp4RequestState final : public er::IOperationProviderRequestState {
 public:
  ~DenseFp4RequestState() override {
    if (lease) lease->store(false, std::memory_order_release);
  }
  // The request slot this state holds until it is destroyed: its index and
  // the slot's in-use flag (shared with the provider, which may be gone first).
  std::uint32_t slot{};
  std::shared_ptr<std::atomic<bool>> lease;
  std::uint32_t synchronized_token{};
  std::uint32_t mtp_length{};   // position of the guaranteed token
  bool draft_valid{};
  std::vector<DraftPrediction> draft_predictions;
  // the batch execute() is walking through the program
  // (RequestState, dense_fp4_provider.cpp:2195-2260)
  std::uint32_t current_batch_rows{};
  std::uint32_t current_batch_first{};
  std::uint32_t current_position{};
  bool exact_decode_enabled{};
  // target rows of the last head whose successors the proposer has not been
  // told yet: positions synchronization_first .. + synchronization_rows
  std::uint32_t synchronization_first{};
  std::uint32_t synchronization_rows{};
  std::uint32_t synchronization_consumed{};
};

struct DeviceFp4Matrix final {
  qllm_fp4_matrix descriptor{};
  void* weights{};
  void* scales{};
};

struct LayerWeights final {
  float* input_norm{};
  float* post_attention_norm{};
  float* query_norm{};
  float* key_norm{};
  // query, key and value rows concatenated: one streaming matrix, one launch
  DeviceFp4Matrix qkv;
  DeviceFp4Matrix output, gate, up, down;
};

// Tensors of the exact-decode operation (validate_exact,
// dense_fp4_provider.cpp:4730-4787): two input norms, the fusion projection
// [hidden, 2*hidden], one transformer block, the draft norm.  Token embedding
// and output head are the target's.
struct MtpWeights final {
  bool ready{};
  float* embedding_norm{};
  float* hidden_norm{};
  float* draft_norm{};
  DeviceFp4Matrix fusion;
  LayerWeights layer;
  qllm_fp4_matrix head_prefix{};   // the first draft_vocabulary rows of the head
};

class Mi355DenseFp4Provider final : public er::IOperationProvider {
 public:
  explicit Mi355DenseFp4Provider(const DenseGeometry& geometry);
  ~Mi355DenseFp4Provider() override;
  Mi355DenseFp4Provider(const Mi355DenseFp4Provider&) = delete;
  Mi355DenseFp4Provider& operator=(const Mi355DenseFp4Provider&) = delete;

  // IOperationProvider
  [[nodiscard]] er::PrepareOperationResult prepare(
      const er::OperationPreparationContext& context) override;
  [[nodiscard]] er::CreateOperationRequestStateResult create_request_state(
      const er::ProgramRequestContext& request) override;
  // One operation of the program on the batch the embedding started
  // (dense_fp4_provider.cpp:10680-10992): token ids and positions arrive as
  // host values, the hidden state travels between operations as a device
  // value, the head returns token ids as a host value.
  [[nodiscard]] er::OperationExecutionHandle execute(
      const er::IPreparedOperation& operation,
      const std::shared_ptr<er::IOperationProviderRequestState>& request_state,
      const er::OperationInvocation& invocation) override;
  [[nodiscard]] er::Status rebind_request_state(
      const std::shared_ptr<er::IOperationProviderRequestState>& state,
      const er::ProgramRequestContext& request) override;
  [[nodiscard]] er::PrepareOperationResult prepare_exact_decode(
      const er::ExactDecodePreparationContext& context) override;
  [[nodiscard]] er::Status synchronize_exact_decode(
      const er::IPreparedOperation& operation,
      const std::shared_ptr<er::IOperationProviderRequestState>& state,
      const er::ExactDecodeSynchronization& synchronization) override;
  [[nodiscard]] er::Status synchronize_exact_decode_batch(
      const er::IPreparedOperation& operation,
      const std::shared_ptr<er::IOperationProviderRequestState>& state,
      const er::ExactDecodeSynchronizationBatch& synchronization) override;
  [[nodiscard]] er::ExactDecodeExecutionHandle execute_exact_decode(
      const er::IPreparedOperation& operation,
      const std::shared_ptr<er::IOperationProviderRequestState>& state,
      const er::ExactDecodeInvocation& invocation) override;

  // A stream that starts at position 0 with `token` guaranteed: there is no
  // earlier target position to synchronise from, so no draft is produced.
  [[nodiscard]] er::Status begin_stream(
      const std::shared_ptr<er::IOperationProviderRequestState>& state,
      std::uint32_t token);
  // Without an MTP layer (geometry.mtp_layers == 0) whoever owns the proposer
  // hands the drafts for the next verify step over here.
  [[nodiscard]] er::Status set_draft_predictions(
      const std::shared_ptr<er::IOperationProviderRequestState>& state,
      std::vector<DraftPrediction> drafts);

  // Random-init weights generated on the device (benchmarks, large tests).
  [[nodiscard]] er::Status load_synthetic_weights(std::uint64_t seed);
  // Fill the KV cache of positions [0, tokens) with encoded N(0,1) rows.
  [[nodiscard]] er::Status prefill_synthetic_kv(std::uint32_t tokens,
                                                std::uint64_t seed);

  // One target pass over `tokens` at consecutive `first_position`.. rows,
  // leaving logits [rows, vocabulary] in logits() (run_target, :8529-8635).
  [[nodiscard]] er::Status run_target(const std::uint32_t* tokens,
                                      std::uint32_t rows,
                                      std::uint32_t first_position);
  // The same pass launched as one HIP graph (captured once per row count;
  // tokens and positions live in device memory, so the graph is replayed
  // unchanged as the stream advances).  execute_exact_decode uses this form.
  [[nodiscard]] er::Status run_target_graph(const std::uint32_t* tokens,
                                            std::uint32_t rows,
                                            std::uint32_t first_position);
  // capture = run_target_graph; replay relaunches the last graph on the same
  // tokens and positions (benchmark loops).
  [[nodiscard]] er::Status capture_target_graph(const std::uint32_t* tokens,
                                                std::uint32_t rows,
                                                std::uint32_t first_position);
  [[nodiscard]] er::Status replay_target_graph();
  [[nodiscard]] er::Status synchronize();
  // Average duration, in microseconds, of one launch of a hot kernel measured
  // with HIP events on the provider's stream: the kernel is launched once per
  // layer (distinct weights / KV each time) for `rounds` passes over the
  // layers; the head, of which there is one, is timed on weights that other
  // launches have pushed out of the last-level cache.  which: "ffn_gate_up", "ffn_down", "qkv", "attention_output",
  // "attention", "lm_head".
  [[nodiscard]] er::Status time_kernel(const std::string& which,
                                       std::uint32_t rounds,
                                       std::uint32_t context_tokens,
                                       double* microseconds,
                                       std::uint64_t* launches);

  [[nodiscard]] er::Status copy_mtp_state(float* host_last_hidden,
                                          float* host_draft_logits);
  [[nodiscard]] const float* logits() const noexcept { return logits_; }
  [[nodiscard]] const float* hidden() const noexcept { return hidden_; }
  [[nodiscard]] void* stream() const noexcept { return stream_; }
  [[nodiscard]] const DenseGeometry& geometry() const noexcept { return g_; }
  // The tall prompt path takes bf16 activations; with Q8 activations a prompt
  // goes through the program in row batches.
  [[nodiscard]] bool supports_tall_prefill() const noexcept {
    return !g_.activation_q8;
  }
  [[nodiscard]] bool profiles_gpu_phases() const noexcept {
    return g_.profile_gpu_phases;
  }
  [[nodiscard]] std::map<std::string, std::uint64_t, std::less<>> telemetry()
      const;
  [[nodiscard]] er::ExecutionProviderModule::ServiceContract service_contract()
      const;

  // Prompt prefill: runs `tokens` (positions first_position ..) through the
  // target in chunks of up to prefill_chunk_rows() rows - the linears on the
  // tall-batch GEMM, attention and the K/V store in row batches of the verify
  // step's size - and returns the head's token for the position after the
  // prompt: selected under the request's sampling profile when the request
  // carries one, the arg-max otherwise.  With a request state (and unless the
  // request says exact_decode_enabled = 0) the proposer is fed the prompt as the
  // worker's feed does through synchronize_exact_decode_batch
  // (runtime/tools/moe_vm_runner.cpp:682-745), and the first drafts are rolled
  // out: the state is then ready for execute_exact_decode at
  // first_position + tokens.size() with the prediction as guaranteed token.
  struct PrefillResult final {
    er::Status status;
    std::uint32_t predicted{};
  };
  [[nodiscard]] PrefillResult prefill(
      const std::shared_ptr<er::IOperationProviderRequestState>& state,
      std::span<const std::uint32_t> tokens, std::uint32_t first_position,
      const er::ProgramRequestContext& request);
  [[nodiscard]] std::uint32_t prefill_chunk_rows() const noexcept {
    return g_.prefill_chunk_rows ? g_.prefill_chunk_rows : 32768U;
  }
  [[nodiscard]] std::uint64_t weight_bytes() const noexcept {
    return weight_bytes_;
  }
  [[nodiscard]] std::uint64_t kv_bytes_per_token_layer() const noexcept;
  [[nodiscard]] std::uint64_t kv_page_bytes() const noexcept {
    return kv_page_bytes_;
  }
  [[nodiscard]] er::Status copy_kv_page(std::uint32_t page_index,
                                        void* host_output);
  // Rows [first_row, first_row + rows) of a weight matrix as row-major codes
  // and scales in host memory, whatever layout the device copy has.  Names:
  // "token_embedding", "output_head", "layer.<n>.qkv|output|gate|up|down",
  // "mtp.fusion", "mtp.layer.qkv|output|gate|up|down".
  [[nodiscard]] er::Status copy_matrix_rows(std::string_view name,
                                            std::uint32_t first_row,
                                            std::uint32_t rows, void* host_codes,
                                            void* host_scales);

 private:
  struct PreparedOperation;
  void allocate_workspaces();
  // the blocks of a target pass on rows [0, rows) of hidden_; with
  // `leave_partials` a residual projection may end as K-split partials that
  // the next norm adds (pending_partials_), otherwise hidden_ is complete
  // when the block returns
  void enqueue_normalise(const float* weight, std::uint32_t rows);
  void enqueue_residual_projection(const qllm_fp4_matrix& matrix,
                                   const std::uint16_t* input,
                                   std::size_t input_bytes, std::uint32_t rows,
                                   bool leave_partials);
  [[nodiscard]] std::uint32_t prefill_splits_for(
      std::uint32_t rows, std::uint32_t attention_batch) const noexcept;
  [[nodiscard]] std::uint32_t prompt_attention_splits(
      std::uint32_t rows, std::uint32_t attention_batch) const noexcept;
  void enqueue_rope_table(std::uint32_t rows, std::uint32_t first_position,
                          bool deferred_positions);
  void enqueue_attention_block(std::uint32_t index, std::uint32_t rows,
                               std::uint32_t first_position,
                               bool deferred_positions, bool leave_partials);
  void enqueue_ffn_block(std::uint32_t index, std::uint32_t rows,
                         bool leave_partials);
  void enqueue_head(std::uint32_t first_row, std::uint32_t rows);
  void enqueue_head_projection(const qllm_fp4_matrix& head,
                               const std::uint16_t* input, float* logits,
                               std::uint32_t rows, std::uint32_t* tokens,
                               const qllm_rollout_step* advance);
  // run_head with a request (dense_fp4_provider.cpp:8433-8517): presence
  // penalty, arg-max or sampling of the single head row in logits_, the
  // emitted token marked
  std::uint32_t select_head_token(const er::ProgramRequestContext& request,
                                  std::uint32_t sample_position);
  [[nodiscard]] er::ExecutionValue device_hidden_value(std::uint32_t rows) const;
  [[nodiscard]] std::uint32_t require_hidden_value(
      const er::ExecutionValue& value) const;
  std::uint32_t pending_partials_{};
  std::shared_ptr<const void> device_lifetime_;
  std::vector<std::shared_ptr<const PreparedOperation>> prepared_attention_;
  std::vector<std::shared_ptr<const PreparedOperation>> prepared_ffn_;
  // What a request keeps on the device between calls.  Kernels and captured
  // graphs address one working set (device_page_table_, presence_,
  // mtp_last_hidden_); when a call arrives for another slot the working set
  // is saved into the outgoing slot and loaded from the incoming one - a page
  // table upload and two small device copies on the provider's stream.
  struct RequestSlot final {
    std::shared_ptr<std::atomic<bool>> leased;
    std::vector<void*> pages;        // this slot's page pointers (host view)
    std::uint8_t* saved_presence{};  // [vocabulary], capacity > 1 only
    float* saved_last_hidden{};      // [hidden], proposer, capacity > 1 only
  };
  void activate(std::uint32_t slot);
  void ensure_pages(std::uint32_t last_position);
  // GPU phase timing (begin_gpu_phase / end_gpu_phase / collect_gpu_phases,
  // dense_fp4_provider.cpp:5691-5738)
  enum class GpuPhase : std::uint32_t { embedding, full_attention, ffn, head, mtp, count };
  struct GpuPhaseEvents final {
    void* start{};
    void* stop{};
    GpuPhase phase{};
  };
  [[nodiscard]] std::size_t begin_gpu_phase(GpuPhase phase);
  void end_gpu_phase(std::size_t index);
  void collect_gpu_phases();
  std::vector<GpuPhaseEvents> gpu_event_pool_;
  std::size_t active_gpu_events_{};
  std::uint64_t gpu_phase_ns_[static_cast<std::size_t>(GpuPhase::count)]{};
  std::uint64_t gpu_measured_batches_{};
  DeviceFp4Matrix upload_matrix(const er::ImmutableModelTensor& tensor,
                                bool tiled);
  // One tiled matrix holding the rows of the given row-major matrices in
  // order (same columns and scale scheme); the parts are released.
  DeviceFp4Matrix concatenate_rows(std::vector<DeviceFp4Matrix> parts);
  float* upload_f32(const er::ImmutableModelTensor& tensor,
                    std::uint32_t elements);
  DeviceFp4Matrix synthetic_matrix(std::uint32_t rows, std::uint32_t columns,
                                   std::uint64_t seed, bool tiled);
  void enqueue_target(const std::uint32_t* device_tokens, std::uint32_t rows,
                      std::uint32_t first_position, bool deferred_positions);
  std::vector<er::SamplingDistribution> distributions_from_top_k(
      const float* logits, std::uint32_t vocabulary, std::size_t stride,
      std::uint32_t rows, const er::ProgramRequestContext& request);
  er::SamplingDistribution distribution_from_logits(
      float* row_logits, std::uint32_t vocabulary, std::uint32_t* device_argmax,
      const er::ProgramRequestContext& request, const std::uint8_t* presence);
  // emitted[token] = 1 for every token (one upload, one launch)
  void mark_presence(std::uint8_t* emitted,
                     std::span<const std::uint32_t> tokens);
  // One proposer pass over `tokens` (run_mtp, dense_fp4_provider.cpp:8681-
  // 8792): row r embeds tokens[r], takes previous_hidden row r (device, F32),
  // is cached at position mtp_length + r and rotated at mtp_length + r + 1.
  // With produce_logits the last row's draft (token + distribution) comes back.
  std::optional<DraftPrediction> run_mtp(
      DenseFp4RequestState& state, std::span<const std::uint32_t> tokens,
      const float* previous_hidden, bool produce_logits,
      const er::ProgramRequestContext* request, const std::uint8_t* presence,
      std::uint32_t sample_position, std::uint32_t random_stream);
  void enqueue_attention(std::uint32_t index, std::uint32_t rows,
                         std::uint32_t first_position, bool deferred_positions,
                         float* query, float* key, float* value,
                         std::uint16_t* attention_out,
                         const float* qkv_partials = nullptr,
                         std::uint32_t qkv_partial_count = 0U);
  // buffers for `rows` prompt rows at a time (allocated on first use)
  void ensure_prefill_workspace(std::uint32_t rows);
  void enqueue_mtp(std::uint32_t rows, const float* previous_hidden,
                   bool produce_logits, std::uint32_t cache_position,
                   bool deferred_positions, std::uint8_t* mark_emitted = nullptr);
  void enqueue_mtp_prefill(std::span<const std::uint32_t> tokens,
                           std::uint32_t position);
  void launch_mtp_graph(std::uint32_t rows, bool chained,
                        std::uint32_t drafts = 0U);
  // run_mtp + extend_mtp_rollout replayed from captured graphs
  void propose_with_graphs(DenseFp4RequestState& state,
                           std::span<const std::uint32_t> tokens,
                           const er::ProgramRequestContext& request,
                           std::uint32_t context_limit);
  // extend_mtp_rollout, dense_fp4_provider.cpp:8794-8852
  void extend_mtp_rollout(DenseFp4RequestState& state,
                          const er::ProgramRequestContext& request,
                          DraftPrediction first, std::uint32_t context_limit);
  void prepare_mtp(std::span<const er::PreparedTensorBinding> tensors);
  void finish_mtp_weights();
  void release();

  DenseGeometry g_;
  mutable std::mutex mutex_;
  void* stream_{};
  std::vector<void*> allocations_;
  std::uint64_t weight_bytes_{};

  DeviceFp4Matrix embedding_{};
  DeviceFp4Matrix head_{};
  float* final_norm_{};
  std::vector<LayerWeights> layers_;
  std::uint32_t attention_ops_{};
  std::uint32_t ffn_ops_{};
  bool embedding_ready_{};
  bool head_ready_{};
  std::shared_ptr<const er::IPreparedOperation> exact_;
  MtpWeights mtp_;

  // KV cache
  std::vector<RequestSlot> slots_;
  std::uint32_t active_slot_{};
  void** device_page_table_{};
  std::uint64_t kv_page_bytes_{};
  std::uint64_t mtp_page_offset_{};   // the proposer's Q8 layer inside a page
  std::uint32_t split_tokens_{};
  std::uint32_t maximum_splits_{};

  // workspaces (device)
  std::uint32_t max_rows_{};
  std::uint32_t* tokens_{};
  float* hidden_{};
  std::uint16_t* normalized_{};
  float* query_{};
  float* key_{};
  float* value_{};
  std::uint16_t* attention_{};
  std::uint16_t* activation_{};
  float* logits_{};
  float* partial_maxima_{};
  float* partial_sums_{};
  float* partial_outputs_{};
  std::int8_t* query_operands_{};       // Q4H attention operands of a batch
  float* query_operand_scales_{};
  float* rope_table_{};                 // [max_rows, rotary_dim / 2] (cos, sin)
  // Pinned host words for the small per-pass transfers: 8 tokens + 4
  // position words up (target pass, proposer pass), 8 chosen tokens down.
  struct HostStaging {
    std::uint32_t target[12];
    std::uint32_t proposer[12];
    std::uint32_t download[8];
    float top_logits[8 * 64];            // top-k readback: logits of all rows,
    std::uint32_t top_tokens[8 * 64];    // then their tokens
    std::uint32_t marks[8];              // tokens whose presence byte is set
  };
  HostStaging* staging_ = nullptr;
  float* projection_partials_ = nullptr;   // [splits][rows][hidden]
  std::uint32_t projection_splits_ = 3U;   // 0 / 1: residual in the epilogue
  // The q/k/v projection cut along K the same way (QLLM_PROVIDER_QKV_SPLITS);
  // the rope + store kernel adds the partials.  0 / 1: one workgroup per
  // tile, the default - its 320 tiles already cover the GPU, and 2..8 cuts
  // measured 11.4-14.5 us against 11.7 us uncut.
  float* qkv_partials_ = nullptr;          // [splits][rows][q + k + v rows]
  std::uint32_t qkv_splits_ = 0U;
  // Q8 activation contract: the quantised rows of the projection about to
  // run, their scales, and the F32 values they were quantised from
  std::int8_t* q8_{};
  float* q8_scales_{};
  float* activation_f32_{};
  float* mtp_fusion_f32_{};   // [rows, 2 * hidden] both input norms of the proposer
  void enqueue_quantise(const float* input, std::uint32_t rows,
                        std::uint32_t columns);
  void enqueue_normalise_q8(const float* input, const float* weight,
                            std::uint32_t rows);
  void* gemm_workspace_{};
  std::size_t gemm_workspace_bytes_{};
  void* select_workspace_{};
  std::size_t select_workspace_bytes_{};
  std::uint32_t* argmax_tokens_{};
  // Presence bytes of the request's emitted tokens and the scratch copy that
  // also carries the drafts of the rollout in progress (sampling_presence_,
  // sampling_proposal_presence_, dense_fp4_provider.cpp:4242-4243); one
  // request at a time, as the KV cache is.
  std::uint8_t* presence_{};
  std::uint8_t* proposal_presence_{};
  std::uint32_t* mark_tokens_{};
  float* top_logits_{};
  std::uint32_t* top_tokens_{};

  // proposer workspaces
  std::uint32_t* mtp_tokens_{};
  float* mtp_embedding_{};
  std::uint16_t* mtp_fusion_input_{};   // bf16 [rows, 2*hidden]
  float* mtp_hidden_{};
  float* mtp_last_hidden_{};
  float* mtp_logits_{};
  std::uint32_t* mtp_argmax_{};
  // prompt prefill workspace
  std::uint32_t prefill_rows_{};
  std::vector<void*> prefill_allocations_;
  std::uint32_t* prefill_tokens_{};
  float* prefill_hidden_{};
  std::uint16_t* prefill_normalized_{};   // bf16 [rows, hidden]
  float* prefill_query_{};
  float* prefill_key_{};
  float* prefill_value_{};
  std::uint16_t* prefill_attention_{};    // bf16 [rows, query_heads * head_dim]
  float* prefill_embedding_{};
  std::uint16_t* prefill_activation_{};   // bf16 [rows, intermediate]
  // split partials of the batched prompt attention: [rows, splits, heads(, d)]
  std::uint32_t prefill_splits_{};
  float* prefill_partial_maxima_{};
  float* prefill_partial_sums_{};
  float* prefill_partial_outputs_{};
  std::uint64_t prefill_tokens_total_{};
  std::uint32_t* mtp_positions_{};      // cache, rotary, context, draft slot
  std::uint32_t* mtp_draft_tokens_{};
  std::vector<void*> mtp_graphs_;       // hipGraphExec_t: passes, then rollouts

  std::uint32_t* positions_{};   // device: cache, rotary, first-context
  std::vector<void*> graphs_;    // hipGraphExec_t per row count
  std::uint32_t last_graph_rows_{};
  bool use_graphs_{true};

  // telemetry (dense_fp4_provider.cpp:3109-3257)
  std::uint64_t exact_calls_{};
  std::uint64_t accepted_drafts_{};
  std::vector<std::uint64_t> accepted_depth_calls_;
  std::uint64_t program_steps_{};
  std::uint64_t sampling_gpu_calls_{};
  std::uint64_t sampling_logit_transfer_bytes_{};
  std::uint64_t mtp_passes_{};
  std::uint64_t mtp_rows_{};
};

// Metadata factory, the analogue of make_sm86_dense_fp4_provider()
// (dense_fp4_provider.cpp:11398-11400).
[[nodiscard]] er::WorkerProviderDefinition make_mi355_dense_fp4_provider();

}  // namespace qllm
