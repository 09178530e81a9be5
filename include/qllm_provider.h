/*
 * C ABI over the MI355X dense-FP4 provider (quantum-llm_amd/provider), for
 * hosts that cannot link the C++ IOperationProvider object directly: test
 * drivers, benchmarks, foreign-language workers.  Each call forwards to the
 * provider method named beside it; the provider itself mirrors the reference's
 * runtime/tools/dense_fp4_provider.cpp.
 *
 * Status codes are those of qllm_kernels.h; qllm_provider_last_error() holds
 * the text of the last failure on the calling thread.  Host pointers are
 * plain process memory; nothing here takes or returns device pointers except
 * qllm_provider_logits / qllm_provider_hidden.
 */
#ifndef QLLM_PROVIDER_H
#define QLLM_PROVIDER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct qllm_provider qllm_provider;

/* Geometry an artifact declares for a dense decoder
 * (validate_dense_fp4_descriptor, dense_fp4_provider.cpp:804-994). */
typedef struct qllm_dense_geometry {
  uint32_t hidden;
  uint32_t intermediate;
  uint32_t layers;
  uint32_t query_heads;
  uint32_t kv_heads;
  uint32_t head_dim;
  uint32_t rotary_dim;
  uint32_t vocabulary;
  float rope_theta;
  float norm_epsilon;
  int32_t output_gated;
  int32_t qk_norm;
  int32_t zero_centered_norm;
  uint32_t scale_scheme;   /* enum qllm_scale_scheme */
  uint32_t kv_encoding;    /* 0 = "q4-f16-per-head", 1 = "fp16" */
  uint32_t kv_page_tokens;
  uint32_t max_context;
  uint32_t draft_depth;
  /* The proposer (run_mtp, dense_fp4_provider.cpp:8681-8852): 1 = the provider
   * runs one MTP layer with its own Q8 KV cache and produces the drafts itself
   * (its tensors are staged before qllm_provider_prepare_exact_decode, roles
   * as in validate_exact :4730-4787: embedding_norm, hidden_norm, draft_norm,
   * fusion_projection, layer.0.*), 0 = drafts arrive through
   * qllm_provider_set_drafts. */
  uint32_t mtp_layers;
  /* Head rows the proposer scores (project_prefix :6280-6308); 0 =
   * min(vocabulary, 65536). */
  uint32_t draft_vocabulary;
  /* Rows of a prompt that go through the tall linears at a time
   * (qllm_provider_prefill); 0 = 32768.  The reference's prompt path runs
   * prefill_chunk_tokens rows per program step (moe_vm_runner.cpp:682-745). */
  uint32_t prefill_chunk_rows;
  /* 1 = per-row Q8 activations into every projection, the reference's default
   * contract (an artifact without dense_activation_input_bf16,
   * prepare_dense_activation dense_fp4_provider.cpp:5983-6003); 0 = bf16
   * activations.  Q8 needs scale_scheme 0 (block-32 UE8M0) and projection
   * widths that are multiples of 64. */
  uint32_t activation_q8;
} qllm_dense_geometry;

const char* qllm_provider_last_error(void);

/* The provider for a geometry given by the host; tensors follow through
 * qllm_provider_stage_tensor / qllm_provider_prepare. */
qllm_provider* qllm_provider_create(const qllm_dense_geometry* geometry);
/* make_<name>_callable_provider(artifact_root, max_context, ..., kv_page_tokens,
 * kv_cache_dtype, ..., mtp_draft_depth) (dense_fp4_provider.cpp:11402-11470)
 * followed by the executor's start-up binding (program_executor.cpp:1725-1826):
 * loads and authenticates the Expert Pack v1 directory, takes the geometry
 * from its model program, uploads every tensor the program's operations name
 * and prepares them, the exact-decode program included.  max_context 0 = the
 * artifact's; kv_page_tokens 0 = 256; kv_cache_dtype NULL or "artifact" =
 * "q4-f16-per-head", or "fp16"; mtp_draft_depth 0 = the artifact's.  NULL on
 * failure, with the reason in qllm_provider_last_error(). */
qllm_provider* qllm_provider_create_from_artifact(const char* artifact_root,
                                                  uint32_t max_context,
                                                  uint32_t kv_page_tokens,
                                                  const char* kv_cache_dtype,
                                                  uint32_t mtp_draft_depth);
void qllm_provider_destroy(qllm_provider* provider);

/* Capability table of make_<name>_provider(): writes up to `capacity`
 * NUL-separated "capability\0" strings, returns the count. */
uint32_t qllm_provider_capabilities(char* buffer, size_t capacity);

/* Stages one host tensor for the next qllm_provider_prepare call.
 * encoding "FP4_E2M1": data = packed codes, scales = scale bytes,
 * quant_abi 3 (UE8M0 / 32) or 16 (binary16 / 16); encoding "F32": data only.
 * The bytes are copied. */
int32_t qllm_provider_stage_tensor(qllm_provider* provider, const char* role,
                                   const char* encoding, uint32_t quant_abi,
                                   uint32_t rows, uint32_t columns,
                                   const void* data, size_t data_bytes,
                                   const void* scales, size_t scale_bytes);

/* IOperationProvider::prepare for one artifact operation with the staged
 * tensors (then clears the staging area). */
int32_t qllm_provider_prepare(qllm_provider* provider, const char* capability);

/* IOperationProvider::prepare_exact_decode (ABI 2). */
int32_t qllm_provider_prepare_exact_decode(qllm_provider* provider,
                                           const char* capability);

/* Random-init model / KV cache generated on the device. */
int32_t qllm_provider_load_synthetic_weights(qllm_provider* provider,
                                             uint64_t seed);
int32_t qllm_provider_prefill_synthetic_kv(qllm_provider* provider,
                                           uint32_t tokens, uint64_t seed);

/* create_request_state + request parameters
 * (moe_vm_runner.cpp:318-347): sampling_temperature_ppm, sampling_top_p_ppm,
 * sampling_top_k, sampling_min_p_ppm, sampling_seed. */
int32_t qllm_provider_begin_request(qllm_provider* provider,
                                    uint32_t temperature_ppm,
                                    uint32_t top_p_ppm, uint32_t top_k,
                                    uint32_t min_p_ppm, uint64_t seed);

/* The same with the request's parameter map spelled out, name by name, as the
 * runner builds it (moe_vm_runner.cpp:318-347): reserved_context_tokens,
 * sampling_temperature_ppm, sampling_top_p_ppm, sampling_top_k,
 * sampling_min_p_ppm, sampling_presence_penalty_biased_ppm (penalty in ppm +
 * 2,000,000), sampling_first_output_position, sampling_seed,
 * exact_decode_enabled.  A sampled request (temperature != 0) without a first
 * output position or with a penalty parameter above 4,000,000 is turned down
 * (dense_fp4_provider.cpp:5502-5513). */
int32_t qllm_provider_begin_request_with(qllm_provider* provider,
                                         const char* const* names,
                                         const uint64_t* values,
                                         uint32_t count);

/* synchronize_exact_decode_batch with one token: the stream stands at
 * `position` with `token` guaranteed (the batch starts at position - 1, the
 * target position the token was chosen from).  With an MTP layer this feeds
 * the proposer that pair - using the hidden state of row 0 of the last target
 * pass - and rolls the drafts for the next verify out; position 0 only marks
 * the start of a stream. */
int32_t qllm_provider_synchronize(qllm_provider* provider, uint32_t token,
                                  uint32_t position);

/* Prompt prefill: `count` tokens at positions first_position .. through the
 * target (linears on the tall-batch GEMM, K/V written to the paged cache),
 * `*predicted` = the greedy token for the position after the prompt, whose
 * logits are row 0 of qllm_provider_copy_logits.  After
 * qllm_provider_begin_request the proposer is fed the prompt too and the
 * first drafts are rolled out, so that qllm_provider_verify can follow with
 * (*predicted, first_position + count).  This is the worker's feed
 * (runtime/tools/moe_vm_runner.cpp:682-745: program-sequence prefill, then
 * synchronize_exact_decode_batch over the prompt in chunks). */
int32_t qllm_provider_prefill(qllm_provider* provider, const uint32_t* tokens,
                              uint32_t count, uint32_t first_position,
                              uint32_t* predicted);

/* Rows [first_row, first_row + rows) of one of the provider's FP4 matrices as
 * row-major codes [rows, padded_columns/2] and scales in host memory, whatever
 * layout the device copy has (tools and tests; a random-init model exists on
 * the device only).  name: "token_embedding", "output_head",
 * "layer.<n>.qkv|output|gate|up|down" (qkv: query, key and value rows in that
 * order), "mtp.fusion", "mtp.layer.qkv|output|gate|up|down". */
int32_t qllm_provider_copy_matrix_rows(qllm_provider* provider, const char* name,
                                       uint32_t first_row, uint32_t rows,
                                       void* host_codes, void* host_scales);

/* One batch through the prepared program, operation by operation, the way
 * the common VM drives a provider (IOperationProvider::execute,
 * runtime/include/expert/runtime/program_executor.hpp:251-254; the reference's
 * execute, runtime/tools/dense_fp4_provider.cpp:10680-10992): `rows` tokens at
 * consecutive `positions` (host arrays), `*next_token` = the head's selection
 * for the last row under the request's sampling parameters.  With exact decode
 * enabled in the request the batch then awaits qllm_provider_synchronize_batch. */
int32_t qllm_provider_execute_program(qllm_provider* provider,
                                      const uint32_t* tokens,
                                      const uint32_t* positions, uint32_t rows,
                                      uint32_t* next_token);

/* synchronize_exact_decode_batch (program_executor.hpp:340-362): next_tokens[r]
 * is the token after target position first_target_position + r; the proposer
 * is fed (token, target hidden state) pairs from the batch the program last
 * executed, and with produce_final_draft the drafts are rolled out. */
int32_t qllm_provider_synchronize_batch(qllm_provider* provider,
                                        const uint32_t* next_tokens,
                                        uint32_t count,
                                        uint32_t first_target_position,
                                        int32_t produce_final_draft);

/* Drafts for the next verify step.  distribution_counts[i] entries of
 * (tokens, probabilities) describe draft i's proposal distribution q; a count
 * of 0 means the one-hot distribution on the draft token (greedy). */
int32_t qllm_provider_set_drafts(qllm_provider* provider,
                                 const uint32_t* draft_tokens,
                                 uint32_t draft_count,
                                 const uint32_t* distribution_counts,
                                 const uint32_t* distribution_tokens,
                                 const double* distribution_probabilities);

/* execute_exact_decode: emitted[0] is the guaranteed token, then the
 * accepted drafts; returns counts through the out parameters. */
int32_t qllm_provider_verify(qllm_provider* provider, uint32_t guaranteed_token,
                             uint32_t position, uint32_t context_limit,
                             uint32_t* emitted, uint32_t* emitted_count,
                             uint32_t* next_token,
                             uint32_t* positions_advanced);

/* run_target alone (no sampling), and its graph-captured replay. */
int32_t qllm_provider_run_target(qllm_provider* provider,
                                 const uint32_t* tokens, uint32_t rows,
                                 uint32_t first_position);
int32_t qllm_provider_capture_target(qllm_provider* provider,
                                     const uint32_t* tokens, uint32_t rows,
                                     uint32_t first_position);
int32_t qllm_provider_replay_target(qllm_provider* provider);
int32_t qllm_provider_synchronize_stream(qllm_provider* provider);

/* Synchronise the provider's stream and copy logits [rows, vocabulary] /
 * hidden state [rows, hidden] of the last target pass to host memory. */
int32_t qllm_provider_copy_logits(qllm_provider* provider, uint32_t rows,
                                  float* host_output);
int32_t qllm_provider_copy_hidden(qllm_provider* provider, uint32_t rows,
                                  float* host_output);

/* Average launch duration (microseconds) of one hot kernel, measured with HIP
 * events on the provider's stream over rounds x layers launches on distinct
 * per-layer data.  which: "ffn_gate_up", "ffn_down", "attention", "lm_head". */
int32_t qllm_provider_time_kernel(qllm_provider* provider, const char* which,
                                  uint32_t rounds, uint32_t context_tokens,
                                  double* microseconds, uint64_t* launches);

/* Bytes of one KV page (all layers) and a host copy of page `page_index`
 * (zero-filled if the page has not been allocated yet). */
uint64_t qllm_provider_kv_page_bytes(const qllm_provider* provider);
int32_t qllm_provider_copy_kv_page(qllm_provider* provider, uint32_t page_index,
                                   void* host_output);

/* The proposer's state after its last pass: hidden state of the last row
 * [hidden] and draft logits [draft_vocabulary] (either may be NULL), and the
 * draft tokens waiting for the next verify step (returns their number). */
int32_t qllm_provider_copy_mtp_state(qllm_provider* provider,
                                     float* host_last_hidden,
                                     float* host_draft_logits);
uint32_t qllm_provider_drafts(const qllm_provider* provider, uint32_t* tokens,
                              uint32_t capacity);
uint32_t qllm_provider_draft_vocabulary(const qllm_provider* provider);

const float* qllm_provider_logits(const qllm_provider* provider);
const float* qllm_provider_hidden(const qllm_provider* provider);
void* qllm_provider_stream(const qllm_provider* provider);
uint64_t qllm_provider_weight_bytes(const qllm_provider* provider);
/* telemetry(): value of one counter, 0 if unknown. */
uint64_t qllm_provider_telemetry(const qllm_provider* provider,
                                 const char* name);

/* ---- host sampling mathematics of the verify step -------------------------
 * The four functions of runtime/include/expert/runtime/speculative_sampling.hpp
 * (make_sampling_distribution :23-27, sample_distribution :29-30,
 * rejection_sample :42-45, counter_uniform :49-52) as the provider links them.
 * They run on the host and need no device.  Distributions cross the boundary
 * as parallel arrays (token ids, double probabilities).  A std::invalid_argument
 * of the reference becomes QLLM_INVALID_ARGUMENT, a std::runtime_error
 * QLLM_INTERNAL; the text is left in qllm_provider_last_error(). */

/* Candidates sorted by descending logit (ties: ascending id).  Writes the
 * retained entries to tokens_out / probabilities_out (capacity >= count) and
 * their number to count_out. */
int32_t qllm_sampling_make_distribution(const float* sorted_logits,
                                        const uint32_t* sorted_tokens,
                                        uint32_t count,
                                        uint32_t temperature_ppm,
                                        uint32_t top_p_ppm, uint32_t min_p_ppm,
                                        uint32_t* tokens_out,
                                        double* probabilities_out,
                                        uint32_t* count_out);
/* Inverse-CDF draw in entry order with uniform in [0, 1). */
int32_t qllm_sampling_sample(const uint32_t* tokens,
                             const double* probabilities, uint32_t count,
                             double uniform, uint32_t* token_out);
/* Leviathan rejection step: accept `proposal` with min(1, p/q), else draw from
 * the normalised residual max(p - q, 0). */
int32_t qllm_sampling_rejection(uint32_t proposal,
                                const uint32_t* target_tokens,
                                const double* target_probabilities,
                                uint32_t target_count,
                                const uint32_t* draft_tokens,
                                const double* draft_probabilities,
                                uint32_t draft_count,
                                double acceptance_uniform,
                                double correction_uniform, int32_t* accepted_out,
                                uint32_t* token_out,
                                double* target_probability_out,
                                double* draft_probability_out);
/* Counter-based uniform in [0, 1): splitmix64 over (seed, position, stream,
 * index), top 53 bits. */
double qllm_sampling_counter_uniform(uint64_t seed, uint32_t position,
                                     uint32_t stream, uint32_t index);

/* ---- artifact reader ----------------------------------------------------------
 * Host only; none of these calls touches a device.  On failure the status is
 * the reference's ErrorCode and the message is in qllm_provider_last_error(). */

/* sha256() of runtime/include/expert/runtime/sha256.hpp:26. */
int32_t qllm_sha256(const void* data, size_t bytes, uint8_t* digest32);
/* The same digest computed without the CPU's SHA instructions, which
 * qllm_sha256 uses where the host has them. */
int32_t qllm_sha256_portable(const void* data, size_t bytes, uint8_t* digest32);

/* ModelArtifact::load (+ configure_mtp_draft_depth when mtp_draft_depth != 0)
 * and, with map_tensors, MappedModelTensorStore::create
 * (runtime/include/expert/runtime/model_artifact.hpp:46-92,
 * model_tensor_store.hpp:15-34). */
typedef struct qllm_artifact qllm_artifact;
int32_t qllm_artifact_open(const char* root, uint32_t mtp_draft_depth,
                           int32_t map_tensors, qllm_artifact** artifact);
void qllm_artifact_close(qllm_artifact* artifact);
/* IModelTensorStore::resolve (program_executor.hpp:57-62): the mapped record
 * of a dense tensor; with check_header the record's 256-byte header is
 * checked against the index entry first (compiler/expert_pack/validate.py:
 * 148-325). */
int32_t qllm_artifact_tensor(qllm_artifact* artifact, const char* name,
                             int32_t check_header, const void** record,
                             uint64_t* record_bytes);

#ifdef __cplusplus
}
#endif
#endif
