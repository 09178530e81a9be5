/*
 * CPU oracle for the speculative MTP-4 verify path.  TEST INFRASTRUCTURE ONLY.
 *
 * This library restates, in plain C, the arithmetic of the reference's verify
 * step (FP4 block-scaled linears, Q4H / exact-F16 decode attention, lm_head
 * token selection and draft acceptance).  It exists so that tests, the smoke
 * check and the benchmark's cpu_baseline leg have something independent of the
 * HIP kernels to compare against.  Nothing in the shipped library links it.
 *
 * Every function names the reference file:line whose arithmetic it follows
 * (paths are relative to the reference tree).  Functions whose results are
 * not fixed by a reference fixture say "parity unpinned" and name the
 * mathematical checks that pin them instead.
 */
#ifndef QLLM_ORACLE_H
#define QLLM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar number formats ------------------------------------------- */

/* Round-to-nearest-even F32 -> BF16 -> F32; Inf/NaN pass through.
 * runtime/src/cpu/fp4_host_executor.cpp:134-139,
 * runtime/tools/dense_fp4_cuda_smoke.cpp:104-113. */
float qo_bf16_round(float value);
uint16_t qo_bf16_bits(float value);
float qo_bf16_value(uint16_t bits);

/* IEEE binary16 round-to-nearest-even conversion (software statement of
 * __float2half_rn / __half2float used at
 * runtime/src/cuda/transformer_kernels.cu:258-263). */
uint16_t qo_f16_bits(float value);
float qo_f16_value(uint16_t bits);

/* OCP E2M1: {0,.5,1,1.5,2,3,4,6} with bit 3 as sign.
 * compiler/expert_pack/fp4_reference.py:12-29,
 * runtime/src/cuda/transformer_kernels.cu:193-201 (value times two). */
float qo_fp4_value(uint8_t code);
int qo_fp4_twice(uint8_t code);

/* UE8M0 power-of-two scale, bias 127; code 0 decodes to 2^-127.
 * runtime/src/cuda/transformer_kernels.cu:203-206,
 * runtime/src/cpu/fp4_host_executor.cpp:37-41. */
float qo_ue8m0_value(uint8_t code);

/* ---- FP4 weight matrices ---------------------------------------------- */

enum qo_scale_scheme {
  QO_SCALE_UE8M0_BLOCK32 = 0, /* reference quant ABI 3 */
  QO_SCALE_F16_BLOCK16 = 1    /* one binary16 scale per 16 K-elements */
};

/* Dequantise one weight row into doubles.  Low nibble holds the even column
 * (compiler/expert_pack/fp4_reference.py:70-78). */
void qo_fp4_decode_row(const uint8_t* codes, const void* scales, int scheme,
                       uint32_t padded_columns, double* out);

/* Closed-form linear: out[m*rows+n] = sum_k act[m][k] * w[n][k], with the
 * products and the sum carried in double and rounded once to F32 (then to
 * BF16 if bf16_output).  act is F32 [batch, padded_columns]; callers round
 * it to BF16 first when the path under test consumes BF16 activations.
 * Follows the bf16 expectation of
 * runtime/tools/dense_fp4_cuda_smoke.cpp:199-215 (block-32) and extends it
 * to block-16 scales; the block-16 form has no reference fixture: parity
 * unpinned by the reference, pinned by reduction to block-32 when adjacent
 * scales are equal powers of two and by brute force on tiny shapes. */
void qo_fp4_linear_f64(const uint8_t* codes, const void* scales, int scheme,
                       uint32_t rows, uint32_t padded_columns,
                       const float* act, uint32_t batch, float* out,
                       int bf16_output);

/* Reference integer path: exact int32 dot of (FP4 value * 2) with Q8
 * activations inside each 32-block, F32 scale-accumulate across blocks in
 * block order, then * activation_scale * 0.5.
 * runtime/src/cpu/fp4_host_executor.cpp:86-132 (scalar branch),
 * runtime/src/cuda/transformer_kernels.cu:1162-1275. */
void qo_fp4_linear_block32_q8(const uint8_t* codes, const uint8_t* scales,
                              uint32_t rows, uint32_t padded_columns,
                              const int8_t* q8, const float* act_scales,
                              uint32_t batch, float* out, int bf16_output);

/* Per-row symmetric Q8: scale = absmax/127 (1.0 when the row is zero),
 * q = clamp(nearbyint(x/scale), -127, 127), columns..padded_columns zeroed.
 * runtime/src/cuda/transformer_kernels.cu:912-946,
 * runtime/src/cpu/fp4_host_executor.cpp:141-152. */
void qo_quantize_q8_rows(const float* in, uint32_t rows, uint32_t columns,
                         uint32_t padded_columns, int bf16_input,
                         int8_t* out, float* scales);

/* Gather + dequantise embedding rows to F32.
 * runtime/src/cuda/transformer_kernels.cu:801-821. */
void qo_fp4_embedding(const uint8_t* codes, const void* scales, int scheme,
                      uint32_t columns, uint32_t padded_columns,
                      const uint32_t* tokens, uint32_t batch, float* out);

/* ---- normalisation and elementwise ------------------------------------ */

/* y = x * rsqrt(mean(x^2)+eps) * (zero_centered ? 1+w : w); w may be NULL
 * (weightless).  Mean in double.
 * runtime/src/cuda/transformer_kernels.cu:2469-2521. */
void qo_rms_norm_rows(const float* in, const float* weight, float* out,
                      uint32_t rows, uint32_t elements, float epsilon,
                      int zero_centered, int bf16_output);

/* out = act(act(silu(gate)) * up), act = bf16 round when bf16_activations.
 * runtime/src/cuda/transformer_kernels.cu:2774-2783. */
void qo_silu_product(const float* gate, const float* up, float* out,
                     uint32_t elements, int bf16_activations);

/* destination += source (optionally bf16-rounded).
 * runtime/src/cuda/transformer_kernels.cu:2522-2528. */
void qo_add_in_place(float* destination, const float* source,
                     uint32_t elements, int bf16_output);

/* ---- attention preparation -------------------------------------------- */

/* In place on one head vector x[head_dim]: optional RMSNorm with (1+w)
 * (weight == NULL skips the norm), then NeoX half-rotation rotary on the
 * first rotary_dim dimensions:
 *   angle = pos * theta^(-2*(i mod half)/rotary_dim)
 *   out   = x*cos + rot*sin,  rot = -x[i+half] (i<half) else x[i-half].
 * runtime/src/cuda/transformer_kernels.cu:3550-3643. */
void qo_head_norm_rope(float* x, const float* weight, uint32_t head_dim,
                       uint32_t rotary_dim, uint32_t position, float epsilon,
                       float theta, int bf16_activations);

/* Q4H ("q4-f16-per-head") geometry.  Inside a page, for one layer:
 *   K codes [kv][page_tokens][d/2] | K scales f16 [kv][page_tokens] |
 *   V codes [kv][page_tokens][d/2] | V scales f16 [kv][page_tokens].
 * runtime/src/cuda/transformer_kernels.cu:241-288,
 * runtime/tools/dense_fp4_cuda_smoke.cpp:1577-1595. */
size_t qo_q4h_layer_bytes(uint32_t page_tokens, uint32_t kv_heads,
                          uint32_t head_dim);

/* Encode one (token, kv_head) K and V vector into its page:
 *   scale = f16(max(absmax/7, 2^-24)), code = clamp(rn(x/scale),-7,7) & 15,
 * even element in the low nibble.
 * runtime/src/cuda/transformer_kernels.cu:251-288,
 * runtime/tools/dense_fp4_cuda_smoke.cpp:1522-1526,1685-1759. */
void qo_q4h_store(uint8_t* page, uint32_t layer, uint32_t page_tokens,
                  uint32_t cache_position, uint32_t kv_head,
                  uint32_t kv_heads, uint32_t head_dim, const float* key,
                  const float* value);

/* Decode one record back to F32 (code * scale). */
void qo_q4h_load(const uint8_t* page, uint32_t layer, uint32_t page_tokens,
                 uint32_t cache_position, uint32_t kv_head,
                 uint32_t kv_heads, uint32_t head_dim, float* key,
                 float* value);

/* Per (row, q head): scale = max(absmax/127, 2^-24), q = clamp(rn(x/s)).
 * query_stride is the distance between consecutive heads in `queries`
 * (2*head_dim for the gated layout).
 * runtime/src/cuda/transformer_kernels.cu:4391-4416,
 * runtime/tools/dense_fp4_cuda_smoke.cpp:1764-1786. */
void qo_quantize_queries_q8(const float* queries, uint32_t rows,
                            uint32_t query_heads, uint32_t head_dim,
                            uint32_t query_stride, int8_t* q8,
                            float* scales);

/* ---- attention ---------------------------------------------------------- */

struct qo_attention_shape {
  uint32_t rows;                 /* query positions (1 + drafts) */
  uint32_t query_heads;
  uint32_t kv_heads;
  uint32_t head_dim;
  uint32_t first_context_tokens; /* row r attends tokens [0, first+r) */
  uint32_t page_tokens;
  uint32_t layer;
  int output_gated;              /* queries laid out [q(d), gate(d)] per head,
                                    output multiplied by sigmoid(gate) */
};

/* Textbook softmax(q.k/sqrt(d)) v over the dequantised Q4H cache, all in
 * double.  queries: F32 [rows, query_heads, (gated?2:1)*head_dim].
 * The float statement in the reference is the staged oracle at
 * runtime/tools/dense_fp4_cuda_smoke.cpp:1980-1985,2064-2089 (bf16 Q/K/V,
 * F32 probabilities); causal rule :1951. */
void qo_attention_q4h_f64(const struct qo_attention_shape* shape,
                          const float* queries,
                          const uint8_t* const* page_table, float* out);

/* The reference's production arithmetic: Q8 queries, integer q.k, F32
 * softmax, probabilities * V-scale requantised to int8 over the whole
 * visible context, integer P.V.
 * runtime/tools/dense_fp4_cuda_smoke.cpp:1950-2063. */
void qo_attention_q4h_int8(const struct qo_attention_shape* shape,
                           const float* queries,
                           const uint8_t* const* page_table, float* out);

/* Q8 KV records (the proposer's cache): per layer, page_tokens*kv_heads key
 * records, then as many value records; record (token % page_tokens)*kv_heads
 * + kv_head holds head_dim int8 codes followed by one binary16 scale:
 *   scale = f16(max(absmax/127, 2^-24)), code = clamp(rn(x/scale), -127, 127).
 * `layer_offset` is the byte offset of the layer inside the page.
 * runtime/src/cuda/transformer_kernels.cu:601-625 (encoder), :5093-5101
 * (record addressing), record size :70-76; independent encoder of the
 * fixture runtime/tools/dense_fp4_cuda_smoke.cpp:1061-1088. */
size_t qo_q8_layer_bytes(uint32_t page_tokens, uint32_t kv_heads,
                         uint32_t head_dim);
void qo_q8_store(uint8_t* page, size_t layer_offset, uint32_t page_tokens,
                 uint32_t position, uint32_t kv_head, uint32_t kv_heads,
                 uint32_t head_dim, const float* key, const float* value);
void qo_q8_load(const uint8_t* page, size_t layer_offset, uint32_t page_tokens,
                uint32_t position, uint32_t kv_head, uint32_t kv_heads,
                uint32_t head_dim, float* key, float* value);

/* Textbook softmax(q.k/sqrt(d)) v over the dequantised Q8 cache, all in
 * double (shape->layer is ignored, the layer sits at layer_offset).  The
 * reference's float statement of the same attention rounds q, k, v and the
 * probabilities to bf16 (runtime/tools/dense_fp4_cuda_smoke.cpp:986-1024,
 * :1138-1167) and accepts 2e-3 between the two (:4921-4926). */
void qo_attention_q8_f64(const struct qo_attention_shape* shape,
                         size_t layer_offset, const float* queries,
                         const uint8_t* const* page_table, float* out);

/* Exact-F16 KV pages: per layer  K [page_tokens][kv][d] then
 * V [page_tokens][kv][d], binary16.
 * runtime/src/cuda/transformer_kernels.cu:6594-6606.
 * f16_probabilities != 0 reproduces the reference's rounding of the query
 * and of each probability to binary16 (:6517-6548, :6630-6642), evaluated
 * over one split; 0 gives the textbook double result on the stored values. */
void qo_attention_f16_f64(const struct qo_attention_shape* shape,
                          const float* queries,
                          const uint8_t* const* page_table,
                          int f16_probabilities, float* out);

/* Split-K merge of flash-decode partials:
 *   M = max m_i; S = sum s_i e^(m_i-M); o = sum o_i e^(m_i-M) / S.
 * partial index = (row*maximum_splits + split)*query_heads + head;
 * active splits of row r = ceil((first_context+r)/split_tokens).
 * gate may be NULL (no output gate).
 * runtime/src/cuda/transformer_kernels.cu:5741-5798. */
void qo_attention_combine(const float* partial_maxima,
                          const float* partial_sums,
                          const float* partial_outputs, const float* gate,
                          uint32_t gate_stride, uint32_t rows,
                          uint32_t query_heads, uint32_t head_dim,
                          uint32_t first_context_tokens,
                          uint32_t split_tokens, uint32_t maximum_splits,
                          float* out);

/* ---- token selection ---------------------------------------------------- */

/* argmax with ties to the lower index; NaN never selected (all-NaN rows
 * return 0xffffffff).  runtime/src/cuda/transformer_kernels.cu:7059-7092. */
uint32_t qo_argmax(const float* values, uint32_t count);

/* Exact descending top-k, ties to the lower id, NaN excluded.
 * runtime/src/cuda/transformer_kernels.cu:7096-7178,
 * comparator runtime/tools/dense_fp4_provider.cpp:781-787.
 * Returns the number of entries written (< k when fewer non-NaN exist). */
uint32_t qo_topk(const float* values, uint32_t count, uint32_t k,
                 float* out_values, uint32_t* out_indices);

/* logits[i] -= penalty where emitted[i] != 0.
 * runtime/src/cuda/transformer_kernels.cu:7180-7186. */
void qo_presence_penalty(float* logits, const uint8_t* emitted,
                         uint32_t count, float penalty);

/* ---- sampling (double precision, fixed summation order) --------------- */

struct qo_token_probability {
  uint32_t token;
  double probability;
};

enum qo_status {
  QO_OK = 0,
  QO_INVALID_ARGUMENT = 1, /* std::invalid_argument in the reference */
  QO_RUNTIME_ERROR = 2     /* std::runtime_error in the reference */
};

/* runtime/src/speculative_sampling.cpp:52-111.  Input is sorted descending
 * (ties: lower id first).  entries must hold `count` slots; *out_count
 * receives the nucleus size. */
int qo_make_sampling_distribution(const float* sorted_logits,
                                  const uint32_t* sorted_tokens,
                                  uint32_t count, uint32_t temperature_ppm,
                                  uint32_t top_p_ppm, uint32_t min_p_ppm,
                                  struct qo_token_probability* entries,
                                  uint32_t* out_count);

/* runtime/src/speculative_sampling.cpp:113-123. */
int qo_sample_distribution(const struct qo_token_probability* entries,
                           uint32_t count, double uniform,
                           uint32_t* out_token);

struct qo_rejection_result {
  int accepted;
  uint32_t token;
  double target_probability;
  double draft_probability;
};

/* runtime/src/speculative_sampling.cpp:125-171.  The residual is walked in
 * ascending token id, as the reference's std::map does. */
int qo_rejection_sample(uint32_t proposal,
                        const struct qo_token_probability* target,
                        uint32_t target_count,
                        const struct qo_token_probability* draft,
                        uint32_t draft_count, double acceptance_uniform,
                        double correction_uniform,
                        struct qo_rejection_result* result);

/* runtime/src/speculative_sampling.cpp:13-18,173-182. */
double qo_counter_uniform(uint64_t seed, uint32_t position, uint32_t stream,
                          uint32_t index);

/* ---- acceptance --------------------------------------------------------- */

struct qo_verify_result {
  uint32_t accepted;       /* number of drafts accepted */
  uint32_t next_token;     /* residual / bonus token */
  int status;              /* enum qo_status */
};

/* Greedy accept-longest-prefix: draft r accepted iff it equals
 * argmax(logits row r); on reject next = that argmax; all accepted ->
 * next = argmax(last row).  This is the one-hot special case of
 * runtime/tools/dense_fp4_provider.cpp:11204-11234. */
struct qo_verify_result qo_accept_greedy(const float* logits,
                                         uint32_t vocabulary,
                                         const uint32_t* drafts,
                                         uint32_t draft_count);

/* Stochastic acceptance loop, runtime/tools/dense_fp4_provider.cpp:
 * 11204-11234.  target[r] / target_counts[r] for r in [0, draft_count];
 * draft[r] for r in [0, draft_count).  Uniform streams 100 (accept),
 * 200 (correction, index = depth) and 300 (bonus). */
struct qo_verify_result qo_accept_stochastic(
    const struct qo_token_probability* const* target,
    const uint32_t* target_counts,
    const struct qo_token_probability* const* draft,
    const uint32_t* draft_counts, const uint32_t* drafts,
    uint32_t draft_count, uint64_t seed, uint32_t position);

/* ---- deterministic synthetic inputs ----------------------------------- */

/* splitmix64 of (seed, index): the stream both the CPU oracle and the GPU
 * fill kernels draw from, so no tensors need to be shipped. */
uint64_t qo_mix64(uint64_t seed, uint64_t index);
/* Uniform in (0,1) and standard normal (Box-Muller on two draws). */
double qo_uniform01(uint64_t seed, uint64_t index);
float qo_normal(uint64_t seed, uint64_t index);

int qo_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
