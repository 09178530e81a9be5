/*
 * C ABI of the MI355X (gfx950) kernel library for the speculative MTP-4
 * verify step.  This is the layer a provider binds where the reference's
 * provider calls the free functions of namespace expert::runtime::cuda
 * (runtime/include/expert/runtime/cuda/transformer_kernels.hpp): raw device
 * pointers, a stream passed as void*, plain integers, no C++ types.
 *
 * Every entry point returns a qllm_status code (0 = ok).  The codes mirror
 * the reference's ErrorCode enum (runtime/include/expert/runtime/storage.hpp:
 * 17-29); the text of the last failure on the calling thread is available
 * from qllm_last_error().  All pointers are device pointers unless a
 * parameter is documented as host memory.  Work is enqueued on `stream`
 * (a hipStream_t; NULL = the default stream) and is not synchronised.
 *
 * The library is HIP-only: there is no CPU fallback.  A call made on a
 * machine without a gfx950 device fails with QLLM_INTERNAL.
 */
#ifndef QLLM_KERNELS_H
#define QLLM_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum qllm_status {
  QLLM_OK = 0,
  QLLM_CANCELLED = 1,
  QLLM_DEADLINE_EXCEEDED = 2,
  QLLM_BACKPRESSURE = 3,
  QLLM_INVALID_ARGUMENT = 4,
  QLLM_OPEN_FAILED = 5,
  QLLM_IO_FAILED = 6,
  QLLM_SHORT_READ = 7,
  QLLM_CHECKSUM_MISMATCH = 8,
  QLLM_UPLOAD_FAILED = 9,
  QLLM_INTERNAL = 10
};

/* Text of the most recent non-ok status returned on this thread. */
const char* qllm_last_error(void);

/* Library build identification: "qllm-hip gfx950 <abi>". */
const char* qllm_version(void);

/* ---- FP4 weight matrices ------------------------------------------------ */

enum qllm_scale_scheme {
  /* Reference quant ABI 3: one UE8M0 byte per 32 padded columns
   * (transformer_kernels.hpp:23-32, struct Fp4Block32Matrix). */
  QLLM_SCALE_UE8M0_BLOCK32 = 0,
  /* One IEEE binary16 scale per 16 columns (the block-16 analogue of
   * struct Nvfp4Block16Matrix, transformer_kernels.hpp:44-54, with an F16
   * scale and no global factors). */
  QLLM_SCALE_F16_BLOCK16 = 1
};

enum qllm_fp4_layout {
  /* The artifact layout: row-major codes and scales as stored in QPack
   * records and handed over by the tensor store. */
  QLLM_LAYOUT_ROW_MAJOR = 0,
  /* The provider's device layout produced once, at upload, by
   * qllm_fp4_prepack: rows grouped in tiles of tile_rows (at most 32), columns
   * in chunks of 64, the sixteen-byte pieces of one (tile, chunk) contiguous
   * in the order the GEMM's lanes consume them, so weights stream in bursts of
   * up to 1 KiB. */
  QLLM_LAYOUT_TILED = 1
};

/* Packed E2M1 codes, low nibble = even column; rows keep their logical column
 * count while storage pads every row to padded_columns (a multiple of 32).
 * Mirrors Fp4Block32Matrix plus the scheme and layout tags. */
typedef struct qllm_fp4_matrix {
  const uint8_t* weights; /* row-major: [rows, padded_columns/2] */
  const void* scales;     /* u8 [rows, padded/32] or f16 [rows, padded/16] */
  uint32_t rows;
  uint32_t columns;
  uint32_t padded_columns;
  uint32_t scale_scheme;  /* enum qllm_scale_scheme */
  uint32_t layout;        /* enum qllm_fp4_layout */
  uint32_t tile_rows;     /* tiled layout: rows per tile, even, 8..32 (0 = 32) */
} qllm_fp4_matrix;

/* Device bytes needed for the tiled copy of a matrix; tile_rows even in
 * 8..32, 0 = 32; other heights return 0. */
size_t qllm_fp4_packed_weight_bytes(uint32_t rows, uint32_t padded_columns,
                                    uint32_t tile_rows);
size_t qllm_fp4_packed_scale_bytes(uint32_t rows, uint32_t padded_columns,
                                   uint32_t scale_scheme, uint32_t tile_rows);

/* Re-lays a row-major matrix (padded_columns % 64 == 0) into the tiled
 * layout with tiles of tile_rows rows (even, 8..32, 0 = 32); `packed`
 * (host struct) receives the descriptor of the copy.  This is the device half
 * of the provider's tensor upload
 * (runtime/tools/dense_fp4_provider.cpp:3486-3660); it moves bytes and changes
 * no value. */
int32_t qllm_fp4_prepack(const qllm_fp4_matrix* source, uint32_t tile_rows,
                         void* packed_weights, void* packed_scales,
                         qllm_fp4_matrix* packed, void* stream);

/* The inverse for a row range: rows [first_row, first_row + row_count) of a
 * matrix in either layout, as row-major codes [row_count, padded_columns/2] and
 * scales (u8 [row_count, padded/32] or f16 [row_count, padded/16]) in device
 * memory.  For tools and tests that need the values a provider holds (a
 * random-init model is generated directly in the tiled layout); moves bytes
 * and changes no value.  No counterpart in the reference, whose device layout
 * is the artifact's. */
int32_t qllm_fp4_unpack_rows(const qllm_fp4_matrix* matrix, uint32_t first_row,
                             uint32_t row_count, void* weights, void* scales,
                             void* stream);

enum qllm_output_kind {
  QLLM_OUT_F32 = 0,         /* float [batch, rows] */
  QLLM_OUT_F32_BF16_ROUNDED = 1, /* float storage, values rounded to bf16
                                    (the reference's bf16_output flag) */
  QLLM_OUT_BF16 = 2         /* bf16 storage [batch, rows] */
};

/* replaces quantize_q8_batch / quantize_q8_batch_bf16
 * (transformer_kernels.hpp:76-83). */
int32_t qllm_quantize_q8_batch(const float* input, int8_t* output,
                               float* scales, uint32_t rows,
                               uint32_t columns, uint32_t padded_columns,
                               int32_t bf16_input, void* stream);

/* replaces convert_f32_to_bf16_batch (transformer_kernels.hpp:84-87). */
int32_t qllm_convert_f32_to_bf16_batch(const float* input, void* output,
                                       size_t output_bytes, uint32_t rows,
                                       uint32_t columns,
                                       uint32_t padded_columns, void* stream);

/* FP4 weights x Q8 activations, batch <= 8; out[m*rows+n].
 * replaces fp4_gemv_q8_batch_weight_reuse (transformer_kernels.hpp:92-97).
 * Block-32 UE8M0 matrices; the streaming layout runs on the matrix cores
 * (qllm_fp4_gemm_q8), the row-major one on a wave per output row. */
int32_t qllm_fp4_gemv_q8_batch(const qllm_fp4_matrix* matrix,
                               const int8_t* input,
                               const float* input_scales, float* output,
                               uint32_t batch, int32_t bf16_output,
                               void* stream);

/* FP4 weights x BF16 activations [batch, padded_columns], F32 accumulate,
 * batch <= 8.  replaces fp4_gemm_bf16_block32
 * (transformer_kernels.hpp:109-112) and extends it to block-16 F16 scales.
 * `residual` (optional, float [batch, rows]) is added to the result before
 * it is stored; output may alias residual. */
int32_t qllm_fp4_gemm_bf16(const qllm_fp4_matrix* matrix, const void* input,
                           size_t input_bytes, void* output,
                           uint32_t output_kind, const float* residual,
                           uint32_t batch, void* stream);

/* One launch for projections that share their input and were stored as one
 * matrix, rows concatenated: segment s receives the next `rows` output rows
 * as its own [batch, rows] array.  The provider uses it for the q, k and v
 * projections of an attention block, three fp4_gemm_bf16_block32 calls in the
 * reference (run_full_attention, dense_fp4_provider.cpp:7004-7011); every
 * output value equals what the separate calls give.  K % 64 == 0, at most
 * three segments. */
typedef struct qllm_gemm_segment {
  void* output;         /* [batch, rows] */
  uint32_t rows;
  uint32_t output_kind; /* enum qllm_output_kind */
} qllm_gemm_segment;
int32_t qllm_fp4_gemm_bf16_split(const qllm_fp4_matrix* matrix,
                                 const void* input, size_t input_bytes,
                                 const qllm_gemm_segment* segments,
                                 uint32_t segment_count, uint32_t batch,
                                 void* stream);

/* The reference's default activation contract on the matrix cores: int8 rows
 * with one F32 scale each (qllm_quantize_q8_batch) against block-32 UE8M0
 * weights in the streaming layout, out = 0.5 * s_m * sum over blocks of
 * 2^(e - 127) * (integer block sum) - the statement of
 * fp4_gemv_q8_batch5_tensor_core_kernel (transformer_kernels.cu:1162-1275),
 * called from project_quantized (dense_fp4_provider.cpp:6229-6267).  Block sums
 * are exact, blocks are accumulated in F32.  K % 64 == 0; input 16-byte
 * aligned, [batch, padded_columns] int8.  `residual` as in qllm_fp4_gemm_bf16.
 * The split form serves q/k/v stored as one matrix, the SwiGLU form stores
 * silu(gate) * up as F32 (silu_product_kernel without bf16 rounding,
 * transformer_kernels.cu:2774-2783): the reference quantises that product to
 * Q8 again before the down projection.  `workspace` of the split and SwiGLU
 * forms: NULL, or the balanced-tail workspace described further down. */
int32_t qllm_fp4_gemm_q8(const qllm_fp4_matrix* matrix, const int8_t* input,
                         const float* input_scales, void* output,
                         uint32_t output_kind, const float* residual,
                         uint32_t batch, void* stream);
int32_t qllm_fp4_gemm_q8_split(const qllm_fp4_matrix* matrix, const int8_t* input,
                               const float* input_scales,
                               const qllm_gemm_segment* segments,
                               uint32_t segment_count, uint32_t batch,
                               void* workspace, size_t workspace_bytes,
                               void* stream);
/* qllm_fp4_gemm_q8 with K cut over k_splits workgroups per tile, as
 * qllm_fp4_gemm_bf16_partial cuts it: partials f32 [k_splits][batch][rows],
 * each already times the row's activation scale; the consumer adds them in
 * index order (qllm_rms_norm_partials_q8_batch does).  Against the one-sum
 * form the F32 additions are regrouped, nothing else. */
int32_t qllm_fp4_gemm_q8_partial(const qllm_fp4_matrix* matrix, const int8_t* input,
                                 const float* input_scales, float* partials,
                                 uint32_t k_splits, uint32_t batch, void* stream);
int32_t qllm_fp4_swiglu_q8(const qllm_fp4_matrix* gate, const qllm_fp4_matrix* up,
                           const int8_t* input, const float* input_scales,
                           float* output, uint32_t batch, void* workspace,
                           size_t workspace_bytes, void* stream);


/* The same product with K cut over k_splits workgroups per tile (tiled layout
 * only, 1 <= k_splits <= 16): partials f32 [k_splits][batch][rows], split s
 * holding the sum over its share of the 64-column chunks.  For matrices with
 * too few rows to occupy the GPU (o and down projections); the consumer adds
 * the partials in index order (qllm_rms_norm_residual_batch does), which
 * keeps the result independent of the launch's timing.  The reference has one
 * thread block per output row group and no such cut
 * (transformer_kernels.cu:7559-7593). */
int32_t qllm_fp4_gemm_bf16_partial(const qllm_fp4_matrix* matrix,
                                   const void* input, size_t input_bytes,
                                   float* partials, uint32_t k_splits,
                                   uint32_t batch, void* stream);

/* Balanced forms of the two launches above and below whose tile count leaves a
 * ragged last round over the CUs (the q/k/v launch: 320 tiles, the gate/up
 * launch: 544 tile pairs, on 256 CUs): the tiles past the last full round are
 * cut along K over as many small workgroups as give every CU one more, equal,
 * share; the small workgroup that finishes a tile last adds the others' sums in
 * a fixed order and runs the epilogue.  Values of the cut tiles differ from the
 * plain launch in F32 summation order only.  `workspace`: device memory of
 * qllm_fp4_gemm_balance_workspace_bytes() bytes, 16-byte aligned, zeroed once
 * by the caller and then left alone (the kernel returns its counters to zero);
 * launches that share a workspace must not overlap.  No counterpart in the
 * reference, whose launches have one thread block per output row group
 * (transformer_kernels.cu:7559-7593). */
size_t qllm_fp4_gemm_balance_workspace_bytes(void);
int32_t qllm_fp4_gemm_bf16_split_balanced(const qllm_fp4_matrix* matrix,
                                          const void* input, size_t input_bytes,
                                          const qllm_gemm_segment* segments,
                                          uint32_t segment_count, uint32_t batch,
                                          void* workspace, size_t workspace_bytes,
                                          void* stream);
int32_t qllm_fp4_swiglu_bf16_balanced(const qllm_fp4_matrix* gate,
                                      const qllm_fp4_matrix* up, const void* input,
                                      size_t input_bytes, void* output,
                                      uint32_t batch, void* workspace,
                                      size_t workspace_bytes, void* stream);

/* Gate and up projections of one SwiGLU block in a single pass over a shared
 * BF16 input: out[m,n] = bf16(bf16(silu(gate[m,n])) * up[m,n]) stored as
 * bf16 [batch, rows].  Fuses two qllm_fp4_gemm_bf16 calls with silu_product
 * (transformer_kernels.hpp:415-418, run_ffn dense_fp4_provider.cpp:8250-8293).
 * Both matrices must share shape and scale scheme. */
int32_t qllm_fp4_swiglu_bf16(const qllm_fp4_matrix* gate,
                             const qllm_fp4_matrix* up, const void* input,
                             size_t input_bytes, void* output,
                             uint32_t batch, void* stream);

/* The GEMM for tall batches (prompt prefill): any batch, a matrix in the tiled
 * layout with 32-row tiles, input bf16 [batch, padded_columns] (16-byte
 * aligned), output [batch, rows] in `output_kind`, optional F32 residual of
 * the same shape.  Workgroups of 128 batch rows x 256 weight rows on the
 * matrix cores.  With UE8M0 scales the arithmetic is the reference's (exact
 * bf16 operands, F32 accumulation); with binary16 scales the scaled weights
 * and the activations enter as binary16 (see the kernel's header).
 * replaces fp4_gemm_bf16_block32 at batch > 8 (transformer_kernels.cu:
 * 1284-1430, launched from :7400-7593). */
int32_t qllm_fp4_gemm_bf16_tall(const qllm_fp4_matrix* matrix, const void* input,
                                size_t input_bytes, void* output,
                                uint32_t output_kind, const float* residual,
                                uint32_t batch, void* stream);
/* The tall GEMM on the gate and the up matrix of a SwiGLU block at once (same
 * shape, scheme and tiled layout): output bf16 [batch, rows] =
 * bf16(bf16(silu(gate . x)) * (up . x)), the rounding points of
 * qllm_silu_product with bf16 activations.  The tall counterpart of
 * qllm_fp4_swiglu_bf16; the reference runs two GEMMs and swiglu_kernel
 * (runtime/tools/dense_fp4_provider.cpp:8250-8293). */
int32_t qllm_fp4_swiglu_bf16_tall(const qllm_fp4_matrix* gate,
                                  const qllm_fp4_matrix* up, const void* input,
                                  size_t input_bytes, void* output_bf16,
                                  uint32_t batch, void* stream);

/* The same with the output columns split over up to three buffers, each a
 * multiple of 32 weight rows (the q, k and v projections stored as one
 * matrix). */
int32_t qllm_fp4_gemm_bf16_tall_split(const qllm_fp4_matrix* matrix,
                                      const void* input, size_t input_bytes,
                                      const qllm_gemm_segment* segments,
                                      uint32_t segment_count, uint32_t batch,
                                      void* stream);

/* replaces fp4_embedding_batch (transformer_kernels.hpp:68-70).  A token
 * outside the matrix (tokens[r] >= rows; a device-side selection over logits
 * without a finite maximum yields 0xffffffff) reads nothing and gives a row of
 * zeros; host callers validate tokens themselves, as the reference does. */
int32_t qllm_fp4_embedding_batch(const qllm_fp4_matrix* matrix,
                                 const uint32_t* tokens, float* output,
                                 uint32_t batch, void* stream);

/* ---- normalisation and elementwise ---------------------------------------- */

/* replaces rms_norm_batch / weightless_rms_norm_batch and the zero-centred
 * variant (transformer_kernels.hpp:303-309).  weight may be NULL.  Exactly
 * one of output_f32 / output_bf16 may be NULL; bf16 rows are padded with
 * zeros to bf16_padded_columns. */
int32_t qllm_rms_norm_batch(const float* input, const float* weight,
                            float* output_f32, void* output_bf16,
                            uint32_t bf16_padded_columns, uint32_t rows,
                            uint32_t elements, float epsilon,
                            int32_t zero_centered, void* stream);

/* RMSNorm of every row followed by its per-row Q8 quantisation, in one launch:
 * normalize_rows then quantize_rows of the reference
 * (dense_fp4_provider.cpp:5740-5778, 5983-5992; kernels
 * transformer_kernels.cu:2469-2503, 912-946) with the same operations on the
 * same F32 values, so codes and scales equal qllm_rms_norm_batch followed by
 * qllm_quantize_q8_batch.  elements % 4 == 0, at most 16384; pointers 16-byte
 * aligned; output_q8 [rows, elements], scales [rows]. */
int32_t qllm_rms_norm_q8_batch(const float* input, const float* weight,
                               int8_t* output_q8, float* scales, uint32_t rows,
                               uint32_t elements, float epsilon,
                               int32_t zero_centered, void* stream);

/* The residual add of a projection computed as K-split partials
 * (qllm_fp4_gemm_bf16_partial) folded into the RMSNorm that follows:
 * hidden[r] += partials[0][r] + ... + partials[count-1][r] (in that order;
 * partials f32 [count][rows][elements]), output_bf16[r] = RMSNorm(hidden[r]).
 * Replaces add_kernel + rms_batch_kernel of the reference
 * (transformer_kernels.cu:2522-2528, 2469-2503) for that case.  elements % 4
 * == 0, at most 16384; pointers 16-byte aligned; 1 <= count <= 16. */
int32_t qllm_rms_norm_residual_batch(float* hidden, const float* partials,
                                     uint32_t partial_count,
                                     const float* weight, void* output_bf16,
                                     uint32_t rows, uint32_t elements,
                                     float epsilon, int32_t zero_centered,
                                     void* stream);

/* The same with the sum written elsewhere: sum[r] = residual[r] + partials[0][r]
 * + ... (from zero when residual is NULL), output_bf16[r] = RMSNorm(sum[r]).
 * The proposer's projections use it: the fusion projection has no residual
 * (run_mtp, dense_fp4_provider.cpp:8716-8735) and a single-row pass leaves its
 * last sum where the next pass reads it (:8766-8783).  `sum` may be
 * `residual`; same limits as above. */
int32_t qllm_rms_norm_partials_batch(const float* residual, float* sum,
                                     const float* partials, uint32_t partial_count,
                                     const float* weight, void* output_bf16,
                                     uint32_t rows, uint32_t elements,
                                     float epsilon, int32_t zero_centered,
                                     void* stream);

/* qllm_rms_norm_partials_batch with the norm's output in per-row Q8 form, as
 * qllm_rms_norm_q8_batch leaves it (normalize_rows + quantize_rows,
 * dense_fp4_provider.cpp:5740-5778, 5983-5992). */
int32_t qllm_rms_norm_partials_q8_batch(const float* residual, float* sum,
                                        const float* partials,
                                        uint32_t partial_count, const float* weight,
                                        int8_t* output_q8, float* scales,
                                        uint32_t rows, uint32_t elements,
                                        float epsilon, int32_t zero_centered,
                                        void* stream);

/* Two normalisations into one bf16 batch: output row r, of 2 * elements
 * columns, is [RMSNorm(first[r]) | RMSNorm(second[r])], each half with its own
 * weight (either may be NULL) and the values of qllm_rms_norm_batch.  The
 * proposer's fusion input; replaces two normalize_rows calls and the two
 * cudaMemcpy2D that interleave them (runtime/tools/dense_fp4_provider.cpp:
 * 8710-8723).  elements % 4 == 0, at most 16384; inputs and weights 16-byte
 * aligned. */
int32_t qllm_rms_norm_concat_batch(const float* first,
                                   const float* first_weight,
                                   const float* second,
                                   const float* second_weight,
                                   void* output_bf16, uint32_t rows,
                                   uint32_t elements, float epsilon,
                                   int32_t zero_centered, void* stream);

/* The same with the first half's rows taken from an FP4 embedding matrix
 * (row-major) at `tokens`: qllm_fp4_embedding_batch folded into the norm - the
 * proposer's embedding lookup and its two input norms in one launch (run_mtp,
 * dense_fp4_provider.cpp:8699-8735).  Same values as the lookup followed by
 * qllm_rms_norm_concat_batch; elements = embedding->columns.  presence (NULL,
 * or vocabulary bytes): the batch's tokens are marked as qllm_mark_presence
 * marks them - the pass over the tokens a verify step emitted
 * (:11261-11270). */
int32_t qllm_rms_norm_concat_embedding_batch(
    const qllm_fp4_matrix* embedding, const uint32_t* tokens,
    const float* first_weight, const float* second, const float* second_weight,
    void* output_bf16, uint32_t rows, float epsilon, int32_t zero_centered,
    uint8_t* presence, void* stream);

/* replaces add_in_place (transformer_kernels.hpp:310-312). */
int32_t qllm_add_in_place(float* destination, const float* source,
                          uint32_t elements, int32_t bf16_output,
                          void* stream);

/* replaces silu_product (transformer_kernels.hpp:415-418). */
int32_t qllm_silu_product(const float* gate, const float* up, float* output,
                          uint32_t elements, int32_t bf16_activations,
                          void* stream);

/* ---- attention: Q4H ("q4-f16-per-head") paged cache ----------------------- */

/* Bytes one layer occupies inside a Q4H page:
 * page_tokens * kv_heads * 2 * (head_dim/2 + 2). */
size_t qllm_q4h_layer_bytes(uint32_t page_tokens, uint32_t kv_heads,
                            uint32_t head_dim);

/* Per-head RMSNorm (1+w) [skipped when the weight pointer is NULL], NeoX
 * rotary on the first rotary_dim dimensions, then Q4H-encode and store the
 * K/V rows of `rows` consecutive positions into their pages.
 * replaces gated_gqa_qkv_rope_cache_paged_q4_per_head_batch
 * (transformer_kernels.hpp:719-729).  query_stride is the distance in floats
 * between consecutive query heads (2*head_dim for the output-gated layout,
 * head_dim for plain GQA); query is updated in place. */
int32_t qllm_qkv_rope_cache_paged_q4h_batch(
    float* query, uint32_t query_stride, float* key, const float* value,
    const float* q_norm_weight, const float* k_norm_weight,
    const void* const* page_table, uint32_t full_attention_layer,
    uint32_t page_tokens, uint32_t first_cache_position,
    uint32_t first_rotary_position, uint32_t rows, uint32_t query_heads,
    uint32_t kv_heads, uint32_t head_dim, uint32_t rotary_dim, float epsilon,
    float rope_theta, int32_t bf16_activations, void* stream);

/* The same operation with the positions read on the device when the kernel
 * runs: device_positions[0] = first cache position, [1] = first rotary
 * position.  Lets a captured HIP graph be replayed at advancing positions. */
int32_t qllm_qkv_rope_cache_paged_q4h_batch_deferred(
    float* query, uint32_t query_stride, float* key, const float* value,
    const float* q_norm_weight, const float* k_norm_weight,
    const void* const* page_table, uint32_t full_attention_layer,
    uint32_t page_tokens, const uint32_t* device_positions, uint32_t rows,
    uint32_t query_heads, uint32_t kv_heads, uint32_t head_dim,
    uint32_t rotary_dim, float epsilon, float rope_theta,
    int32_t bf16_activations, void* stream);

/* The same operation fed by a q/k/v projection that was computed as K-split
 * partials (qllm_fp4_gemm_bf16_partial on the matrix holding the query, key
 * and value rows in that order): partials f32 [partial_count][rows]
 * [query_heads * query_stride + 2 * kv_heads * head_dim].  Every (row, head)
 * workgroup first adds its slice of the partials in index order into `query`
 * (dense rows of query_heads * query_stride floats), `key` and `value`, then
 * goes on as qllm_qkv_rope_cache_paged_q4h_batch; device_positions, when not
 * NULL, replaces the two positions as in the deferred form.  The reference
 * has one thread block per output row group in its projection and no such cut
 * (runtime/tools/dense_fp4_provider.cpp:7004-7011). */
int32_t qllm_qkv_rope_cache_paged_q4h_from_partials(
    const float* partials, uint32_t partial_count, float* query,
    uint32_t query_stride, float* key, float* value,
    const float* q_norm_weight, const float* k_norm_weight,
    const void* const* page_table, uint32_t full_attention_layer,
    uint32_t page_tokens, uint32_t first_cache_position,
    uint32_t first_rotary_position, const uint32_t* device_positions,
    uint32_t rows, uint32_t query_heads, uint32_t kv_heads, uint32_t head_dim,
    uint32_t rotary_dim, float epsilon, float rope_theta,
    int32_t bf16_activations, void* stream);

/* The same operation (partials may be NULL: query, key and value then hold the
 * projection already), which also leaves the rotated queries as the operands
 * of qllm_attention_paged_q4h: per KV head and 16-row tile of its rows *
 * (query_heads / kv_heads) matrix rows (row r, head h of the group at r *
 * group + h) and per 64 elements of head_dim, a high and a low int8 plane of
 * 1 KiB in matrix-core order, query = scale * (128 * high + low) to 15 bits of
 * the row's largest magnitude; query_operand_scales holds 16 floats per row
 * tile and KV head, the scale times log2(e) / (16 sqrt(head_dim)).
 * query_operands: qllm_q4h_query_operand_bytes() bytes, 16-byte aligned; rows
 * of a tile past the batch are left untouched.  head_dim in {128, 256},
 * rows * (query_heads / kv_heads) <= 48 (32 at head_dim 256).  The reference
 * quantises its queries in a kernel of its own
 * (quantize_gqa_queries_q8_kernel, transformer_kernels.cu:4391-4416). */
size_t qllm_q4h_query_operand_bytes(uint32_t rows, uint32_t query_heads,
                                    uint32_t kv_heads, uint32_t head_dim);
int32_t qllm_qkv_rope_cache_paged_q4h_prepared(
    const float* partials, uint32_t partial_count, float* query,
    uint32_t query_stride, float* key, float* value,
    const float* q_norm_weight, const float* k_norm_weight,
    const void* const* page_table, uint32_t full_attention_layer,
    uint32_t page_tokens, uint32_t first_cache_position,
    uint32_t first_rotary_position, const uint32_t* device_positions,
    uint32_t rows, uint32_t query_heads, uint32_t kv_heads, uint32_t head_dim,
    uint32_t rotary_dim, float epsilon, float rope_theta,
    int32_t bf16_activations, int8_t* query_operands,
    float* query_operand_scales, void* stream);

/* The same per-head RMSNorm + rotary without the K/V store, for caches that
 * store K/V separately.  replaces gated_gqa_qkv_rope_fp16_batch
 * (runtime/src/cuda/transformer_kernels.cu:3645-3726). */
int32_t qllm_qkv_rope_batch(float* query, uint32_t query_stride, float* key,
                            const float* q_norm_weight,
                            const float* k_norm_weight,
                            uint32_t first_rotary_position, uint32_t rows,
                            uint32_t query_heads, uint32_t kv_heads,
                            uint32_t head_dim, uint32_t rotary_dim,
                            float epsilon, float rope_theta,
                            int32_t bf16_activations, void* stream);

/* qllm_qkv_rope_batch with the position read on the device when the kernel
 * runs: device_positions[1] = first rotary position. */
int32_t qllm_qkv_rope_batch_deferred(float* query, uint32_t query_stride,
                                     float* key, const float* q_norm_weight,
                                     const float* k_norm_weight,
                                     const uint32_t* device_positions,
                                     uint32_t rows, uint32_t query_heads,
                                     uint32_t kv_heads, uint32_t head_dim,
                                     uint32_t rotary_dim, float epsilon,
                                     float rope_theta,
                                     int32_t bf16_activations, void* stream);

/* replaces store_gqa_kv_paged_q4_per_head_batch (the store-only form used
 * by runtime/tools/dense_fp4_cuda_smoke.cpp:1828-1832). */
int32_t qllm_store_kv_paged_q4h_batch(const float* key, const float* value,
                                      const void* const* page_table,
                                      uint32_t full_attention_layer,
                                      uint32_t page_tokens,
                                      uint32_t first_cache_position,
                                      uint32_t rows, uint32_t kv_heads,
                                      uint32_t head_dim, void* stream);

/* replaces quantize_gqa_queries_q8 (transformer_kernels.hpp:851-854). */
int32_t qllm_quantize_gqa_queries_q8(const float* query,
                                     uint32_t query_stride, int8_t* q8,
                                     float* query_scales, uint32_t rows,
                                     uint32_t query_heads, uint32_t head_dim,
                                     void* stream);

/* Mirrors PagedQ4BfpGatedGqaAttentionLaunch (transformer_kernels.hpp:826-846)
 * for gated_gqa_attention_microbatch_paged_q4_per_head_tensor_core. */
typedef struct qllm_q4h_attention_launch {
  const float* query;           /* [rows, query_heads, query_stride], 16-byte
                                   aligned; the kernel quantises it itself
                                   unless the next two fields are set */
  const int8_t* q8_queries;     /* NULL, or the query operands that
                                   qllm_qkv_rope_cache_paged_q4h_prepared left
                                   for these rows (two int8 planes, not the
                                   reference's single Q8 plane) */
  const float* query_scales;    /* NULL, or the operand scales of the same call */
  const void* const* page_table;
  void* output;                 /* [rows, query_heads, head_dim] */
  float* partial_maxima;        /* [rows, maximum_splits, query_heads] */
  float* partial_sums;          /* same */
  float* partial_outputs;       /* [rows, maximum_splits, query_heads, d] */
  uint32_t first_context_tokens;/* row r attends tokens [0, first + r) */
  uint32_t rows;
  uint32_t full_attention_layer;
  uint32_t page_tokens;
  uint32_t query_heads;
  uint32_t kv_heads;
  uint32_t head_dim;
  uint32_t split_tokens;        /* tokens per context split, a multiple of 64;
                                   0 = balanced: the context's 64-token tiles
                                   are dealt evenly over maximum_splits
                                   workgroups, whatever the context length
                                   (no counterpart in the reference) */
  uint32_t maximum_splits;      /* <= 2048 */
  uint32_t query_stride;        /* floats between heads in `query` */
  int32_t output_gated;         /* multiply by sigmoid(query[d + i]) */
  uint32_t output_kind;         /* QLLM_OUT_F32 or QLLM_OUT_BF16 */
  void* stream;
  /* Optional (NULL = unused).  When set, first_context_tokens is read from
   * device_positions[2] when the kernels run and the launch covers all
   * maximum_splits, so a captured graph can be replayed as the context
   * grows.  No counterpart in the reference struct. */
  const uint32_t* device_positions;
} qllm_q4h_attention_launch;

/* Split phase + split-K combine.  rows * (query_heads/kv_heads) <= 48,
 * head_dim in {128, 256}, page_tokens % 64 == 0, split_tokens % 64 == 0.
 * The pages must hold every 64-token tile that overlaps the context. */
int32_t qllm_attention_paged_q4h(const qllm_q4h_attention_launch* launch);
/* The same launch doing the rotary kernel's work for the batch as well (the
 * reference keeps them apart: gated_gqa_qkv_rope_paged_batch_kernel,
 * transformer_kernels.cu:3550-3643, then the attention kernel).  launch->query
 * holds the projection's raw query rows and is left as it is; key / value
 * [rows, kv_heads, head_dim] the raw K and V rows.  Every workgroup normalises
 * (weights may be NULL) and rotates the query rows of its KV head with the
 * (cos, sin) pairs of rope_table - qllm_rope_table, [rows][rotary_dim / 2][2] -
 * and quantises them as qllm_qkv_rope_cache_paged_q4h_prepared does; the
 * batch's K/V records (cache positions first_cache_position .. + rows - 1, the
 * last `rows` tokens of the context: first_cache_position + 1 ==
 * first_context_tokens) are encoded by the workgroups that attend them and
 * written to their pages by one of them.  With launch->device_positions the
 * cache position is device_positions[0].  Outputs and page bytes equal those of
 * the two separate launches. */
typedef struct qllm_q4h_fused_rope {
  const float* key;
  const float* value;
  const float* q_norm_weight;   /* NULL: no per-head norm */
  const float* k_norm_weight;
  const float* rope_table;
  uint32_t rotary_dim;
  float epsilon;
  uint32_t first_cache_position;
  int32_t bf16_activations;
} qllm_q4h_fused_rope;
int32_t qllm_attention_paged_q4h_fused(const qllm_q4h_attention_launch* launch,
                                       const qllm_q4h_fused_rope* rope);
/* (cos, sin) of the rotary angles of rows at positions first_rotary_position
 * .. + rows - 1 (or from device_positions[1]), pair p of row r at
 * table[(r * rotary_dim / 2 + p) * 2]: the values the rotary kernels compute
 * for themselves (angle = position * theta^(-2p / rotary_dim)). */
int32_t qllm_rope_table(float* table, uint32_t rows, uint32_t rotary_dim,
                        uint32_t first_rotary_position, float rope_theta,
                        int32_t bf16_activations,
                        const uint32_t* device_positions, void* stream);
/* Many micro-batches in one launch (prompt prefill): the launch's `rows` rows
 * are attended in batches of `batch_rows` consecutive rows, batch b exactly as
 * a launch of its own with first_context_tokens + b * batch_rows would be
 * (row r of the whole attends tokens [0, first_context_tokens + r)), all
 * batches side by side in one grid.  query, output and the partial buffers
 * hold `rows` rows; batch_rows * (query_heads/kv_heads) <= 48 (32 at head_dim
 * 256); rows <= 65535; device_positions must be NULL.  No counterpart in the
 * reference, whose prefill attention is a kernel of its own
 * (transformer_kernels.cu:9906-10153). */
int32_t qllm_attention_paged_q4h_batched(const qllm_q4h_attention_launch* launch,
                                         uint32_t batch_rows);

/* The same attention for a long run of prompt rows (head_dim 128,
 * split_tokens 0): eight consecutive batches share a workgroup, which fetches
 * every cache tile once for the eight and converts its V codes and scales to
 * matrix-core operands once; every batch (one wave) walks the tiles of its
 * own context in order, so sums differ from the batched launch's in the last
 * bits (other order of F32 additions), the records read and the arithmetic per
 * score are the same.  maximum_splits cuts the tiles of a workgroup's longest
 * context evenly (1 when rows / (8 batch_rows) * kv_heads workgroups fill the
 * GPU).  Replaces the reference's prefill attention
 * (transformer_kernels.cu:9906-10153: 64-row query blocks per cache tile). */
int32_t qllm_attention_paged_q4h_prompt(const qllm_q4h_attention_launch* launch,
                                        uint32_t batch_rows);

/* ---- attention: exact F16 paged cache ---------------------------------------- */

/* Per-layer page layout: K [page_tokens][kv_heads][head_dim] then
 * V [page_tokens][kv_heads][head_dim], binary16
 * (transformer_kernels.cu:6594-6606).
 * replaces store_gqa_kv_fp16_to_paged. */
int32_t qllm_store_kv_paged_f16_batch(const float* key, const float* value,
                                      const void* const* page_table,
                                      uint32_t full_attention_layer,
                                      uint32_t page_tokens,
                                      uint32_t first_cache_position,
                                      uint32_t rows, uint32_t kv_heads,
                                      uint32_t head_dim, void* stream);

/* Mirrors DeviceFp16GatedGqaAttentionLaunch (transformer_kernels.hpp:
 * 1071-1092), paged-device form, for gated_gqa_attention_staged_device_fp16.
 * Unlike the reference's sequential split loop, splits run in parallel and
 * are merged by the same combine kernel as the Q4H path. */
typedef struct qllm_f16_attention_launch {
  const float* query;
  const void* const* device_pages;
  void* output;
  float* partial_maxima;
  float* partial_sums;
  float* partial_outputs;
  uint32_t first_context_tokens;
  uint32_t rows;
  uint32_t device_page_layer;
  uint32_t device_page_tokens;
  uint32_t query_heads;
  uint32_t kv_heads;
  uint32_t head_dim;
  uint32_t split_tokens;
  uint32_t maximum_splits;
  uint32_t query_stride;
  int32_t output_gated;
  uint32_t output_kind;
  void* stream;
} qllm_f16_attention_launch;

int32_t qllm_attention_paged_f16(const qllm_f16_attention_launch* launch);
/* The batched form for prompt prefill, as qllm_attention_paged_q4h_batched. */
int32_t qllm_attention_paged_f16_batched(const qllm_f16_attention_launch* launch,
                                         uint32_t batch_rows);

/* ---- attention: Q8 paged cache (the proposer's) ------------------------------- */

/* Symmetric int8 codes with one binary16 scale per K or V head record,
 *   scale = f16(max(absmax/127, 2^-24)), code = clamp(rn(x/scale), -127, 127)
 * (transformer_kernels.cu:601-625).  The reference interleaves codes and scale
 * in records of head_dim + 2 bytes; this library keeps the same values in
 * planes, `page_offset_bytes` (a multiple of 16) into the page:
 *   K codes [page_tokens][kv_heads][head_dim] int8, V codes likewise,
 *   K scales [kv_heads][page_tokens] binary16, V scales likewise
 * - qllm_q8_layer_bytes() per layer, the reference's size.  The pages are
 * private to the provider, so the placement is not an interface.
 * replaces store_gqa_kv_paged_q8_batch (transformer_kernels.hpp:403-409). */
size_t qllm_q8_layer_bytes(uint32_t page_tokens, uint32_t kv_heads,
                           uint32_t head_dim);
int32_t qllm_store_kv_paged_q8_batch(const float* key, const float* value,
                                     const void* const* page_table,
                                     size_t page_offset_bytes,
                                     uint32_t page_tokens,
                                     uint32_t first_cache_position,
                                     uint32_t rows, uint32_t kv_heads,
                                     uint32_t head_dim, void* stream);

/* The same store with the position read on the device when the kernel runs:
 * device_positions[0] = first cache position. */
int32_t qllm_store_kv_paged_q8_batch_deferred(
    const float* key, const float* value, const void* const* page_table,
    size_t page_offset_bytes, uint32_t page_tokens,
    const uint32_t* device_positions, uint32_t rows, uint32_t kv_heads,
    uint32_t head_dim, void* stream);

/* qllm_qkv_rope_batch and qllm_store_kv_paged_q8_batch in one launch: the
 * rotary of a batch's queries and keys, then the rotated key and the value of
 * every (row, kv head) as Q8 records - the proposer's
 * gated_gqa_qkv_rope_paged_batch_kernel<q8> (transformer_kernels.cu:3550-3643,
 * records :601-625).  Same values and bytes as the two launches.
 * device_positions (NULL, or device words read when the kernel runs): word 0
 * the first cache position, word 1 the first rotary position. */
int32_t qllm_qkv_rope_store_q8_batch(
    float* query, uint32_t query_stride, float* key, const float* value,
    const float* q_norm_weight, const float* k_norm_weight,
    const void* const* page_table, size_t page_offset_bytes, uint32_t page_tokens,
    uint32_t first_cache_position, uint32_t first_rotary_position,
    const uint32_t* device_positions, uint32_t rows, uint32_t query_heads,
    uint32_t kv_heads, uint32_t head_dim, uint32_t rotary_dim, float epsilon,
    float rope_theta, int32_t bf16_activations, void* stream);

/* replaces gated_gqa_attention_microbatch_paged_q8_tensor_core and
 * gated_gqa_attention_decode_paged_q8_tensor_core (transformer_kernels.hpp:
 * 873, 944; launch struct PagedQ8GatedGqaPrefillLaunch): row r attends tokens
 * [0, first_context_tokens + r).  Codes enter the matrix cores as exact
 * binary16 integers, the query as binary16 (the reference rounds q, k, v and
 * the probabilities to bf16), splits run in parallel and share the combine
 * kernel of the other caches.  page_tokens % 32 == 0, head_dim 128 or 256,
 * rows * (query_heads/kv_heads) <= 48 (32 at head_dim 256), split_tokens % 32
 * == 0 (0 = context dealt evenly over maximum_splits workgroups per KV head). */
typedef struct qllm_q8_attention_launch {
  const float* query;
  const void* const* device_pages;
  void* output;
  float* partial_maxima;
  float* partial_sums;
  float* partial_outputs;
  size_t page_offset_bytes;
  uint32_t first_context_tokens;
  uint32_t rows;
  uint32_t page_tokens;
  uint32_t query_heads;
  uint32_t kv_heads;
  uint32_t head_dim;
  uint32_t split_tokens;
  uint32_t maximum_splits;
  uint32_t query_stride;
  int32_t output_gated;
  uint32_t output_kind;
  void* stream;
  /* optional: when set, first_context_tokens is read from
   * device_positions[2] when the kernels run and every split is launched */
  const uint32_t* device_positions;
} qllm_q8_attention_launch;

int32_t qllm_attention_paged_q8(const qllm_q8_attention_launch* launch);

/* qllm_attention_paged_q8 for a prompt chunk: `rows` query rows served in
 * batches of batch_rows (grid layer z = rows z*batch_rows ..., each row with
 * its own context first_context_tokens + row), one launch and one combine.
 * Partials are laid out by global row.  rows <= 65535; device_positions must
 * be NULL.  No counterpart in the reference, which feeds the proposer five
 * rows at a time (dense_fp4_provider.cpp:8681-8792). */
int32_t qllm_attention_paged_q8_batched(const qllm_q8_attention_launch* launch,
                                        uint32_t batch_rows);

/* ---- token selection ------------------------------------------------------------ */

/* Chains greedy proposer passes on the device (no counterpart in the
 * reference, whose rollout, dense_fp4_provider.cpp:8794-8852, returns to the
 * host after every pass): selected[0] becomes next_token[0] and
 * draft_tokens[device_positions[3]] (when that slot is below `capacity`);
 * device_positions[0..2] - cache position, rotary position, context tokens -
 * advance by `rows`, the pass's row count, and the draft slot [3] by one. */
int32_t qllm_rollout_advance(const uint32_t* selected, uint32_t* next_token,
                             uint32_t* draft_tokens, uint32_t capacity,
                             uint32_t rows, uint32_t* device_positions,
                             void* stream);

/* A head: logits [batch, rows] = matrix . input (qllm_fp4_gemm_bf16, F32
 * output) and tokens[m] = arg-max of row m (qllm_argmax_batch's ordering:
 * larger first, ties to the lower id, NaN never, 0xffffffff for a row without
 * a selectable value), in two launches: the projection's epilogue leaves every
 * tile's best (value, row) in `workspace`, one block per batch row picks the
 * winner.  Replaces the projection followed by argmax_batch_kernel in run_head
 * (dense_fp4_provider.cpp:8393-8432; kernel transformer_kernels.cu:7059-7092)
 * without the second pass over the logits.  With `advance` (batch 1) the
 * winner is also handed on as qllm_rollout_advance does.  K % 64 == 0. */
typedef struct qllm_rollout_step {
  uint32_t* next_token;        /* device: the next pass's input token */
  uint32_t* draft_tokens;      /* device: draft list, entry positions[3] */
  uint32_t capacity;           /* entries of draft_tokens */
  uint32_t rows;               /* positions 0..2 advance by this */
  uint32_t* device_positions;  /* device: cache, rotary, context, draft slot */
} qllm_rollout_step;
size_t qllm_fp4_head_workspace_bytes(const qllm_fp4_matrix* matrix, uint32_t batch);
int32_t qllm_fp4_head_argmax(const qllm_fp4_matrix* matrix, const void* input,
                             size_t input_bytes, float* logits, uint32_t batch,
                             uint32_t* tokens, void* workspace,
                             size_t workspace_bytes,
                             const qllm_rollout_step* advance, void* stream);

/* replaces argmax_batch (transformer_kernels.hpp:1266-1269): ties to the
 * lower index, NaN never wins.  workspace: at least
 * qllm_argmax_workspace_bytes(count, batch) bytes of device memory. */
size_t qllm_argmax_workspace_bytes(uint32_t count, uint32_t batch);
int32_t qllm_argmax_batch(const float* values, uint32_t count,
                          uint32_t batch, uint32_t* output, void* workspace,
                          size_t workspace_bytes, void* stream);

/* qllm_argmax_batch for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid it): the same
 * kernels and results, the stage-1 partials in a fixed 64 KiB array inside
 * the library's code object instead of a workspace.  No counterpart in the
 * reference.  Calls no allocating routine.  Limit: ceil(count / 2048) * batch
 * <= 8192 (qllm_argmax_workspace_bytes(count, batch) <=
 * qllm_argmax_static_capacity_bytes()); larger requests fail with
 * QLLM_INVALID_ARGUMENT.  Every call on a GPU shares that GPU's array: calls
 * that overlap on one GPU (different streams, threads or provider instances)
 * race, and nothing detects it.  The first call on a device looks the array's
 * address up and must be made outside stream capture; later calls only launch
 * kernels. */
size_t qllm_argmax_static_capacity_bytes(void);
int32_t qllm_argmax_batch_static(const float* values, uint32_t count,
                                 uint32_t batch, uint32_t* output,
                                 void* stream);

/* replaces topk_logits (transformer_kernels.hpp:1271-1290): exact descending
 * top-k of one row, ties to the lower id, NaN excluded, k <= 1024. */
size_t qllm_topk_workspace_bytes(uint32_t count, uint32_t top_k);
int32_t qllm_topk_logits(const float* values, uint32_t count, uint32_t top_k,
                         float* output_values, uint32_t* output_indices,
                         void* workspace, size_t workspace_bytes,
                         void* stream);

/* The same selection for `rows` rows of logits in two launches (k <= 64):
 * values f32 [rows][row_stride] (the first `count` of each row), outputs
 * [rows][top_k].  Same order, ties and padding as qllm_topk_logits.  The
 * reference selects row by row (topk_logits, transformer_kernels.cu:7096-7178,
 * one call per target row, dense_fp4_provider.cpp:8331-8391). */
size_t qllm_topk_batch_workspace_bytes(uint32_t count, uint32_t top_k,
                                       uint32_t rows);
int32_t qllm_topk_logits_batch(const float* values, uint32_t count,
                               size_t row_stride, uint32_t top_k, uint32_t rows,
                               float* output_values, uint32_t* output_indices,
                               void* workspace, size_t workspace_bytes,
                               void* stream);

/* replaces apply_presence_penalty (transformer_kernels.hpp:1292-1294). */
int32_t qllm_apply_presence_penalty(float* logits, const uint8_t* emitted,
                                    uint32_t count, float penalty,
                                    void* stream);

/* The same penalty for the `rows` rows of one verify step in one launch
 * (logits f32 [rows][row_stride], the first `count` of each row): row r is
 * penalised at the tokens marked in `emitted` and at drafts[0 .. r-1], the
 * tokens the rows before it carry (drafts: device, rows - 1 entries).  The
 * reference penalises row by row and marks draft r in a scratch copy of the
 * presence bytes in between (runtime/tools/dense_fp4_provider.cpp:
 * 11182-11202). */
int32_t qllm_apply_presence_penalty_rows(float* logits, size_t row_stride,
                                         const uint8_t* emitted,
                                         const uint32_t* drafts, uint32_t rows,
                                         uint32_t count, float penalty,
                                         void* stream);

/* emitted[tokens[i]] = 1 for up to 64 device-resident tokens (entries >= count
 * are ignored).  Replaces the per-token cudaMemset of the reference
 * (dense_fp4_provider.cpp:11261-11270, 8822-8847). */
int32_t qllm_mark_presence(uint8_t* emitted, const uint32_t* tokens,
                           uint32_t token_count, uint32_t count, void* stream);

/* ---- synthetic data (benchmarks and tests) ------------------------------------- */

/* Fill device memory from a counter-based generator (splitmix64 of seed and
 * element index), so a host restatement can rebuild the same bytes.
 * kind: 0 = uniform bytes, 1 = N(0,1) float, 2 = N(0,1) bf16,
 *       3 = log-normal(0, 0.5) binary16, 4 = N(0,1) binary16,
 *       5 = UE8M0 codes uniform in [124, 130]. */
int32_t qllm_fill_random(void* destination, size_t elements, uint32_t kind,
                         uint64_t seed, void* stream);

#ifdef __cplusplus
}
#endif
#endif
