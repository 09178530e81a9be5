// Exact-F16 paged KV cache: K/V store and decode attention.
// (attention kernel follows; this first part is the page store)
#include "common.hpp"

namespace qllm {
namespace {

// Per-layer page layout: K [page_tokens][kv_heads][head_dim] then
// V [page_tokens][kv_heads][head_dim], binary16
// (runtime/src/cuda/transformer_kernels.cu:6594-6606).
__global__ void f16_store_kernel(const float* key, const float* value,
                                 const void* const* page_table, uint32_t layer,
                                 uint32_t page_tokens,
                                 uint32_t first_cache_position,
                                 uint32_t kv_heads, uint32_t head_dim) {
  const uint32_t row = blockIdx.y;
  const uint32_t width = kv_heads * head_dim;
  const uint32_t item = blockIdx.x * blockDim.x + threadIdx.x;
  if (item >= width) return;
  const uint32_t position = first_cache_position + row;
  uint16_t* page = static_cast<uint16_t*>(
      const_cast<void*>(page_table[position / page_tokens]));
  const size_t page_values = static_cast<size_t>(page_tokens) * width;
  uint16_t* keys = page + static_cast<size_t>(layer) * 2u * page_values;
  const size_t target =
      static_cast<size_t>(position % page_tokens) * width + item;
  const size_t source = static_cast<size_t>(row) * width + item;
  keys[target] = static_cast<uint16_t>(f32_to_f16_bits(key[source]));
  keys[page_values + target] =
      static_cast<uint16_t>(f32_to_f16_bits(value[source]));
}

}  // namespace
}  // namespace qllm

using namespace qllm;

extern "C" int32_t qllm_store_kv_paged_f16_batch(
    const float* key, const float* value, const void* const* page_table,
    uint32_t full_attention_layer, uint32_t page_tokens,
    uint32_t first_cache_position, uint32_t rows, uint32_t kv_heads,
    uint32_t head_dim, void* stream) {
  if (!key || !value || !page_table || !page_tokens || !rows || !kv_heads ||
      !head_dim || first_cache_position > 0xffffffffu - (rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid F16 K/V store");
  const uint32_t width = kv_heads * head_dim;
  f16_store_kernel<<<dim3((width + 255u) / 256u, rows), 256, 0,
                     as_stream(stream)>>>(key, value, page_table,
                                          full_attention_layer, page_tokens,
                                          first_cache_position, kv_heads,
                                          head_dim);
  return launched("F16 K/V store");
}

extern "C" int32_t qllm_attention_paged_f16(
    const qllm_f16_attention_launch* launch) {
  (void)launch;
  return fail(QLLM_INTERNAL, "exact-F16 attention kernel is not built yet");
}
