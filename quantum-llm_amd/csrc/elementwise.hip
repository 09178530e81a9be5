// Small per-row kernels of the verify step: activation quantisation,
// embedding gather, RMSNorm, residual add, SiLU product, synthetic fills.
// Each replaces the reference launcher named beside its entry point.
#include "common.hpp"

#include <algorithm>
#include <cstdio>
#include <cstring>

namespace qllm {

namespace {
thread_local char last_error[256] = "";
}

int32_t fail(int32_t code, const char* message) {
  std::snprintf(last_error, sizeof(last_error), "%s", message);
  return code;
}

int32_t checked(hipError_t error, const char* what) {
  if (error == hipSuccess) return QLLM_OK;
  std::snprintf(last_error, sizeof(last_error), "%s: %s", what,
                hipGetErrorString(error));
  return QLLM_INTERNAL;
}

namespace {

// transformer_kernels.cu:912-946
__global__ __launch_bounds__(256) void quantize_q8_batch_kernel(
    const float* input, int8_t* output, float* scales, uint32_t columns,
    uint32_t padded_columns, bool bf16_input) {
  __shared__ float scratch[4];
  const uint32_t row = blockIdx.x;
  const float* source = input + static_cast<size_t>(row) * columns;
  int8_t* target = output + static_cast<size_t>(row) * padded_columns;
  float maximum = 0.0f;
  for (uint32_t column = threadIdx.x; column < columns; column += blockDim.x) {
    const float value = bf16_input ? bf16_round(source[column]) : source[column];
    maximum = fmaxf(maximum, fabsf(value));
  }
  maximum = block_max(maximum, scratch);
  const float scale = maximum > 0.0f ? maximum / 127.0f : 1.0f;
  if (threadIdx.x == 0) scales[row] = scale;
  for (uint32_t column = threadIdx.x; column < padded_columns;
       column += blockDim.x) {
    int quantized = 0;
    if (column < columns) {
      const float value =
          bf16_input ? bf16_round(source[column]) : source[column];
      quantized = __float2int_rn(__fdiv_rn(value, scale));
    }
    quantized = max(-127, min(127, quantized));
    target[column] = static_cast<int8_t>(quantized);
  }
}

// transformer_kernels.cu:948-959
__global__ __launch_bounds__(256) void convert_f32_to_bf16_batch_kernel(
    const float* input, uint16_t* output, uint32_t columns,
    uint32_t padded_columns) {
  const uint32_t row = blockIdx.x;
  const float* source = input + static_cast<size_t>(row) * columns;
  uint16_t* target = output + static_cast<size_t>(row) * padded_columns;
  for (uint32_t column = threadIdx.x; column < padded_columns;
       column += blockDim.x)
    target[column] = column < columns
                         ? static_cast<uint16_t>(f32_to_bf16_bits(source[column]))
                         : 0u;
}

// transformer_kernels.cu:801-821
__global__ __launch_bounds__(256) void fp4_embedding_batch_kernel(
    const uint8_t* weights, const uint8_t* scales, uint32_t scheme,
    const uint32_t* tokens, float* output, uint32_t columns,
    uint32_t padded_columns, uint32_t vocabulary) {
  const uint32_t request = blockIdx.x;
  const size_t token = tokens[request];
  if (token >= vocabulary) {
    // a token chosen on the device from logits without a finite maximum: no
    // row to read, the caller rejects the token when it sees it
    for (uint32_t column = threadIdx.x; column < columns; column += blockDim.x)
      output[static_cast<size_t>(request) * columns + column] = 0.0f;
    return;
  }
  const uint8_t* row_codes = weights + token * (padded_columns / 2u);
  for (uint32_t column = threadIdx.x; column < columns; column += blockDim.x) {
    const uint8_t byte = row_codes[column / 2u];
    const uint32_t code = (column & 1u) ? byte >> 4 : byte & 0x0fu;
    const uint32_t index = code & 7u;
    const float twice = index <= 4u ? static_cast<float>(index)
                        : index == 5u ? 6.0f
                        : index == 6u ? 8.0f
                                      : 12.0f;
    float scale;
    if (scheme == QLLM_SCALE_F16_BLOCK16)
      scale = f16_bits_to_f32(reinterpret_cast<const uint16_t*>(
          scales)[token * (padded_columns / 16u) + column / 16u]);
    else
      scale = ue8m0_to_f32(scales[token * (padded_columns / 32u) + column / 32u]);
    const float value = twice * 0.5f * scale;
    output[static_cast<size_t>(request) * columns + column] =
        (code & 8u) ? -value : value;
  }
}

// Same values as fp4_embedding_batch_kernel, eight columns (one dword of
// codes, half a scale block) per thread and the row spread over blockIdx.y,
// so that a one-token lookup is not a single workgroup's serial loop.
__global__ __launch_bounds__(256) void fp4_embedding_batch_wide_kernel(
    const uint8_t* weights, const uint8_t* scales, uint32_t scheme,
    const uint32_t* tokens, float* output, uint32_t columns,
    uint32_t padded_columns, uint32_t vocabulary) {
  const uint32_t request = blockIdx.x;
  const uint32_t column = (blockIdx.y * blockDim.x + threadIdx.x) * 8u;
  if (column >= columns) return;
  const size_t token = tokens[request];
  if (token >= vocabulary) {   // see fp4_embedding_batch_kernel
    float4* destination = reinterpret_cast<float4*>(
        output + static_cast<size_t>(request) * columns + column);
    destination[0] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    destination[1] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    return;
  }
  const uint32_t codes = *reinterpret_cast<const uint32_t*>(
      weights + token * (padded_columns / 2u) + column / 2u);
  float scale;
  if (scheme == QLLM_SCALE_F16_BLOCK16)
    scale = f16_bits_to_f32(reinterpret_cast<const uint16_t*>(
        scales)[token * (padded_columns / 16u) + column / 16u]);
  else
    scale = ue8m0_to_f32(scales[token * (padded_columns / 32u) + column / 32u]);
  float values[8];
#pragma unroll
  for (uint32_t i = 0; i < 8u; ++i) {
    const uint32_t code = (codes >> (4u * i)) & 0x0fu;
    const uint32_t index = code & 7u;
    const float twice = index <= 4u ? static_cast<float>(index)
                        : index == 5u ? 6.0f
                        : index == 6u ? 8.0f
                                      : 12.0f;
    const float value = twice * 0.5f * scale;
    values[i] = (code & 8u) ? -value : value;
  }
  float4* destination = reinterpret_cast<float4*>(
      output + static_cast<size_t>(request) * columns + column);
  destination[0] = make_float4(values[0], values[1], values[2], values[3]);
  destination[1] = make_float4(values[4], values[5], values[6], values[7]);
}

// transformer_kernels.cu:2469-2521
__global__ __launch_bounds__(256) void rms_norm_batch_kernel(
    const float* input, const float* weight, float* output_f32,
    uint16_t* output_bf16, uint32_t bf16_padded_columns, uint32_t elements,
    float epsilon, bool zero_centered) {
  __shared__ float scratch[4];
  const uint32_t row = blockIdx.x;
  const float* x = input + static_cast<size_t>(row) * elements;
  float square = 0.0f;
  for (uint32_t index = threadIdx.x; index < elements; index += blockDim.x)
    square = fmaf(x[index], x[index], square);
  square = block_sum(square, scratch);
  const float inverse =
      rsqrtf(square / static_cast<float>(elements) + epsilon);
  const uint32_t limit = output_bf16 && bf16_padded_columns > elements
                             ? bf16_padded_columns
                             : elements;
  for (uint32_t index = threadIdx.x; index < limit; index += blockDim.x) {
    float value = 0.0f;
    if (index < elements) {
      float factor = 1.0f;
      if (weight) factor = zero_centered ? 1.0f + weight[index] : weight[index];
      value = x[index] * inverse * factor;
      if (output_f32)
        output_f32[static_cast<size_t>(row) * elements + index] = value;
    }
    if (output_bf16)
      output_bf16[static_cast<size_t>(row) * bf16_padded_columns + index] =
          static_cast<uint16_t>(f32_to_bf16_bits(value));
  }
}

// Same operation for rows of up to 16384 elements (a multiple of 4): up to
// 1024 threads per row, the row is read once with 16-byte loads and kept in
// registers between the reduction and the scaling.
// One row of up to 16 * blockDim.x elements (a multiple of four):
// `out_f32` / `out_bf16` point at the row's outputs (either may be null) and
// bf16 columns [elements, bf16_columns) are zeroed.
// With `partial_count` > 0 the row normalised is input_row + partials[0] +
// partials[1] + ... (added in that order; partial p of the row lies
// `partial_stride` floats after partial p - 1) and that sum is also written
// back to `sum_out`.
// Columns 4 * vector .. + 3 of a row-major FP4 row as F32: the values
// fp4_embedding_batch_kernel gives (twice(code) * 0.5 * scale, sign applied
// last).
__device__ __forceinline__ float4 fp4_row_vector(const uint8_t* codes_row,
                                                 const uint8_t* scales_row,
                                                 uint32_t scheme, uint32_t vector) {
  const uint32_t column = vector * 4u;
  const uint32_t codes =
      *reinterpret_cast<const uint16_t*>(codes_row + column / 2u);
  const float scale =
      scheme == QLLM_SCALE_F16_BLOCK16
          ? f16_bits_to_f32(reinterpret_cast<const uint16_t*>(scales_row)[column / 16u])
          : ue8m0_to_f32(scales_row[column / 32u]);
  float values[4];
#pragma unroll
  for (uint32_t i = 0; i < 4u; ++i) {
    const uint32_t code = (codes >> (4u * i)) & 0x0fu;
    const uint32_t index = code & 7u;
    const float twice = index <= 4u ? static_cast<float>(index)
                        : index == 5u ? 6.0f
                        : index == 6u ? 8.0f
                                      : 12.0f;
    const float value = twice * 0.5f * scale;
    values[i] = (code & 8u) ? -value : value;
  }
  return make_float4(values[0], values[1], values[2], values[3]);
}

// four values -> four Q8 codes: clamp(rn(value / scale), -127, 127)
// (transformer_kernels.cu:912-946), packed low byte first
__device__ __forceinline__ uint32_t q8_pack4(float4 value, float scale) {
  const auto code = [scale](float x) {
    const int rounded = __float2int_rn(__fdiv_rn(x, scale));
    return static_cast<uint32_t>(max(-127, min(127, rounded))) & 0xffu;
  };
  return code(value.x) | (code(value.y) << 8) | (code(value.z) << 16) |
         (code(value.w) << 24);
}

// Per-row Q8 of rows of up to 5 * 4096 values: the row is fetched once and
// stays in registers between the maximum and the codes.  columns % 4 == 0.
__global__ __launch_bounds__(1024) void quantize_q8_wide_kernel(
    const float* input, int8_t* output, float* scales, uint32_t columns,
    uint32_t padded_columns) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  const float4* x = reinterpret_cast<const float4*>(input + row * columns);
  const uint32_t vectors = columns / 4u;
  float4 values[5];
  float maximum = 0.0f;
#pragma unroll
  for (int slot = 0; slot < 5; ++slot) {
    const uint32_t index = slot * 1024u + threadIdx.x;
    values[slot] = index < vectors ? x[index] : make_float4(0.f, 0.f, 0.f, 0.f);
    maximum = fmaxf(maximum, fmaxf(fmaxf(fabsf(values[slot].x), fabsf(values[slot].y)),
                                   fmaxf(fabsf(values[slot].z), fabsf(values[slot].w))));
  }
  maximum = block_max(maximum, scratch);
  const float scale = maximum > 0.0f ? maximum / 127.0f : 1.0f;
  if (threadIdx.x == 0) scales[row] = scale;
  uint32_t* target = reinterpret_cast<uint32_t*>(output + row * padded_columns);
#pragma unroll
  for (int slot = 0; slot < 5; ++slot) {
    const uint32_t index = slot * 1024u + threadIdx.x;
    if (index < vectors) target[index] = q8_pack4(values[slot], scale);
  }
  for (uint32_t index = vectors + threadIdx.x; index < padded_columns / 4u;
       index += 1024u)
    target[index] = 0u;
}

__device__ __forceinline__ void rms_norm_row_wide(
    const float* input_row, const float* weight, float* out_f32,
    uint16_t* out_bf16, uint32_t bf16_columns, uint32_t elements,
    float epsilon, bool zero_centered, float* scratch,
    const float* partial_row = nullptr, uint32_t partial_count = 0u,
    size_t partial_stride = 0u, float* sum_out = nullptr,
    int8_t* out_q8 = nullptr, float* out_q8_scale = nullptr,
    const uint8_t* fp4_codes_row = nullptr, const uint8_t* fp4_scales_row = nullptr,
    uint32_t fp4_scheme = 0u) {
  // with fp4_codes_row the row is an FP4 embedding row, decoded on the way in
  const float4* x = reinterpret_cast<const float4*>(input_row);
  const uint32_t vectors = elements / 4u;
  // the row and its weights are fetched together, before the reduction
  float4 values[4];
  float4 factors[4];
  float square = 0.0f;
#pragma unroll
  for (int slot = 0; slot < 4; ++slot) {
    const uint32_t index = slot * blockDim.x + threadIdx.x;
    values[slot] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (index < vectors)
      values[slot] = fp4_codes_row ? fp4_row_vector(fp4_codes_row, fp4_scales_row,
                                                    fp4_scheme, index)
                     : input_row   ? x[index]
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
    factors[slot] = make_float4(1.f, 1.f, 1.f, 1.f);
    if (weight && index < vectors)
      factors[slot] = reinterpret_cast<const float4*>(weight)[index];
  }
  if (partial_count) {
#pragma unroll
    for (int slot = 0; slot < 4; ++slot) {
      const uint32_t index = slot * blockDim.x + threadIdx.x;
      if (index >= vectors) continue;
      // the first four partials are requested together (one round trip), then
      // added in index order like the rest
      float4 early[4];
#pragma unroll
      for (uint32_t p = 0; p < 4u; ++p)
        if (p < partial_count)
          early[p] =
              reinterpret_cast<const float4*>(partial_row + p * partial_stride)[index];
#pragma unroll
      for (uint32_t p = 0; p < 4u; ++p)
        if (p < partial_count) {
          values[slot].x += early[p].x; values[slot].y += early[p].y;
          values[slot].z += early[p].z; values[slot].w += early[p].w;
        }
      for (uint32_t p = 4u; p < partial_count; ++p) {
        const float4 part =
            reinterpret_cast<const float4*>(partial_row + p * partial_stride)[index];
        values[slot].x += part.x; values[slot].y += part.y;
        values[slot].z += part.z; values[slot].w += part.w;
      }
      reinterpret_cast<float4*>(sum_out)[index] = values[slot];
    }
  }
#pragma unroll
  for (int slot = 0; slot < 4; ++slot) {
    square = fmaf(values[slot].x, values[slot].x, square);
    square = fmaf(values[slot].y, values[slot].y, square);
    square = fmaf(values[slot].z, values[slot].z, square);
    square = fmaf(values[slot].w, values[slot].w, square);
  }
  square = block_sum(square, scratch);
  const float inverse =
      rsqrtf(square / static_cast<float>(elements) + epsilon);
#pragma unroll
  for (int slot = 0; slot < 4; ++slot) {
    const uint32_t index = slot * blockDim.x + threadIdx.x;
    if (index >= vectors) continue;
    float4 factor = factors[slot];
    if (weight && zero_centered) {
      factor.x += 1.0f; factor.y += 1.0f; factor.z += 1.0f; factor.w += 1.0f;
    }
    float4 result;
    result.x = values[slot].x * inverse * factor.x;
    result.y = values[slot].y * inverse * factor.y;
    result.z = values[slot].z * inverse * factor.z;
    result.w = values[slot].w * inverse * factor.w;
    if (out_f32) reinterpret_cast<float4*>(out_f32)[index] = result;
    if (out_bf16) {
      uint2 packed;
      packed.x = f32_to_bf16_bits(result.x) | (f32_to_bf16_bits(result.y) << 16);
      packed.y = f32_to_bf16_bits(result.z) | (f32_to_bf16_bits(result.w) << 16);
      reinterpret_cast<uint2*>(out_bf16)[index] = packed;
    }
    values[slot] = result;
  }
  if (out_q8) {
    // the row quantised as quantize_q8_batch_kernel quantises the F32 norm
    // output (same operations on the same values)
    float maximum = 0.0f;
#pragma unroll
    for (int slot = 0; slot < 4; ++slot) {
      if (slot * blockDim.x + threadIdx.x >= vectors) continue;
      maximum = fmaxf(maximum, fmaxf(fmaxf(fabsf(values[slot].x), fabsf(values[slot].y)),
                                     fmaxf(fabsf(values[slot].z), fabsf(values[slot].w))));
    }
    maximum = block_max(maximum, scratch);
    const float scale = maximum > 0.0f ? maximum / 127.0f : 1.0f;
    if (threadIdx.x == 0) *out_q8_scale = scale;
#pragma unroll
    for (int slot = 0; slot < 4; ++slot) {
      const uint32_t index = slot * blockDim.x + threadIdx.x;
      if (index >= vectors) continue;
      reinterpret_cast<uint32_t*>(out_q8)[index] = q8_pack4(values[slot], scale);
    }
  }
  if (out_bf16)
    for (uint32_t index = elements + threadIdx.x; index < bf16_columns;
         index += blockDim.x)
      out_bf16[index] = 0u;
}

__global__ __launch_bounds__(1024) void rms_norm_batch_wide_kernel(
    const float* input, const float* weight, float* output_f32,
    uint16_t* output_bf16, uint32_t bf16_padded_columns, uint32_t elements,
    float epsilon, bool zero_centered) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  rms_norm_row_wide(
      input + row * elements, weight,
      output_f32 ? output_f32 + row * elements : nullptr,
      output_bf16 ? output_bf16 + row * bf16_padded_columns : nullptr,
      bf16_padded_columns, elements, epsilon, zero_centered, scratch);
}

// RMSNorm of a row straight into its per-row Q8 form (normalize_rows followed
// by quantize_rows, dense_fp4_provider.cpp:5740-5778, 5983-5992, in one launch).
__global__ __launch_bounds__(1024) void rms_norm_q8_kernel(
    const float* input, const float* weight, int8_t* output_q8, float* scales,
    uint32_t elements, float epsilon, bool zero_centered) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  rms_norm_row_wide(input + row * elements, weight, nullptr, nullptr, 0u, elements,
                    epsilon, zero_centered, scratch, nullptr, 0u, 0u, nullptr,
                    output_q8 + row * elements, scales + row);
}

// The same on a row that is first completed from K-split partial sums
// (rms_norm_residual_kernel below, with the Q8 output of rms_norm_q8_kernel).
__global__ __launch_bounds__(1024) void rms_norm_residual_q8_kernel(
    const float* residual, float* sum, const float* partials,
    uint32_t partial_count, const float* weight, int8_t* output_q8, float* scales,
    uint32_t elements, float epsilon, bool zero_centered) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  rms_norm_row_wide(residual ? residual + row * elements : nullptr, weight, nullptr,
                    nullptr, 0u, elements, epsilon, zero_centered, scratch,
                    partials + row * elements, partial_count,
                    static_cast<size_t>(gridDim.x) * elements, sum + row * elements,
                    output_q8 + row * elements, scales + row);
}

// sum[r] = residual[r] + partials[0][r] + ... + partials[count-1][r] (from zero
// without a residual), then its RMSNorm in bf16: the residual add of a
// projection whose K was cut over workgroups (qllm_fp4_gemm_bf16_partial)
// folded into the norm that follows it.  `sum` may be `residual`.
__global__ __launch_bounds__(1024) void rms_norm_residual_kernel(
    const float* residual, float* sum, const float* partials,
    uint32_t partial_count, const float* weight, uint16_t* output_bf16,
    uint32_t elements, float epsilon, bool zero_centered) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  rms_norm_row_wide(residual ? residual + row * elements : nullptr, weight, nullptr,
                    output_bf16 + row * elements, elements, elements, epsilon,
                    zero_centered, scratch, partials + row * elements,
                    partial_count, static_cast<size_t>(gridDim.x) * elements,
                    sum + row * elements);
}

// Row r of the output is [RMSNorm(first[r]) | RMSNorm(second[r])] in bf16:
// blockIdx.y picks the half.
__global__ __launch_bounds__(1024) void rms_norm_concat_kernel(
    const float* first, const float* first_weight, const float* second,
    const float* second_weight, uint16_t* output_bf16, uint32_t elements,
    float epsilon, bool zero_centered) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  const bool second_half = blockIdx.y != 0u;
  rms_norm_row_wide(
      (second_half ? second : first) + row * elements,
      second_half ? second_weight : first_weight, nullptr,
      output_bf16 + row * 2u * elements + (second_half ? elements : 0u),
      elements, elements, epsilon, zero_centered, scratch);
}

// The proposer's input: row r of the output is [RMSNorm(embedding of
// tokens[r]) | RMSNorm(second[r])] in bf16 - the embedding lookup
// (fp4_embedding_batch_kernel) folded into the first half's norm.  A token
// outside the vocabulary gives a row of zeros, as the lookup does.
__global__ __launch_bounds__(1024) void rms_norm_concat_embedding_kernel(
    const uint8_t* codes, const uint8_t* scales, uint32_t scheme,
    uint32_t padded_columns, uint32_t vocabulary, const uint32_t* tokens,
    const float* first_weight, const float* second, const float* second_weight,
    uint16_t* output_bf16, uint32_t elements, float epsilon, bool zero_centered,
    uint8_t* presence) {
  __shared__ float scratch[16];
  const size_t row = blockIdx.x;
  uint16_t* out = output_bf16 + row * 2u * elements;
  if (blockIdx.y != 0u) {
    rms_norm_row_wide(second + row * elements, second_weight, nullptr,
                      out + elements, elements, elements, epsilon, zero_centered,
                      scratch);
    return;
  }
  const size_t token = tokens[row];
  // (mark_presence_kernel's store, for callers whose batch is emitted tokens)
  if (presence && threadIdx.x == 0u && token < vocabulary) presence[token] = 1u;
  if (token >= vocabulary) {
    for (uint32_t index = threadIdx.x; index < elements; index += blockDim.x)
      out[index] = 0u;
    return;
  }
  const size_t scale_row_bytes = scheme == QLLM_SCALE_F16_BLOCK16
                                     ? padded_columns / 8u
                                     : padded_columns / 32u;
  rms_norm_row_wide(nullptr, first_weight, nullptr, out, elements, elements, epsilon,
                    zero_centered, scratch, nullptr, 0u, 0u, nullptr, nullptr, nullptr,
                    codes + token * (padded_columns / 2u),
                    scales + token * scale_row_bytes, scheme);
}

// transformer_kernels.cu:2522-2528
__global__ void add_kernel(float* destination, const float* source,
                           uint32_t count, bool bf16_output) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) {
    const float value = destination[i] + source[i];
    destination[i] = bf16_output ? bf16_round(value) : value;
  }
}

// transformer_kernels.cu:2774-2783
__global__ void silu_product_kernel(const float* gate, const float* up,
                                    float* output, uint32_t count,
                                    bool bf16_activations) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) {
    float activated = gate[i] / (1.0f + expf(-gate[i]));
    if (bf16_activations) activated = bf16_round(activated);
    const float value = activated * up[i];
    output[i] = bf16_activations ? bf16_round(value) : value;
  }
}

__device__ __forceinline__ float uniform_open(uint64_t bits) {
  return (static_cast<float>(bits >> 40) + 0.5f) * (1.0f / 16777216.0f);
}

__device__ __forceinline__ float normal_from(uint64_t seed, uint64_t index) {
  const float u1 = uniform_open(mix64(seed, 2u * index));
  const float u2 = uniform_open(mix64(seed, 2u * index + 1u));
  return sqrtf(-2.0f * logf(u1)) * cosf(6.2831853f * u2);
}

__global__ void fill_random_kernel(void* destination, size_t elements,
                                   uint32_t kind, uint64_t seed) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t index = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
       index < elements; index += stride) {
    switch (kind) {
      case 0:
        static_cast<uint8_t*>(destination)[index] =
            static_cast<uint8_t>(mix64(seed, index) >> 24);
        break;
      case 1:
        static_cast<float*>(destination)[index] = normal_from(seed, index);
        break;
      case 2:
        static_cast<uint16_t*>(destination)[index] =
            static_cast<uint16_t>(f32_to_bf16_bits(normal_from(seed, index)));
        break;
      case 3:
        static_cast<uint16_t*>(destination)[index] = static_cast<uint16_t>(
            f32_to_f16_bits(expf(0.5f * normal_from(seed, index))));
        break;
      case 4:
        static_cast<uint16_t*>(destination)[index] =
            static_cast<uint16_t>(f32_to_f16_bits(normal_from(seed, index)));
        break;
      default:
        static_cast<uint8_t*>(destination)[index] =
            static_cast<uint8_t>(124u + (mix64(seed, index) >> 32) % 7u);
        break;
    }
  }
}

}  // namespace
}  // namespace qllm

using namespace qllm;

extern "C" const char* qllm_last_error(void) { return last_error; }

extern "C" const char* qllm_version(void) { return "qllm-hip gfx950 1"; }

extern "C" int32_t qllm_quantize_q8_batch(const float* input, int8_t* output,
                                          float* scales, uint32_t rows,
                                          uint32_t columns,
                                          uint32_t padded_columns,
                                          int32_t bf16_input, void* stream) {
  if (!input || !output || !scales || !rows || !columns ||
      padded_columns < columns)
    return fail(QLLM_INVALID_ARGUMENT, "invalid Q8 batch quantization");
  const bool wide =
      !bf16_input && columns % 4u == 0u && padded_columns % 4u == 0u &&
      columns <= 5u * 4096u &&
      ((reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(output)) &
       15u) == 0u;
  if (wide)
    quantize_q8_wide_kernel<<<rows, 1024, 0, as_stream(stream)>>>(
        input, output, scales, columns, padded_columns);
  else
    quantize_q8_batch_kernel<<<rows, 256, 0, as_stream(stream)>>>(
        input, output, scales, columns, padded_columns, bf16_input != 0);
  return launched("quantize Q8 batch");
}

extern "C" int32_t qllm_rms_norm_q8_batch(const float* input, const float* weight,
                                          int8_t* output_q8, float* scales,
                                          uint32_t rows, uint32_t elements,
                                          float epsilon, int32_t zero_centered,
                                          void* stream) {
  const auto aligned = [](const void* pointer) {
    return reinterpret_cast<uintptr_t>(pointer) % 16u == 0u;
  };
  if (!input || !output_q8 || !scales || !rows || rows > 65535u || !elements ||
      elements % 4u != 0u || elements > 16384u || !(epsilon > 0.0f) ||
      !aligned(input) || !aligned(output_q8) || (weight && !aligned(weight)))
    return fail(QLLM_INVALID_ARGUMENT, "invalid Q8 RMSNorm");
  rms_norm_q8_kernel<<<rows, 1024, 0, as_stream(stream)>>>(
      input, weight, output_q8, scales, elements, epsilon, zero_centered != 0);
  return launched("Q8 RMSNorm");
}

extern "C" int32_t qllm_rms_norm_partials_q8_batch(
    const float* residual, float* sum, const float* partials,
    uint32_t partial_count, const float* weight, int8_t* output_q8, float* scales,
    uint32_t rows, uint32_t elements, float epsilon, int32_t zero_centered,
    void* stream) {
  const auto aligned = [](const void* pointer) {
    return reinterpret_cast<uintptr_t>(pointer) % 16u == 0u;
  };
  if (!sum || !partials || !partial_count || partial_count > 16u || !output_q8 ||
      !scales || !rows || rows > 65535u || !elements || elements % 4u != 0u ||
      elements > 16384u || !(epsilon > 0.0f) || !aligned(residual) || !aligned(sum) ||
      !aligned(partials) || !aligned(output_q8) || (weight && !aligned(weight)))
    return fail(QLLM_INVALID_ARGUMENT, "invalid Q8 RMSNorm of partial sums");
  rms_norm_residual_q8_kernel<<<rows, 1024, 0, as_stream(stream)>>>(
      residual, sum, partials, partial_count, weight, output_q8, scales, elements,
      epsilon, zero_centered != 0);
  return launched("Q8 RMSNorm of partial sums");
}

extern "C" int32_t qllm_convert_f32_to_bf16_batch(
    const float* input, void* output, size_t output_bytes, uint32_t rows,
    uint32_t columns, uint32_t padded_columns, void* stream) {
  if (!input || !output || !rows || !columns || padded_columns < columns ||
      output_bytes < static_cast<size_t>(rows) * padded_columns * 2u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid F32 to BF16 conversion");
  convert_f32_to_bf16_batch_kernel<<<rows, 256, 0, as_stream(stream)>>>(
      input, static_cast<uint16_t*>(output), columns, padded_columns);
  return launched("convert F32 to BF16");
}

extern "C" int32_t qllm_fp4_embedding_batch(const qllm_fp4_matrix* matrix,
                                            const uint32_t* tokens,
                                            float* output, uint32_t batch,
                                            void* stream) {
  if (!matrix || !matrix->weights || !matrix->scales || !matrix->rows ||
      !matrix->columns || matrix->padded_columns < matrix->columns ||
      matrix->padded_columns % 32u || matrix->scale_scheme > 1u ||
      matrix->layout != QLLM_LAYOUT_ROW_MAJOR || !tokens ||
      !output || !batch)
    return fail(QLLM_INVALID_ARGUMENT, "invalid FP4 embedding batch");
  const bool wide =
      matrix->columns % 8u == 0u && matrix->padded_columns % 8u == 0u &&
      ((reinterpret_cast<uintptr_t>(matrix->weights) & 3u) |
       (reinterpret_cast<uintptr_t>(output) & 15u)) == 0u;
  if (wide)
    fp4_embedding_batch_wide_kernel<<<dim3(batch, (matrix->columns / 8u + 255u) / 256u),
                                      256, 0, as_stream(stream)>>>(
        matrix->weights, static_cast<const uint8_t*>(matrix->scales),
        matrix->scale_scheme, tokens, output, matrix->columns,
        matrix->padded_columns, matrix->rows);
  else
    fp4_embedding_batch_kernel<<<batch, 256, 0, as_stream(stream)>>>(
        matrix->weights, static_cast<const uint8_t*>(matrix->scales),
        matrix->scale_scheme, tokens, output, matrix->columns,
        matrix->padded_columns, matrix->rows);
  return launched("FP4 embedding batch");
}

extern "C" int32_t qllm_rms_norm_batch(const float* input, const float* weight,
                                       float* output_f32, void* output_bf16,
                                       uint32_t bf16_padded_columns,
                                       uint32_t rows, uint32_t elements,
                                       float epsilon, int32_t zero_centered,
                                       void* stream) {
  if (!input || (!output_f32 && !output_bf16) || !rows || !elements ||
      !(epsilon > 0.0f) ||
      (output_bf16 && bf16_padded_columns < elements))
    return fail(QLLM_INVALID_ARGUMENT, "invalid RMSNorm batch");
  const bool aligned =
      ((reinterpret_cast<uintptr_t>(input) |
        reinterpret_cast<uintptr_t>(weight) |
        reinterpret_cast<uintptr_t>(output_f32)) & 15u) == 0u &&
      (reinterpret_cast<uintptr_t>(output_bf16) & 7u) == 0u;
  if (elements % 4u == 0u && elements <= 16384u && aligned &&
      bf16_padded_columns % 4u == 0u)
    rms_norm_batch_wide_kernel<<<rows, 1024, 0, as_stream(stream)>>>(
        input, weight, output_f32, static_cast<uint16_t*>(output_bf16),
        bf16_padded_columns, elements, epsilon, zero_centered != 0);
  else
    rms_norm_batch_kernel<<<rows, 256, 0, as_stream(stream)>>>(
        input, weight, output_f32, static_cast<uint16_t*>(output_bf16),
        bf16_padded_columns, elements, epsilon, zero_centered != 0);
  return launched("RMSNorm batch");
}

extern "C" int32_t qllm_rms_norm_residual_batch(
    float* hidden, const float* partials, uint32_t partial_count,
    const float* weight, void* output_bf16, uint32_t rows, uint32_t elements,
    float epsilon, int32_t zero_centered, void* stream) {
  const auto aligned = [](const void* pointer) {
    return reinterpret_cast<uintptr_t>(pointer) % 16u == 0u;
  };
  if (!hidden || !partials || !partial_count || partial_count > 16u ||
      !output_bf16 || !rows || rows > 65535u || !elements ||
      elements % 4u != 0u || elements > 16384u || !aligned(hidden) ||
      !aligned(partials) || !aligned(output_bf16) || (weight && !aligned(weight)))
    return fail(QLLM_INVALID_ARGUMENT, "invalid residual RMSNorm");
  // (measured on rows of 5120: 320 threads, four float4 each, take 6.0 us
  // against 4.75 us with 1024: one CU's few waves wait longer for the row)
  rms_norm_residual_kernel<<<rows, 1024, 0, as_stream(stream)>>>(
      hidden, hidden, partials, partial_count, weight,
      static_cast<uint16_t*>(output_bf16), elements, epsilon, zero_centered != 0);
  return launched("residual RMSNorm");
}

extern "C" int32_t qllm_rms_norm_partials_batch(
    const float* residual, float* sum, const float* partials,
    uint32_t partial_count, const float* weight, void* output_bf16, uint32_t rows,
    uint32_t elements, float epsilon, int32_t zero_centered, void* stream) {
  const auto aligned = [](const void* pointer) {
    return reinterpret_cast<uintptr_t>(pointer) % 16u == 0u;
  };
  if (!sum || !partials || !partial_count || partial_count > 16u ||
      !output_bf16 || !rows || rows > 65535u || !elements ||
      elements % 4u != 0u || elements > 16384u || !aligned(residual) ||
      !aligned(sum) || !aligned(partials) || !aligned(output_bf16) ||
      (weight && !aligned(weight)))
    return fail(QLLM_INVALID_ARGUMENT, "invalid RMSNorm of partial sums");
  rms_norm_residual_kernel<<<rows, 1024, 0, as_stream(stream)>>>(
      residual, sum, partials, partial_count, weight,
      static_cast<uint16_t*>(output_bf16), elements, epsilon, zero_centered != 0);
  return launched("RMSNorm of partial sums");
}

extern "C" int32_t qllm_rms_norm_concat_batch(
    const float* first, const float* first_weight, const float* second,
    const float* second_weight, void* output_bf16, uint32_t rows,
    uint32_t elements, float epsilon, int32_t zero_centered, void* stream) {
  if (!first || !second || !output_bf16 || !rows || !elements ||
      elements % 4u || elements > 16384u || !(epsilon > 0.0f) ||
      ((reinterpret_cast<uintptr_t>(first) |
        reinterpret_cast<uintptr_t>(first_weight) |
        reinterpret_cast<uintptr_t>(second) |
        reinterpret_cast<uintptr_t>(second_weight)) & 15u) ||
      (reinterpret_cast<uintptr_t>(output_bf16) & 7u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid RMSNorm concat batch");
  rms_norm_concat_kernel<<<dim3(rows, 2u), 1024, 0, as_stream(stream)>>>(
      first, first_weight, second, second_weight,
      static_cast<uint16_t*>(output_bf16), elements, epsilon,
      zero_centered != 0);
  return launched("RMSNorm concat batch");
}

extern "C" int32_t qllm_rms_norm_concat_embedding_batch(
    const qllm_fp4_matrix* embedding, const uint32_t* tokens,
    const float* first_weight, const float* second, const float* second_weight,
    void* output_bf16, uint32_t rows, float epsilon, int32_t zero_centered,
    uint8_t* presence, void* stream) {
  if (!embedding || !embedding->weights || !embedding->scales || !embedding->rows ||
      embedding->layout != QLLM_LAYOUT_ROW_MAJOR || embedding->scale_scheme > 1u ||
      embedding->padded_columns < embedding->columns ||
      embedding->padded_columns % 32u || !tokens || !second || !output_bf16 ||
      !rows || !embedding->columns || embedding->columns % 4u ||
      embedding->columns > 16384u || !(epsilon > 0.0f) ||
      ((reinterpret_cast<uintptr_t>(first_weight) |
        reinterpret_cast<uintptr_t>(second) |
        reinterpret_cast<uintptr_t>(second_weight)) & 15u) ||
      (reinterpret_cast<uintptr_t>(embedding->weights) & 1u) ||
      (reinterpret_cast<uintptr_t>(embedding->scales) & 1u) ||
      (reinterpret_cast<uintptr_t>(output_bf16) & 7u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid RMSNorm concat of an embedding batch");
  rms_norm_concat_embedding_kernel<<<dim3(rows, 2u), 1024, 0, as_stream(stream)>>>(
      embedding->weights, static_cast<const uint8_t*>(embedding->scales),
      embedding->scale_scheme, embedding->padded_columns, embedding->rows, tokens,
      first_weight, second, second_weight, static_cast<uint16_t*>(output_bf16),
      embedding->columns, epsilon, zero_centered != 0, presence);
  return launched("RMSNorm concat of an embedding batch");
}

extern "C" int32_t qllm_add_in_place(float* destination, const float* source,
                                     uint32_t elements, int32_t bf16_output,
                                     void* stream) {
  if (!destination || !source || !elements)
    return fail(QLLM_INVALID_ARGUMENT, "invalid residual add");
  add_kernel<<<(elements + 255u) / 256u, 256, 0, as_stream(stream)>>>(
      destination, source, elements, bf16_output != 0);
  return launched("residual add");
}

extern "C" int32_t qllm_silu_product(const float* gate, const float* up,
                                     float* output, uint32_t elements,
                                     int32_t bf16_activations, void* stream) {
  if (!gate || !up || !output || !elements)
    return fail(QLLM_INVALID_ARGUMENT, "invalid SiLU product");
  silu_product_kernel<<<(elements + 255u) / 256u, 256, 0, as_stream(stream)>>>(
      gate, up, output, elements, bf16_activations != 0);
  return launched("SiLU product");
}

extern "C" int32_t qllm_fill_random(void* destination, size_t elements,
                                    uint32_t kind, uint64_t seed,
                                    void* stream) {
  if (!destination || !elements || kind > 5u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid random fill");
  const size_t blocks = (elements + 255u) / 256u;
  const unsigned grid =
      static_cast<unsigned>(blocks < 65536u ? blocks : 65536u);
  fill_random_kernel<<<grid, 256, 0, as_stream(stream)>>>(destination, elements,
                                                          kind, seed);
  return launched("random fill");
}
