// Shared device helpers and host-side status plumbing for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstddef>
#include <cstdint>

#include "qllm_kernels.h"

namespace qllm {

// Records `message` as the calling thread's last error and returns `code`.
int32_t fail(int32_t code, const char* message);
// Maps a HIP error (after a launch or runtime call) to a status code.
int32_t checked(hipError_t error, const char* what);
inline int32_t launched(const char* what) {
  return checked(hipPeekAtLastError(), what);
}
inline hipStream_t as_stream(void* stream) {
  return static_cast<hipStream_t>(stream);
}

constexpr int kWave = 64;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(2))) int i32x2;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}

// Round-to-nearest-even F32 -> BF16 bit pattern; Inf/NaN keep their class.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float value) {
  uint32_t bits = __float_as_uint(value);
  if ((bits & 0x7f800000u) == 0x7f800000u) {
    uint32_t high = bits >> 16;
    if (bits & 0x007fffffu) high |= 0x40u;
    return high;
  }
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return bits >> 16;
}

__device__ __forceinline__ float bf16_round(float value) {
  return bf16_bits_to_f32(f32_to_bf16_bits(value));
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits16) {
  const _Float16 half = __builtin_bit_cast(_Float16, static_cast<unsigned short>(bits16));
  return static_cast<float>(half);
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float value) {
  const _Float16 half = static_cast<_Float16>(value);  // v_cvt_f16_f32, RN-even
  return __builtin_bit_cast(unsigned short, half);
}

// UE8M0 scale byte -> float; code 0 is 2^-127 (a subnormal).
__device__ __forceinline__ float ue8m0_to_f32(uint32_t code) {
  return __uint_as_float(code == 0u ? 0x00400000u : code << 23);
}

// Two E2M1 codes (byte `Sel` of `packed`) -> two bf16 values, exact.
template <int Sel>
__device__ __forceinline__ bf16x2 fp4x2_to_bf16(uint32_t packed, float scale) {
  return __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(packed, scale, Sel);
}

__device__ __forceinline__ float wave_sum(float value) {
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1)
    value += __shfl_xor(value, offset, kWave);
  return value;
}

__device__ __forceinline__ float wave_max(float value) {
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1)
    value = fmaxf(value, __shfl_xor(value, offset, kWave));
  return value;
}

// Block-wide sum / max over up to 1024 threads using one LDS word per wave.
// `scratch` must hold at least blockDim.x/64 floats; all threads call.
__device__ __forceinline__ float block_sum(float value, float* scratch) {
  value = wave_sum(value);
  const int wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[wave] = value;
  __syncthreads();
  float total = 0.0f;
  for (int index = 0; index < waves; ++index) total += scratch[index];
  return total;
}

__device__ __forceinline__ float block_max(float value, float* scratch) {
  value = wave_max(value);
  const int wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[wave] = value;
  __syncthreads();
  float total = scratch[0];
  for (int index = 1; index < waves; ++index)
    total = fmaxf(total, scratch[index]);
  return total;
}

// What a captured proposer pass does with its arg-max token before the next
// pass starts (qllm_rollout_advance): the token becomes the next pass's input
// and the next entry of the draft list, the positions move on by `rows`.
struct RolloutAdvance {
  uint32_t* next_token;
  uint32_t* draft_tokens;
  uint32_t capacity;
  uint32_t rows;
  uint32_t* positions;
};

// Stage 2 of an arg-max whose stage-1 partials lie in [batch][blocks] arrays
// (select.hip); with `advance` (batch 1) the same launch also advances the
// rollout with the winner.
int32_t launch_argmax_final(const float* partial_values,
                            const uint32_t* partial_indices, uint32_t blocks,
                            uint32_t batch, uint32_t* output,
                            const RolloutAdvance* advance, hipStream_t stream);

// splitmix64 counter generator shared with the host-side restatement.
__host__ __device__ inline uint64_t mix64(uint64_t seed, uint64_t index) {
  uint64_t value = seed ^ (index * 0x9e3779b97f4a7c15ull + 0x632be59bd9b4e019ull);
  value += 0x9e3779b97f4a7c15ull;
  value = (value ^ (value >> 30)) * 0xbf58476d1ce4e5b9ull;
  value = (value ^ (value >> 27)) * 0x94d049bb133111ebull;
  return value ^ (value >> 31);
}

}  // namespace qllm
