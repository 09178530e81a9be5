// Pieces shared by the paged decode-attention split kernels (Q4H and exact
// F16 caches): lane-group reductions, the scalar page-table fetch, and the
// merge of a workgroup's eight wave states into one split partial.
#pragma once

#include "common.hpp"

#include <type_traits>

namespace qllm {

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kSplitWaves = 8;
constexpr float kMaskedMax = -1.0e30f;

// max over the lanes {l, l^16, l^32, l^48}
__device__ __forceinline__ float quad_row_max(float value) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(value),
                                            __float_as_uint(value), false, false);
  value = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(value),
                                            __float_as_uint(value), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// max over all 64 lanes without the LDS pipeline: four cross-lane steps inside
// each row of 16 lanes, then the rows
__device__ __forceinline__ float wave_max_in_registers(float value) {
  const auto step = [](float v, auto control) {
    const int moved = __builtin_amdgcn_update_dpp(
        __float_as_int(v), __float_as_int(v), decltype(control)::value, 0xf, 0xf,
        false);
    return fmaxf(v, __int_as_float(moved));
  };
  value = step(value, std::integral_constant<int, 0xb1>{});    // quad_perm 1,0,3,2
  value = step(value, std::integral_constant<int, 0x4e>{});    // quad_perm 2,3,0,1
  value = step(value, std::integral_constant<int, 0x141>{});   // row_half_mirror
  value = step(value, std::integral_constant<int, 0x140>{});   // row_mirror
  return quad_row_max(value);
}

__device__ __forceinline__ float quad_row_sum(float value) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(value),
                                            __float_as_uint(value), false, false);
  value = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(value),
                                            __float_as_uint(value), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Page table entry at a wave-uniform index, fetched with a scalar load (the
// table is never written while attention kernels run), so everything derived
// from the page address stays in scalar registers.
__device__ __forceinline__ const void* uniform_page(
    const void* const* page_table, uint32_t index) {
  typedef const void* __attribute__((address_space(4))) const* constant_table;
  return ((constant_table)page_table)[index];
}

// Tells the compiler that a pointer every lane computes alike is wave-uniform,
// so that it can live in scalar registers.
__device__ __forceinline__ const uint8_t* uniform_pointer(const uint8_t* pointer) {
  const uint64_t bits = reinterpret_cast<uint64_t>(pointer);
  const uint32_t low =
      __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits));
  const uint32_t high =
      __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits >> 32));
  return reinterpret_cast<const uint8_t*>((static_cast<uint64_t>(high) << 32) | low);
}

// Direct global -> LDS loads (no VGPRs): lane l of the wave fetches 16 (4)
// bytes at base + offset[l] and they land at lds + 16*l (4*l).  `base` and
// `lds` are wave-uniform.  Written as assembly so that the address stays in
// the scalar-base + 32-bit-lane-offset form (one VGPR for all loads of a tile)
// and so that the compiler, which would otherwise wait for every outstanding
// load before any later LDS access, leaves the waiting to this kernel.
__device__ __forceinline__ void copy16_to_lds(const uint8_t* base,
                                              uint32_t lane_offset,
                                              uint32_t lds) {
  uint32_t saved_m0;  // M0 carries the LDS address; it is put back afterwards
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %3\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved_m0) : "v"(lane_offset), "s"(base), "s"(lds) : "memory");
}
__device__ __forceinline__ void copy4_to_lds(const uint8_t* base,
                                             uint32_t lane_offset,
                                             uint32_t lds) {
  uint32_t saved_m0;  // M0 carries the LDS address; it is put back afterwards
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %3\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dword %1, %2\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved_m0) : "v"(lane_offset), "s"(base), "s"(lds) : "memory");
}

// at most COUNT vmem loads (direct-to-LDS loads included) still in flight
template <int COUNT>
__device__ __forceinline__ void vmem_wait() {
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"(COUNT) : "memory");
}
// Lane index recomputed where it is needed (two instructions) instead of
// being kept in a register across the tile loop.
__device__ __forceinline__ uint32_t fresh_lane_index() {
  uint32_t lane;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0"
               : "=v"(lane));
  return lane;
}
__device__ __forceinline__ uint32_t lds_address(const void* pointer) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) const void*)pointer));
}

// A word of a small device-side parameter block (step positions) that no
// kernel writes: fetched with a scalar load, like the page table.
__device__ __forceinline__ uint32_t uniform_word(const uint32_t* words,
                                                 uint32_t index) {
  typedef const uint32_t __attribute__((address_space(4)))* constant_words;
  return ((constant_words)words)[index];
}

// One wave writes the K (kind 0) or V (kind 1) vector of (cache slot, kv head)
// into the proposer's Q8 layer at `layer_base` (page + the layer's offset):
// codes [kind][slot][kv head][head_dim] int8, then scales [kind][kv head]
// [page_tokens] binary16; scale = f16(max(absmax / 127, 2^-24)), code =
// clamp(rn(x / scale), -127, 127) (transformer_kernels.cu:601-625).  `source`
// may lie in LDS or in global memory.
__device__ __forceinline__ void q8_encode_record(const float* source,
                                                 uint32_t head_dim, uint8_t* layer_base,
                                                 uint32_t kind, uint32_t slot,
                                                 uint32_t kv_head, uint32_t kv_heads,
                                                 uint32_t page_tokens, uint32_t lane) {
  const size_t codes_bytes = static_cast<size_t>(page_tokens) * kv_heads * head_dim;
  const size_t record = static_cast<size_t>(slot) * kv_heads + kv_head;
  float maximum = 0.0f;
  for (uint32_t index = lane; index < head_dim; index += 64u)
    maximum = fmaxf(maximum, fabsf(source[index]));
  maximum = wave_max(maximum);
  const uint32_t scale_bits = f32_to_f16_bits(fmaxf(maximum / 127.0f, 0x1p-24f));
  const float scale = f16_bits_to_f32(scale_bits);
  int8_t* codes =
      reinterpret_cast<int8_t*>(layer_base + kind * codes_bytes) + record * head_dim;
  for (uint32_t index = lane; index < head_dim; index += 64u) {
    const int code = max(-127, min(127, __float2int_rn(source[index] / scale)));
    codes[index] = static_cast<int8_t>(code);
  }
  if (lane == 0u) {
    uint16_t* scales = reinterpret_cast<uint16_t*>(layer_base + 2u * codes_bytes) +
                       static_cast<size_t>(kind) * kv_heads * page_tokens;
    scales[static_cast<size_t>(kv_head) * page_tokens + slot] =
        static_cast<uint16_t>(scale_bits);
  }
}

// Tiles [first, last) of the context that wave `wave` of split `split` walks.
// split_tokens == 0: balanced - the context's tiles are dealt evenly over
// every wave of the grid row, whatever the context length.  Otherwise split
// s covers tokens [s*split_tokens, (s+1)*split_tokens) and its tiles are dealt
// evenly over the workgroup's waves.
// tail_work (balanced only): what the waves at the end of the context do
// besides their tiles, in tiles' worth of time - the deal is over
// context_tiles + tail_work tiles of which the last tail_work do not exist, so
// those waves walk that many fewer.
__device__ __forceinline__ void wave_tile_range(uint32_t context_tiles,
                                                uint32_t tile_tokens,
                                                uint32_t split_tokens,
                                                uint32_t split, uint32_t splits,
                                                uint32_t wave,
                                                uint32_t& tile_first,
                                                uint32_t& tile_last,
                                                uint32_t tail_work = 0u) {
  if (split_tokens == 0u) {
    // floor(slot * tiles / slots) in 32-bit arithmetic: with tiles = q * slots
    // + r it is slot * q + floor(slot * r / slots), and slot * r < slots^2
    const uint32_t slots = splits * kSplitWaves;
    const uint32_t slot = split * kSplitWaves + wave;
    const uint32_t dealt = context_tiles + tail_work;
    const uint32_t quotient = dealt / slots;
    const uint32_t remainder = dealt - quotient * slots;
    tile_first = min(slot * quotient + slot * remainder / slots, context_tiles);
    tile_last = min((slot + 1u) * quotient + (slot + 1u) * remainder / slots,
                    context_tiles);
  } else {
    const uint32_t split_tiles = split_tokens / tile_tokens;
    const uint32_t begin = min(split * split_tiles, context_tiles);
    const uint32_t count = min(begin + split_tiles, context_tiles) - begin;
    tile_first = begin + wave * count / kSplitWaves;
    tile_last = begin + (wave + 1u) * count / kSplitWaves;
  }
}

struct PartialTarget {
  float* partial_maxima;   // [rows, maximum_splits, query_heads]
  float* partial_sums;     // same
  float* partial_outputs;  // [rows, maximum_splits, query_heads, D]
  uint32_t maximum_splits;
  uint32_t query_heads;
  uint32_t kv_head;
  uint32_t split;
  uint32_t group;          // query heads per KV head
  uint32_t matrix_rows;    // rows * group
};

// Merges the eight wave states of a workgroup and writes the split partial.
// A wave's state: per row tile rt (16 matrix rows; lane (col = lane%16, quad =
// lane/16) owns matrix row 16*rt + col) the running maximum (log2 units) and
// sum, and out[dt][rt] = O^T elements d = 16*dt + 4*quad .. +3 of that row.
//  1. every wave publishes its (max, sum) per row; all waves derive the
//     merged maximum and bring their own accumulators to it.
//  2. the accumulators are summed reduce-scatter style, eight 1 KiB register
//     vectors (one per receiving wave) at a time: each wave drops the eight
//     vectors of the group into LDS, lane-linear (no bank conflicts), and
//     wave v adds up vector v of all eight waves in a fixed order.  Wave v
//     ends up owning vectors v, v+8, ... of the result and writes them out.
// `pool` needs 64 KiB of LDS, `summary` 512*RT bytes per wave; both may
// overlap whatever the tile loop used (the function starts with a barrier).
template <int D, int RT>
__device__ __forceinline__ void merge_wave_states(
    float (&running_max)[RT], float (&running_sum)[RT],
    f32x4 (&out)[D / 16][RT], float* pool, float2* summary, uint32_t wave,
    uint32_t lane, const PartialTarget& target) {
  constexpr int DT = D / 16;
  constexpr int VECTORS = DT * RT;   // f32x4 accumulator vectors per wave
  static_assert(VECTORS % kSplitWaves == 0, "vectors are dealt to 8 waves");
  const uint32_t col = lane & 15u;
  const uint32_t quad = lane >> 4;
  __syncthreads();  // tiles done: the LDS they used is free
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
    summary[(wave * RT + rt) * 64 + lane] =
        make_float2(running_max[rt], running_sum[rt]);
  __syncthreads();
  float merged_max[RT], merged_sum[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    float2 part[kSplitWaves];
    float maximum = kMaskedMax;
#pragma unroll
    for (int w = 0; w < kSplitWaves; ++w) {
      part[w] = summary[(w * RT + rt) * 64 + lane];
      maximum = fmaxf(maximum, part[w].x);
    }
    float sum = 0.0f;
#pragma unroll
    for (int w = 0; w < kSplitWaves; ++w)
      sum = fmaf(part[w].y, __builtin_amdgcn_exp2f(part[w].x - maximum), sum);
    const float factor = __builtin_amdgcn_exp2f(running_max[rt] - maximum);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) out[dt][rt][i] *= factor;
    merged_max[rt] = maximum;
    merged_sum[rt] = sum;
  }
  f32x4 merged[VECTORS / kSplitWaves];
#pragma unroll
  for (int group_index = 0; group_index < VECTORS / kSplitWaves; ++group_index) {
#pragma unroll
    for (int v = 0; v < kSplitWaves; ++v) {
      const int k = group_index * kSplitWaves + v;
      *reinterpret_cast<f32x4*>(pool + ((wave * kSplitWaves + v) * 64 + lane) * 4u) =
          out[k / RT][k % RT];
    }
    __syncthreads();
    f32x4 total = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int w = 0; w < kSplitWaves; ++w)
      total += *reinterpret_cast<const f32x4*>(
          pool + ((w * kSplitWaves + wave) * 64 + lane) * 4u);
    merged[group_index] = total;
    __syncthreads();
  }

  // partials: wave v writes the vectors it owns, wave 0 also max and sum
#pragma unroll
  for (int group_index = 0; group_index < VECTORS / kSplitWaves; ++group_index) {
    const uint32_t k = group_index * kSplitWaves + wave;
    const uint32_t dt = k / RT;
    const uint32_t rt = k % RT;
    const uint32_t matrix_row = 16u * rt + col;
    if (matrix_row >= target.matrix_rows) continue;
    const uint32_t row = matrix_row / target.group;
    const uint32_t head = target.kv_head * target.group + matrix_row % target.group;
    const size_t partial =
        (static_cast<size_t>(row) * target.maximum_splits + target.split) *
            target.query_heads + head;
    *reinterpret_cast<f32x4*>(target.partial_outputs + partial * D + 16u * dt +
                              4u * quad) = merged[group_index];
  }
  if (wave != 0u || quad != 0u) return;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const uint32_t matrix_row = 16u * rt + col;
    if (matrix_row >= target.matrix_rows) continue;
    const uint32_t row = matrix_row / target.group;
    const uint32_t head = target.kv_head * target.group + matrix_row % target.group;
    const size_t partial =
        (static_cast<size_t>(row) * target.maximum_splits + target.split) *
            target.query_heads + head;
    target.partial_maxima[partial] = merged_max[rt];
    target.partial_sums[partial] = merged_sum[rt];
  }
}

}  // namespace qllm
