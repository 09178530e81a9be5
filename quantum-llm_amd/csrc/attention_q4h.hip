// Decode attention over the Q4H ("q4-f16-per-head") paged KV cache for a
// micro-batch of query rows (1 guaranteed + drafts), plus the K/V store and
// query quantisation that precede it.
//
// Replaces, from runtime/src/cuda/transformer_kernels.cu of the reference:
//   store_paged_kv_record<q4_per_head>                         :241-288
//   gated_gqa_qkv_rope_paged_batch_kernel<q4_per_head>         :3550-3643
//   quantize_gqa_queries_q8_kernel                             :4391-4416
//   gated_gqa_attention_paged_bfp_microbatch_split_kernel      :4420-4976
//   gated_gqa_attention_paged_fp4_prefill_combine_kernel       :5741-5798
//
// Split kernel, one workgroup (8 waves) per (kv head, context split); each
// wave walks 64-token tiles of the split with its own online-softmax state:
//   scores  S[tok][row] = K4 . Q15       v_mfma_i32_16x16x64_i8, exact ints:
//           K nibbles are widened to int8*16 with two bit operations and the
//           query is carried as two int8 planes (15 bits), built in-kernel
//           from the F32 query - a single Q8 plane, as the reference uses,
//           is ~1e-2 away from exact attention on N(0,1) inputs
//   softmax in F32 per lane (a lane owns one query row of a 16-row tile)
//   output  O^T[d][row] += V^T . P^T     v_mfma_f32_16x16x32_f16, V staged
//           through LDS and read back transposed with ds_read_b64_tr_b4,
//           the per-token V scale folded into the nibble->f16 conversion.
// The eight wave states are merged in LDS and one (max, sum, unnormalised
// output) partial per (row, split, head) is written; the combine kernel
// merges the splits.  Maxima are kept in the log2 domain.
#include "attention_common.hpp"

#include <algorithm>
#include <utility>

namespace qllm {
namespace {


struct Q4hPlanes {
  const uint8_t* key_codes;
  const uint8_t* key_scales;
  const uint8_t* value_codes;
  const uint8_t* value_scales;
};

__host__ __device__ inline size_t q4h_layer_bytes(uint32_t page_tokens,
                                                  uint32_t kv_heads,
                                                  uint32_t head_dim) {
  return static_cast<size_t>(page_tokens) * kv_heads * 2u *
         (head_dim / 2u + 2u);
}

__device__ __forceinline__ Q4hPlanes q4h_planes(const void* page,
                                                uint32_t layer,
                                                uint32_t page_tokens,
                                                uint32_t kv_heads,
                                                uint32_t head_dim) {
  const size_t records = static_cast<size_t>(page_tokens) * kv_heads;
  Q4hPlanes planes;
  planes.key_codes = static_cast<const uint8_t*>(page) +
                     layer * q4h_layer_bytes(page_tokens, kv_heads, head_dim);
  planes.key_scales = planes.key_codes + records * (head_dim / 2u);
  planes.value_codes = planes.key_scales + records * 2u;
  planes.value_scales = planes.value_codes + records * (head_dim / 2u);
  return planes;
}

// Prepared query operands of one KV head: for every 16-row tile of its
// rows * group matrix rows and every 64-wide k-step of head_dim a high and a
// low int8 plane of 1 KiB in matrix-core operand order (lane (col, quad) owns
// bytes [16 * (16 * quad + col), +16) of a plane), q = scale * (128 * high +
// low); the scales, already multiplied by log2(e) / (16 sqrt(head_dim)), are
// a separate array of 16 floats per row tile.
__host__ __device__ inline uint32_t q4h_row_tiles(uint32_t rows, uint32_t group) {
  return (rows * group + 15u) / 16u;
}
__host__ __device__ inline size_t q4h_operand_plane_bytes(uint32_t row_tiles,
                                                          uint32_t head_dim) {
  return static_cast<size_t>(row_tiles) * (head_dim / 64u) * 2u * 1024u;
}

struct SplitArgs {
  const float* query;
  // Optional: the query operands as qkv_rope_q4h_kernel prepares them (see
  // q4h_query_operand_bytes); the kernel then copies them instead of
  // quantising `query`.
  const uint8_t* query_operands;
  const float* query_operand_scales;
  uint32_t query_stride;
  const void* const* page_table;
  float* partial_maxima;
  float* partial_sums;
  float* partial_outputs;
  uint32_t first_context_tokens;
  uint32_t rows;
  uint32_t layer;
  uint32_t page_tokens;
  uint32_t query_heads;
  uint32_t kv_heads;
  uint32_t split_tokens;
  uint32_t maximum_splits;
  const uint32_t* device_positions;  // optional: [2] = first_context_tokens
  // Batched launch (prompt prefill): workgroups of grid layer z take rows
  // [z * batch_rows, +batch_rows) of `rows`, each layer a launch of its own as
  // far as the kernel is concerned.  0 = one batch holds all rows.
  uint32_t batch_rows;
  // Fused rotary and K/V store (the FUSED instantiation): `query` then holds
  // the projection's raw rows, raw_key / raw_value the batch's K and V rows,
  // rope_table the rows' (cos, sin) as rope_table_kernel leaves them.
  const float* raw_key;
  const float* raw_value;
  const float* q_weight;
  const float* k_weight;
  const float2* rope_table;
  uint32_t rotary_dim;
  float epsilon;
  uint32_t first_cache_position;   // or device_positions[0]
  uint32_t bf16_activations;
};




// LDS reads of staged tiles.  They are written as inline assembly on purpose:
// the compiler then does not know that they touch memory a direct-to-LDS load
// may still be filling, so it inserts no blanket "wait for every outstanding
// load" in front of them, and the kernel places its own, exact waits
// (vmem loads complete in issue order).  The values are not valid until
// lds_wait() has been given them.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

template <int OFFSET>
__device__ __forceinline__ u32x4 lds_read16(uint32_t address) {
  u32x4 result;
  asm volatile("ds_read_b128 %0, %1 offset:%2"
               : "=v"(result) : "v"(address), "n"(OFFSET));
  return result;
}
template <int OFFSET>
__device__ __forceinline__ u32x2 lds_read8(uint32_t address) {
  u32x2 result;
  asm volatile("ds_read_b64 %0, %1 offset:%2"
               : "=v"(result) : "v"(address), "n"(OFFSET));
  return result;
}
// 16x16 transpose of 4-bit elements across each group of 16 lanes
template <int OFFSET>
__device__ __forceinline__ u32x2 lds_read8_transposed4(uint32_t address) {
  u32x2 result;
  asm volatile("ds_read_b64_tr_b4 %0, %1 offset:%2"
               : "=v"(result) : "v"(address), "n"(OFFSET));
  return result;
}
// waits for the LDS reads above and ties the values to the wait
template <int N, typename T>
__device__ __forceinline__ void lds_wait(T (&values)[N]) {
  static_assert(N == 4 || N == 8 || N == 16, "unsupported operand count");
  if constexpr (N == 4)
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(values[0]), "+v"(values[1]), "+v"(values[2]),
                   "+v"(values[3]) :: "memory");
  else if constexpr (N == 8)
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(values[0]), "+v"(values[1]), "+v"(values[2]),
                   "+v"(values[3]), "+v"(values[4]), "+v"(values[5]),
                   "+v"(values[6]), "+v"(values[7]) :: "memory");
  else
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(values[0]), "+v"(values[1]), "+v"(values[2]),
                   "+v"(values[3]), "+v"(values[4]), "+v"(values[5]),
                   "+v"(values[6]), "+v"(values[7]), "+v"(values[8]),
                   "+v"(values[9]), "+v"(values[10]), "+v"(values[11]),
                   "+v"(values[12]), "+v"(values[13]), "+v"(values[14]),
                   "+v"(values[15]) :: "memory");
}
// Global loads the compiler's wait insertion does not see, for values whose
// arrival the kernel waits for itself (vmem_wait_units, then tie()): a wait the
// compiler places counts only the loads it knows, so it would also wait for
// every direct-to-LDS load issued after them.  `base` is wave-uniform.
typedef float f32x2 __attribute__((ext_vector_type(2)));
template <int OFFSET>
__device__ __forceinline__ float load_f32_uncounted(const void* base,
                                                    uint32_t byte_offset) {
  float value;
  asm volatile("global_load_dword %0, %1, %2 offset:%3"
               : "=v"(value) : "v"(byte_offset), "s"(base), "n"(OFFSET) : "memory");
  return value;
}
__device__ __forceinline__ f32x2 load_f32x2_uncounted(const void* base,
                                                      uint32_t byte_offset) {
  f32x2 value;
  asm volatile("global_load_dwordx2 %0, %1, %2"
               : "=v"(value) : "v"(byte_offset), "s"(base) : "memory");
  return value;
}
// orders every use of `value` after the volatile statements before this one
template <typename T>
__device__ __forceinline__ void tie(T& value) {
  asm volatile("" : "+v"(value));
}
// at most `units` * UNIT vmem loads still in flight; `units` is wave-uniform
template <int UNIT>
__device__ __forceinline__ void vmem_wait_units(uint32_t units) {
  static_assert(4 * UNIT < 64, "vmcnt holds six bits");
  if (units == 0u) vmem_wait<0>();
  else if (units == 1u) vmem_wait<UNIT>();
  else if (units == 2u) vmem_wait<2 * UNIT>();
  else if (units == 3u) vmem_wait<3 * UNIT>();
  else vmem_wait<4 * UNIT>();
}
// (value & mask) | (base & ~mask) in one instruction
__device__ __forceinline__ uint32_t insert_bits(uint32_t mask, uint32_t value,
                                                uint32_t base) {
  uint32_t result;
  asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(result) : "s"(mask), "v"(value), "v"(base));
  return result;
}
// One wave encodes one (token, kv head) K or V vector.
__device__ __forceinline__ void q4h_encode_record(const float* source,
                                                  uint32_t head_dim,
                                                  uint8_t* codes,
                                                  uint8_t* scale_slot,
                                                  uint32_t lane) {
  float maximum = 0.0f;
  for (uint32_t index = lane; index < head_dim; index += 64u)
    maximum = fmaxf(maximum, fabsf(source[index]));
  maximum = wave_max(maximum);
  const uint32_t scale_bits =
      f32_to_f16_bits(fmaxf(__fdiv_rn(maximum, 7.0f), 0x1p-24f));
  const float scale = f16_bits_to_f32(scale_bits);
  if (lane == 0u)
    *reinterpret_cast<uint16_t*>(scale_slot) = static_cast<uint16_t>(scale_bits);
  for (uint32_t pair = lane; pair < head_dim / 2u; pair += 64u) {
    const int low = max(-7, min(7, __float2int_rn(__fdiv_rn(source[2u * pair], scale))));
    const int high =
        max(-7, min(7, __float2int_rn(__fdiv_rn(source[2u * pair + 1u], scale))));
    codes[pair] = static_cast<uint8_t>((low & 0x0f) | ((high & 0x0f) << 4));
  }
}

// Per-head RMSNorm(1+w) and NeoX rotary; one wave per (head, row).  The
// rotated row is left in `rotated` (LDS) for a caller that goes on to encode
// it, and written to `write_back` unless that is null.  TABLE: cosine and sine
// of the row's position come from `table_row` [rotary_dim / 2] (as
// rope_table_kernel leaves them) instead of being computed here.
template <bool TABLE>
__device__ __forceinline__ void head_norm_rope_impl(
    const float* x, float* write_back, const float* weight, uint32_t head_dim,
    uint32_t rotary_dim, uint32_t position, float epsilon, float theta,
    bool bf16_activations, const float2* table_row, float* shared,
    float* rotated, uint32_t lane) {
  if (weight) {
    float square = 0.0f;
    for (uint32_t index = lane; index < head_dim; index += 64u)
      square = fmaf(x[index], x[index], square);
    square = wave_sum(square);
    const float inverse =
        rsqrtf(square / static_cast<float>(head_dim) + epsilon);
    for (uint32_t index = lane; index < head_dim; index += 64u) {
      const float value = x[index] * inverse * (1.0f + weight[index]);
      shared[index] = bf16_activations ? bf16_round(value) : value;
    }
  } else {
    for (uint32_t index = lane; index < head_dim; index += 64u)
      shared[index] = x[index];
  }
  __builtin_amdgcn_wave_barrier();
  const uint32_t half = rotary_dim / 2u;
  for (uint32_t index = lane; index < head_dim; index += 64u) {
    float result = shared[index];
    if (index < rotary_dim) {
      const uint32_t pair = index % half;
      const float other =
          index < half ? -shared[index + half] : shared[index - half];
      float sine, cosine;
      if constexpr (TABLE) {
        const float2 entry = table_row[pair];
        cosine = entry.x;
        sine = entry.y;
      } else {
        const float angle =
            static_cast<float>(position) *
            powf(theta, -2.0f * static_cast<float>(pair) /
                            static_cast<float>(rotary_dim));
        sincosf(angle, &sine, &cosine);
        if (bf16_activations) {
          cosine = bf16_round(cosine);
          sine = bf16_round(sine);
        }
      }
      // one rounding order wherever this is compiled in
      result = __fmaf_rn(shared[index], cosine, __fmul_rn(other, sine));
    }
    result = bf16_activations ? bf16_round(result) : result;
    if (write_back) write_back[index] = result;
    rotated[index] = result;
  }
  __builtin_amdgcn_wave_barrier();
}

__device__ __forceinline__ void head_norm_rope(float* x, const float* weight,
                                               uint32_t head_dim,
                                               uint32_t rotary_dim,
                                               uint32_t position, float epsilon,
                                               float theta, bool bf16_activations,
                                               float* shared, float* rotated,
                                               uint32_t lane) {
  head_norm_rope_impl<false>(x, x, weight, head_dim, rotary_dim, position,
                             epsilon, theta, bf16_activations, nullptr, shared,
                             rotated, lane);
}

// The same arithmetic on a row that is already in registers (lane l holds
// elements l, l + 64, ...: x, the norm weights and the (cos, sin) of each
// element's pair), so that a caller can fetch several rows at once and pay one
// memory round trip for all of them.  The rotated row is left in `rotated`.
template <int N>
__device__ __forceinline__ void head_norm_rope_registers(
    const float (&x)[N], const float (&weight)[N], bool has_weight,
    uint32_t rotary_dim, const float2 (&entry)[N], float epsilon,
    bool bf16_activations, float* shared, float* rotated, uint32_t lane) {
  constexpr uint32_t head_dim = 64u * N;
  if (has_weight) {
    float square = 0.0f;
#pragma unroll
    for (int k = 0; k < N; ++k) square = fmaf(x[k], x[k], square);
    square = wave_sum(square);
    const float inverse =
        rsqrtf(square / static_cast<float>(head_dim) + epsilon);
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const float value = x[k] * inverse * (1.0f + weight[k]);
      shared[lane + 64u * k] = bf16_activations ? bf16_round(value) : value;
    }
  } else {
#pragma unroll
    for (int k = 0; k < N; ++k) shared[lane + 64u * k] = x[k];
  }
  __builtin_amdgcn_wave_barrier();
  const uint32_t half = rotary_dim / 2u;
#pragma unroll
  for (int k = 0; k < N; ++k) {
    const uint32_t index = lane + 64u * k;
    float result = shared[index];
    if (index < rotary_dim) {
      const float other =
          index < half ? -shared[index + half] : shared[index - half];
      result = __fmaf_rn(shared[index], entry[k].x, __fmul_rn(other, entry[k].y));
    }
    rotated[index] = bf16_activations ? bf16_round(result) : result;
  }
  __builtin_amdgcn_wave_barrier();
}

// The same once more without LDS, for rotary halves that are a multiple of 64
// elements: both elements of a pair then sit in the same lane.  The rotated
// row is returned in `rotated` (registers).
template <int N>
__device__ __forceinline__ void head_norm_rope_in_lane(
    const float (&x)[N], const float (&weight)[N], bool has_weight,
    uint32_t rotary_dim, const float2 (&entry)[N], float epsilon,
    bool bf16_activations, float (&rotated)[N], uint32_t lane) {
  constexpr uint32_t head_dim = 64u * N;
  float value[N];
  if (has_weight) {
    float square = 0.0f;
#pragma unroll
    for (int k = 0; k < N; ++k) square = fmaf(x[k], x[k], square);
    square = wave_sum(square);
    const float inverse =
        rsqrtf(square / static_cast<float>(head_dim) + epsilon);
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const float scaled = x[k] * inverse * (1.0f + weight[k]);
      value[k] = bf16_activations ? bf16_round(scaled) : scaled;
    }
  } else {
#pragma unroll
    for (int k = 0; k < N; ++k) value[k] = x[k];
  }
  const int shift = static_cast<int>(rotary_dim / 128u);   // pair distance in k
#pragma unroll
  for (int k = 0; k < N; ++k) {
    float result = value[k];
    if (k < 2 * shift) {
      float partner = 0.0f;
#pragma unroll
      for (int j = 0; j < N; ++j)
        if (k < shift ? j == k + shift : j + shift == k) partner = value[j];
      const float other = k < shift ? -partner : partner;
      result = __fmaf_rn(value[k], entry[k].x, __fmul_rn(other, entry[k].y));
    }
    rotated[k] = bf16_activations ? bf16_round(result) : result;
  }
}

// Cosine and sine of rows' rotary angles, one (cos, sin) per (row, pair): what
// head_norm_rope computes for itself, once per step instead of once per layer.
__global__ void rope_table_kernel(float2* table, uint32_t rotary_dim,
                                  uint32_t first_rotary_position, float theta,
                                  bool bf16_activations,
                                  const uint32_t* device_positions) {
  if (device_positions)
    first_rotary_position = uniform_word(device_positions, 1u);
  const uint32_t half = rotary_dim / 2u;
  const uint32_t row = blockIdx.x;
  for (uint32_t pair = threadIdx.x; pair < half; pair += blockDim.x) {
    const float angle =
        static_cast<float>(first_rotary_position + row) *
        powf(theta, -2.0f * static_cast<float>(pair) /
                        static_cast<float>(rotary_dim));
    float sine, cosine;
    sincosf(angle, &sine, &cosine);
    if (bf16_activations) {
      cosine = bf16_round(cosine);
      sine = bf16_round(sine);
    }
    table[row * half + pair] = make_float2(cosine, sine);
  }
}

// D = head_dim (128 or 256), RT = number of 16-row tiles (rows*group <= 16*RT).
//
// Each wave owns a contiguous run of 64-token tiles.  A tile's K codes, V
// codes and scales travel global -> LDS with direct loads into a wave-private
// staging area [K codes + scales | V codes]; each half is refilled with the
// next tile as soon as the current tile has been read out of it, so the
// loads fly while the matrix cores and the softmax work on registers.
//
// FUSED: the kernel also does what qkv_rope_q4h_kernel does for the batch.
// Every workgroup rotates (and, with weights, normalises) the query rows of
// its KV head itself and quantises them straight into the operand area - this
// work hides behind the flight of the first tile.  The batch's own K/V records
// are encoded by the workgroups whose tiles reach them, into LDS, and laid over
// the staged tile before it is read (the cache pages need not hold them yet);
// the workgroup that owns the context's last tile also writes them to the
// pages for later steps.
template <int D, int RT, bool FUSED = false>
__global__ __launch_bounds__(kSplitWaves * 64) void q4h_attention_split_kernel(
    const SplitArgs launch_args) {
  // a batched launch narrows the arguments to the batch of this grid layer
  SplitArgs args = launch_args;
  if (!FUSED && launch_args.batch_rows) {
    // (the batches with the longest contexts, the last rows, are dispatched first)
    const uint32_t first_row =
        (gridDim.z - 1u - blockIdx.z) * launch_args.batch_rows;
    const size_t first_partial = static_cast<size_t>(first_row) *
                                 launch_args.maximum_splits *
                                 launch_args.query_heads;
    args.rows = min(launch_args.batch_rows, launch_args.rows - first_row);
    args.first_context_tokens = launch_args.first_context_tokens + first_row;
    args.query = launch_args.query + static_cast<size_t>(first_row) *
                                         launch_args.query_heads *
                                         launch_args.query_stride;
    args.partial_maxima = launch_args.partial_maxima + first_partial;
    args.partial_sums = launch_args.partial_sums + first_partial;
    args.partial_outputs = launch_args.partial_outputs + first_partial * D;
  }
  // Everything the prologue reads from the argument block is asked for here,
  // in one round trip, not piece by piece along its chain of dependencies.
  asm volatile("" ::"s"(args.query), "s"(args.page_table),
               "s"(args.device_positions), "s"(args.query_operands),
               "s"(args.query_operand_scales), "s"(args.query_stride),
               "s"(args.first_context_tokens), "s"(args.rows), "s"(args.layer),
               "s"(args.page_tokens), "s"(args.query_heads), "s"(args.kv_heads),
               "s"(args.split_tokens));
  if constexpr (FUSED)
    asm volatile("" ::"s"(args.raw_key), "s"(args.raw_value), "s"(args.q_weight),
                 "s"(args.k_weight), "s"(args.rope_table), "s"(args.rotary_dim),
                 "s"(args.first_cache_position), "s"(args.bf16_activations));
  constexpr int KSTEPS = D / 64;      // int8 MFMA k-steps over head_dim
  constexpr int DT = D / 16;          // 16-wide tiles of head_dim
  constexpr int ROW = D / 2;          // bytes of codes per token
  constexpr int CODES = 64 * ROW;     // bytes of K (or V) codes per tile
  // staging area of a wave: K codes | K scales | V codes | V scales
  constexpr int STAGE = 2 * CODES + 512;
  constexpr int PASSES = ROW / 16;    // direct loads per code plane and tile
  constexpr int KS_LOADS = PASSES + 1;       // K codes + K scales
  constexpr int V_LOADS = PASSES + 1;        // V codes + V scales
  static_assert(KS_LOADS == V_LOADS, "the waits count loads in units of one half tile");
  // Tiles of a wave in flight.  At head_dim 128 LDS holds two staging areas
  // per wave: the wave's first two tiles set out together at the start (at
  // 32K tokens a wave has two tiles in all), and a tile's half is refilled
  // with the tile after the next.
  constexpr int DEPTH = 1;
  __shared__ __attribute__((aligned(16)))
  uint8_t stage[kSplitWaves * STAGE * DEPTH];
  // query operands in MFMA order, then per matrix row its scale and the number
  // of tokens it may attend
  __shared__ __attribute__((aligned(16)))
  uint8_t exchange[RT * KSTEPS * 2 * 1024 + 2 * RT * 64];

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t col = lane & 15u;   // query row inside a row tile / token / d
  const uint32_t quad = lane >> 4;   // 0..3
  const uint32_t kv_head = blockIdx.x;
  const uint32_t split = blockIdx.y;
  const uint32_t group = args.query_heads / args.kv_heads;
  const uint32_t matrix_rows = args.rows * group;
  const uint32_t first_context_tokens =
      args.device_positions ? uniform_word(args.device_positions, 2u)
                            : args.first_context_tokens;
  const uint32_t last_context = first_context_tokens + args.rows - 1u;
  const uint32_t context_tiles = (last_context + 63u) / 64u;

  // tiles [tile_first, tile_last) of this wave
  uint32_t tile_first, tile_last;
  // (fused: the workgroup at the end of the context also encodes the batch's
  // K/V records, lays them over its tiles and writes them to their pages -
  // about two tiles' worth of time for each of its waves.  The plain kernel
  // deals the same way, so that both add up a context in the same order.)
  constexpr uint32_t kTailWork = 2u * kSplitWaves;
  wave_tile_range(context_tiles, 64u, args.split_tokens, split, gridDim.y, wave,
                  tile_first, tile_last, kTailWork);

  // the wave's staging areas: tile t of the wave uses area t % DEPTH
  uint8_t* const stage_base = stage + wave * (STAGE * DEPTH);
  const uint32_t stage_k_lds =
      __builtin_amdgcn_readfirstlane(lds_address(stage_base));
  const uint32_t stage_s_lds = stage_k_lds + CODES;
  const uint32_t stage_v_lds = stage_s_lds + 256;
  const uint32_t stage_vs_lds = stage_v_lds + CODES;
  float* exchange_scale =
      reinterpret_cast<float*>(exchange + RT * KSTEPS * 2 * 1024);
  uint32_t* exchange_limit =
      reinterpret_cast<uint32_t*>(exchange + RT * KSTEPS * 2 * 1024 + RT * 64);

  constexpr uint32_t kParts = ROW / 16;        // 16-byte pieces per token
  constexpr uint32_t kPassRows = 64 / kParts;  // LDS rows per pass
  // V scales sit one V code plane + one K scale plane past the K scales
  const uint32_t value_scale_distance =
      args.page_tokens * args.kv_heads * (ROW + 2u);

  // KS_LOADS direct loads: K codes and K scales of a tile.  Pass `pass` covers
  // the 1 KiB at pass*1024 of the tile's K rows; lanes 0..31 then fetch the
  // scales of tokens 2l, 2l+1 (lanes 32..63 repeat them).
  auto stage_keys = [&](uint32_t tile, uint32_t area) {
    const uint32_t lane_now = fresh_lane_index();
    const uint32_t tile_begin = tile * 64u;
    const void* page = uniform_page(args.page_table, tile_begin / args.page_tokens);
    const Q4hPlanes planes =
        q4h_planes(page, args.layer, args.page_tokens, args.kv_heads, D);
    const size_t record0 = static_cast<size_t>(kv_head) * args.page_tokens +
                           tile_begin % args.page_tokens;
    const uint8_t* key_rows = uniform_pointer(planes.key_codes + record0 * ROW);
    const uint8_t* key_scales = uniform_pointer(planes.key_scales + record0 * 2u);
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass)
      copy16_to_lds(key_rows + pass * 1024, lane_now * 16u,
                    stage_k_lds + area + pass * 1024);
    copy4_to_lds(key_scales, 4u * (lane_now & 31u), stage_s_lds + area);
  };
  // V_LOADS direct loads: V codes and V scales of a tile.  V row R holds token
  // 16*((R/4)%4) + 4*(R/16) + R%4, so the 16 tokens a lane group reads back
  // transposed sit in 16 consecutive rows; the lane's share of that map is
  // separable from the pass's share.
  auto stage_values = [&](uint32_t tile, uint32_t area) {
    const uint32_t lane_now = fresh_lane_index();
    const uint32_t lane_row = lane_now / kParts;  // row inside a pass
    const uint32_t value_lane_offset =
        (16u * ((lane_row >> 2) & 3u) + 4u * (lane_row >> 4) + (lane_row & 3u)) *
            ROW + (lane_now % kParts) * 16u;
    const uint32_t tile_begin = tile * 64u;
    const void* page = uniform_page(args.page_table, tile_begin / args.page_tokens);
    const Q4hPlanes planes =
        q4h_planes(page, args.layer, args.page_tokens, args.kv_heads, D);
    const size_t record0 = static_cast<size_t>(kv_head) * args.page_tokens +
                           tile_begin % args.page_tokens;
    const uint8_t* value_rows =
        uniform_pointer(planes.value_codes + record0 * ROW);
    const uint8_t* value_scales = uniform_pointer(
        planes.key_scales + record0 * 2u + value_scale_distance);
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
      const uint32_t first_row = pass * kPassRows;
      const uint32_t pass_token = 16u * ((first_row >> 2) & 3u) +
                                  4u * (first_row >> 4) + (first_row & 3u);
      copy16_to_lds(value_rows + pass_token * ROW, value_lane_offset,
                    stage_v_lds + area + pass * 1024);
    }
    copy4_to_lds(value_scales, 4u * (lane_now & 31u), stage_vs_lds + area);
  };
  // The wave's first DEPTH tiles set out; returns how many half tiles (K or V
  // of one tile) that put in flight.
  auto stage_first_tiles = [&]() -> uint32_t {
    uint32_t halves = 0u;
#pragma unroll
    for (int ahead = 0; ahead < DEPTH; ++ahead)
      if (tile_first + ahead < tile_last) {
        stage_keys(tile_first + ahead, ahead * STAGE);
        stage_values(tile_first + ahead, ahead * STAGE);
        halves += 2u;
      }
    return halves;
  };

  // ---- query operands (B side of S = K.Q), built once per workgroup ---------
  // The F32 query row is quantised here to 15 bits and split into two int8
  // planes, q = scale * (128*hi + lo) with hi in [-127,127], lo in [-64,63],
  // so the integer scores carry the query to ~3e-5 relative instead of the
  // 4e-3 of a single Q8 plane.  The operands are published in MFMA order.
  static_assert(RT * KSTEPS <= kSplitWaves, "one wave per operand pair");
  // fused mode: scratch of the per-wave rotary, then the batch's fresh K/V
  // records [K codes | V codes | K scale | V scale] of this KV head
  constexpr int RECORD = D + 16;
  // (the fused launch takes at most 16 rows)
  constexpr int FRESH_ROWS = FUSED ? 16 : 1;
  // at head_dim 256 the rotary scratch lies in the (still empty) staging area
  // and the first tile sets out after the query work: LDS has no room for both
  constexpr bool SCRATCH_IN_STAGE = D == 256;
  __shared__ float rope_scratch[FUSED && !SCRATCH_IN_STAGE ? kSplitWaves * 2 * D : 1];
  __shared__ __attribute__((aligned(16))) uint8_t fresh[FRESH_ROWS * RECORD];
  uint32_t first_cache_position = 0u;
  bool reaches_batch = false;   // some tile of this workgroup holds batch tokens
  if constexpr (FUSED) {
    first_cache_position = args.device_positions ? uniform_word(args.device_positions, 0u)
                                                 : args.first_cache_position;
    float* shared = SCRATCH_IN_STAGE ? reinterpret_cast<float*>(stage_base)
                                     : rope_scratch + wave * (2 * D);
    float* rotated = shared + D;
    const uint32_t half = args.rotary_dim / 2u;
    constexpr int N = D / 64;                       // elements of a row per lane
    constexpr int ROWS_PER_WAVE = RT * 16 / kSplitWaves;
    // Everything the wave will need comes in one round trip: its query rows
    // (matrix rows wave, wave + 8, ...), the batch's K/V row it encodes, norm
    // weights and the rows' (cos, sin).  The loads before the tiles are ones
    // the kernel waits for itself, so that the tiles stay in flight behind
    // them while the rows are rotated and quantised.
    float q_values[ROWS_PER_WAVE][N];
    f32x2 q_entry_raw[ROWS_PER_WAVE][N];
    float weights[2][N];                            // query norm, key norm
    // (without norm weights the loads read the query buffer instead and their
    // values go unused: no branch, no wait of its own)
    const float* q_weight = args.q_weight ? args.q_weight : args.query;
    const float* k_weight = args.k_weight ? args.k_weight : args.query;
    [&]<int... K>(std::integer_sequence<int, K...>) {
      ((weights[0][K] = load_f32_uncounted<256 * K>(uniform_pointer(
            reinterpret_cast<const uint8_t*>(q_weight)), 4u * lane)), ...);
      ((weights[1][K] = load_f32_uncounted<256 * K>(uniform_pointer(
            reinterpret_cast<const uint8_t*>(k_weight)), 4u * lane)), ...);
    }(std::make_integer_sequence<int, N>{});
    // (rows past the batch fetch the last row again; nothing uses the values.
    // Row and head of matrix row wave + 8 item follow from those of the row
    // before, all on the scalar unit)
    uint32_t pair_of_lane[N];
    if ((half & (half - 1u)) == 0u) {
#pragma unroll
      for (int k = 0; k < N; ++k) pair_of_lane[k] = (lane + 64u * k) & (half - 1u);
    } else {
#pragma unroll
      for (int k = 0; k < N; ++k) pair_of_lane[k] = (lane + 64u * k) % half;
    }
    {
      uint32_t row = wave / group;
      uint32_t member = wave % group;
      const uint32_t row_step = kSplitWaves / group;
      const uint32_t member_step = kSplitWaves % group;
#pragma unroll
      for (int item = 0; item < ROWS_PER_WAVE; ++item) {
        const uint32_t fetched_row = min(row, args.rows - 1u);
        const float* source = reinterpret_cast<const float*>(uniform_pointer(
            reinterpret_cast<const uint8_t*>(
                args.query + (fetched_row * args.query_heads + kv_head * group +
                              member) * args.query_stride)));
        const float2* entries = reinterpret_cast<const float2*>(uniform_pointer(
            reinterpret_cast<const uint8_t*>(args.rope_table + fetched_row * half)));
        [&]<int... K>(std::integer_sequence<int, K...>) {
          ((q_values[item][K] = load_f32_uncounted<256 * K>(source, 4u * lane)), ...);
          ((q_entry_raw[item][K] =
                load_f32x2_uncounted(entries, 8u * pair_of_lane[K])), ...);
        }(std::make_integer_sequence<int, N>{});
        member += member_step;
        row += row_step;
        if (member >= group) {
          member -= group;
          ++row;
        }
      }
    }
    uint32_t workgroup_first, workgroup_last, unused;
    wave_tile_range(context_tiles, 64u, args.split_tokens, split, gridDim.y, 0u,
                    workgroup_first, unused, kTailWork);
    wave_tile_range(context_tiles, 64u, args.split_tokens, split, gridDim.y,
                    kSplitWaves - 1u, unused, workgroup_last, kTailWork);
    reaches_batch = workgroup_first < workgroup_last &&
                    workgroup_last * 64u > first_cache_position;
    // the wave's first tiles set out first: the work below hides behind them
    uint32_t halves_in_flight = 0u;
    if (!SCRATCH_IN_STAGE) halves_in_flight = stage_first_tiles();
    // batch rows wave, wave + 8, ... are this wave's to encode (one for the
    // usual batches; the rest, if any, are fetched when their turn comes)
    const bool writes_pages = reaches_batch && workgroup_last == context_tiles;
    float k_values[N], v_values[N];
    float2 k_entry[N];
    const auto fetch_record = [&](uint32_t row) {
      const size_t source = (static_cast<size_t>(row) * args.kv_heads + kv_head) * D;
#pragma unroll
      for (int k = 0; k < N; ++k) {
        const uint32_t index = lane + 64u * k;
        k_values[k] = args.raw_key[source + index];
        v_values[k] = args.raw_value[source + index];
        k_entry[k] = args.rope_table[row * half + pair_of_lane[k]];
      }
    };
    if (reaches_batch && wave < args.rows) {
      fetch_record(wave);
      halves_in_flight = 0u;   // these loads came after the tiles: wait for all
    }
    // where element lane + 64 k of a row goes inside the row's operand bytes:
    // k-step 2 (d / 128) + (d % 32) / 16, lane quad (d % 128) / 32, byte slot
    // (even elements of each half of 8 first, then the odd ones)
    uint32_t piece_of_lane[N];
#pragma unroll
    for (int k = 0; k < N; ++k) {
      const uint32_t index = lane + 64u * k;
      const uint32_t within = index % 128u;
      const uint32_t step = 2u * (index / 128u) + (within % 32u) / 16u;
      const uint32_t j = index % 16u;
      piece_of_lane[k] = step * 2048u + (within / 32u) * 256u + (j & 8u) +
                         ((j & 1u) << 2) + ((j & 7u) >> 1);
    }
    const bool pairs_in_lane = half % 64u == 0u;

    // Rows past the batch go through the same arithmetic as zero rows (zero
    // operands, the smallest scale, the first row's limit): no branch between
    // the rows, so their instruction streams interleave.
    const bool has_q_weight = args.q_weight != nullptr;
    const bool bf16_rounding = args.bf16_activations != 0u;
    // The wave's last row is past the batch in the usual shapes (40 matrix rows
    // in 48 slots): it alone sits behind a branch, which leaves it out then.
    const bool last_item_live =
        wave + kSplitWaves * (ROWS_PER_WAVE - 1) < matrix_rows;
    // loads complete in issue order: the rows, their (cos, sin) and the weights
    // are here once nothing but the tiles issued after them is in flight
    vmem_wait_units<KS_LOADS>(halves_in_flight);
    float2 q_entry[ROWS_PER_WAVE][N];
#pragma unroll
    for (int k = 0; k < N; ++k) {
      tie(weights[0][k]);
      tie(weights[1][k]);
    }
#pragma unroll
    for (int item = 0; item < ROWS_PER_WAVE; ++item)
#pragma unroll
      for (int k = 0; k < N; ++k) {
        tie(q_values[item][k]);
        tie(q_entry_raw[item][k]);
        q_entry[item][k] = make_float2(q_entry_raw[item][k][0], q_entry_raw[item][k][1]);
      }
    const auto quantise_rows = [&](auto rotate) {
#pragma unroll
      for (int item = 0; item < ROWS_PER_WAVE; ++item) {
        const uint32_t matrix_row = wave + kSplitWaves * item;
        if (item == ROWS_PER_WAVE - 1 && !last_item_live) {
          if (lane < KSTEPS * 2u * 4u)
            *reinterpret_cast<uint4*>(
                exchange + ((matrix_row / 16u) * KSTEPS * 2u + lane / 4u) * 1024u +
                (16u * (lane % 4u) + matrix_row % 16u) * 16u) =
                make_uint4(0u, 0u, 0u, 0u);
          if (lane == 0u) {
            exchange_scale[matrix_row] =
                0x1p-100f *
                (1.4426950408889634f / (16.0f * sqrtf(static_cast<float>(D))));
            exchange_limit[matrix_row] = first_context_tokens;
          }
          continue;
        }
        const uint32_t row_tile = matrix_row / 16u;
        const uint32_t column = matrix_row % 16u;
        const bool valid = matrix_row < matrix_rows;
        float source[N];
#pragma unroll
        for (int k = 0; k < N; ++k) source[k] = valid ? q_values[item][k] : 0.0f;
        float row_values[N];
        rotate(source, q_entry[item], row_values);
        float maximum = 0.0f;
#pragma unroll
        for (int k = 0; k < N; ++k) maximum = fmaxf(maximum, fabsf(row_values[k]));
        maximum = wave_max_in_registers(maximum);
        const float scale = fmaxf(maximum * (1.0f / 16319.0f), 0x1p-100f);
        const float inverse = 1.0f / scale;
        uint8_t* row_pieces =
            exchange + row_tile * (KSTEPS * 2048u) + column * 16u;   // wave-uniform
#pragma unroll
        for (int k = 0; k < N; ++k) {
          int quantized = __float2int_rn(row_values[k] * inverse);
          quantized = max(-16319, min(16319, quantized));
          const int high = (quantized + 64) >> 7;  // floor((v + 64) / 128)
          const int low = quantized - (high << 7);
          row_pieces[piece_of_lane[k]] = static_cast<uint8_t>(high);
          row_pieces[piece_of_lane[k] + 1024u] = static_cast<uint8_t>(low);
        }
        if (lane == 0u) {
          exchange_scale[matrix_row] =
              scale *
              (1.4426950408889634f / (16.0f * sqrtf(static_cast<float>(D))));
          exchange_limit[matrix_row] =
              first_context_tokens + (valid ? matrix_row / group : 0u);
        }
      }
    };
    if (pairs_in_lane && !has_q_weight && !bf16_rounding) {
      // the usual case, straight-line: rotary only, both halves of a pair in
      // the lane
      const int shift = static_cast<int>(args.rotary_dim / 128u);
      quantise_rows([&](const float (&x)[N], const float2 (&entry)[N],
                        float (&result)[N]) {
#pragma unroll
        for (int k = 0; k < N; ++k) {
          result[k] = x[k];
          if (k < 2 * shift) {
            float partner = 0.0f;
#pragma unroll
            for (int j = 0; j < N; ++j)
              if (k < shift ? j == k + shift : j + shift == k) partner = x[j];
            const float other = k < shift ? -partner : partner;
            result[k] = __fmaf_rn(x[k], entry[k].x, __fmul_rn(other, entry[k].y));
          }
        }
      });
    } else if (pairs_in_lane) {
      quantise_rows([&](const float (&x)[N], const float2 (&entry)[N],
                        float (&result)[N]) {
        head_norm_rope_in_lane<N>(x, weights[0], has_q_weight, args.rotary_dim, entry,
                                  args.epsilon, bf16_rounding, result, lane);
      });
    } else {
      quantise_rows([&](const float (&x)[N], const float2 (&entry)[N],
                        float (&result)[N]) {
        head_norm_rope_registers<N>(x, weights[0], has_q_weight, args.rotary_dim,
                                    entry, args.epsilon, bf16_rounding, shared,
                                    rotated, lane);
#pragma unroll
        for (int k = 0; k < N; ++k) result[k] = rotated[lane + 64u * k];
        __builtin_amdgcn_wave_barrier();   // `rotated` is reused by the next row
      });
    }
    if (reaches_batch) {
      for (uint32_t row = wave; row < args.rows; row += kSplitWaves) {
        if (row != wave) fetch_record(row);
        uint8_t* record = fresh + row * RECORD;
        head_norm_rope_registers<N>(k_values, weights[1], args.k_weight != nullptr,
                                    args.rotary_dim, k_entry, args.epsilon,
                                    args.bf16_activations != 0u, shared, rotated,
                                    lane);
        q4h_encode_record(rotated, D, record, record + D, lane);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int k = 0; k < N; ++k) shared[lane + 64u * k] = v_values[k];
        __builtin_amdgcn_wave_barrier();
        q4h_encode_record(shared, D, record + ROW, record + D + 2, lane);
        __builtin_amdgcn_wave_barrier();
        if (writes_pages) {
          // the record goes to its page for the steps to come
          const uint32_t position = first_cache_position + row;
          uint8_t* page = static_cast<uint8_t*>(const_cast<void*>(
              args.page_table[position / args.page_tokens]));
          const Q4hPlanes planes =
              q4h_planes(page, args.layer, args.page_tokens, args.kv_heads, D);
          const size_t slot = static_cast<size_t>(kv_head) * args.page_tokens +
                              position % args.page_tokens;
          constexpr uint32_t kWords = ROW / 4u;   // dwords of codes per record
          if (lane < kWords)
            reinterpret_cast<uint32_t*>(
                const_cast<uint8_t*>(planes.key_codes) + slot * ROW)[lane] =
                reinterpret_cast<const uint32_t*>(record)[lane];
          if (lane < kWords)
            reinterpret_cast<uint32_t*>(
                const_cast<uint8_t*>(planes.value_codes) + slot * ROW)[lane] =
                reinterpret_cast<const uint32_t*>(record + ROW)[lane];
          if (lane == 0u)
            *reinterpret_cast<uint16_t*>(
                const_cast<uint8_t*>(planes.key_scales) + slot * 2u) =
                *reinterpret_cast<const uint16_t*>(record + D);
          if (lane == 1u)
            *reinterpret_cast<uint16_t*>(
                const_cast<uint8_t*>(planes.value_scales) + slot * 2u) =
                *reinterpret_cast<const uint16_t*>(record + D + 2);
        }
      }
    }
    if (SCRATCH_IN_STAGE && tile_first < tile_last) {
      // every lane is done with the scratch before the tile lands on it
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_wave_barrier();
      stage_first_tiles();
    }
    // a workgroup that fetched batch records or wrote them to their pages has
    // loads and stores of other kinds in flight: the tile loop counts tiles only
    if (reaches_batch) vmem_wait<0>();
  } else if (args.query_operands) {
    // prepared by the rotary kernel: the planes go straight to LDS, one KiB
    // per wave and load, the scales with them
    constexpr uint32_t kPlanes = RT * KSTEPS * 2;
    const uint32_t lane_now = fresh_lane_index();
    const uint32_t exchange_lds =
        __builtin_amdgcn_readfirstlane(lds_address(exchange));
    const uint8_t* planes = uniform_pointer(
        args.query_operands + static_cast<size_t>(kv_head) * kPlanes * 1024u);
#pragma unroll
    for (uint32_t plane = 0; plane < (kPlanes + kSplitWaves - 1u) / kSplitWaves;
         ++plane) {
      const uint32_t index = plane * kSplitWaves + wave;
      if (index < kPlanes)
        copy16_to_lds(planes + index * 1024u, lane_now * 16u,
                      exchange_lds + index * 1024u);
    }
    if (wave == kSplitWaves - 1u && lane_now < RT * 16u) {
      const uint8_t* scales = uniform_pointer(reinterpret_cast<const uint8_t*>(
          args.query_operand_scales + static_cast<size_t>(kv_head) * RT * 16u));
      copy4_to_lds(scales, lane_now * 4u, exchange_lds + kPlanes * 1024u);
      const uint32_t row = lane_now < matrix_rows ? lane_now / group : 0u;
      exchange_limit[lane_now] = first_context_tokens + row;
    }
  }
  // the wave's first tile sets out before the query work below, which its
  // flight time covers
  uint32_t halves_after_operands = 0u;
  if (!FUSED) halves_after_operands = stage_first_tiles();
  if (FUSED) {
  } else if (args.query_operands) {
    // the operands were asked for before the tiles
    vmem_wait_units<KS_LOADS>(halves_after_operands);
  } else if (wave < static_cast<uint32_t>(RT * KSTEPS)) {
    // wave u builds k-step u % KSTEPS of row tile u / KSTEPS (the row's scale
    // needs the whole row, so every such wave reads all of it)
    const uint32_t rt = wave / KSTEPS;
    const uint32_t step = wave % KSTEPS;
    const uint32_t matrix_row = 16u * rt + col;
    const bool valid = matrix_row < matrix_rows;
    const uint32_t row = valid ? matrix_row / group : 0u;
    const uint32_t head = kv_head * group + (valid ? matrix_row % group : 0u);
    const size_t record = static_cast<size_t>(row) * args.query_heads + head;
    float values[16];
    float maximum = 0.0f;
#pragma unroll
    for (int h = 0; h < KSTEPS; ++h) {
      const uint32_t d0 = 128u * (h / 2) + 32u * quad + 16u * (h % 2);
#pragma unroll
      for (int piece = 0; piece < 4; ++piece) {
        float4 loaded = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (valid)
          loaded = *reinterpret_cast<const float4*>(
              args.query + record * args.query_stride + d0 + 4u * piece);
        if (static_cast<uint32_t>(h) == step) {
          values[4 * piece + 0] = loaded.x;
          values[4 * piece + 1] = loaded.y;
          values[4 * piece + 2] = loaded.z;
          values[4 * piece + 3] = loaded.w;
        }
        maximum = fmaxf(maximum, fmaxf(fmaxf(fabsf(loaded.x), fabsf(loaded.y)),
                                       fmaxf(fabsf(loaded.z), fabsf(loaded.w))));
      }
    }
    maximum = quad_row_max(maximum);
    const float scale = fmaxf(maximum * (1.0f / 16319.0f), 0x1p-100f);
    const float inverse = 1.0f / scale;
    if (quad == 0u && step == 0u) {
      exchange_scale[16 * rt + col] =
          scale * (1.4426950408889634f / (16.0f * sqrtf(static_cast<float>(D))));
      exchange_limit[16 * rt + col] = first_context_tokens + row;
    }
    uint32_t high_bytes[16], low_bytes[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      int quantized = __float2int_rn(values[j] * inverse);
      quantized = max(-16319, min(16319, quantized));
      const int high = (quantized + 64) >> 7;  // floor((v+64)/128)
      const int low = quantized - (high << 7);
      high_bytes[j] = static_cast<uint32_t>(high) & 0xffu;
      low_bytes[j] = static_cast<uint32_t>(low) & 0xffu;
    }
    // byte order inside each 8-element half: even d first, then odd d,
    // matching the order in which the key nibbles are widened
    const int order[16] = {0, 2, 4, 6, 1, 3, 5, 7, 8, 10, 12, 14, 9, 11, 13, 15};
    i32x4 high_operand, low_operand;
#pragma unroll
    for (int word = 0; word < 4; ++word) {
      uint32_t high_word = 0u, low_word = 0u;
#pragma unroll
      for (int byte = 0; byte < 4; ++byte) {
        high_word |= high_bytes[order[4 * word + byte]] << (8 * byte);
        low_word |= low_bytes[order[4 * word + byte]] << (8 * byte);
      }
      high_operand[word] = static_cast<int>(high_word);
      low_operand[word] = static_cast<int>(low_word);
    }
    *reinterpret_cast<i32x4*>(exchange + (wave * 2u + 0u) * 1024u + lane * 16u) =
        high_operand;
    *reinterpret_cast<i32x4*>(exchange + (wave * 2u + 1u) * 1024u + lane * 16u) =
        low_operand;
  }
  __syncthreads();

  // The operands stay in LDS and are re-read for every 16-token sub-tile, and
  // so are the per-row scale (> 0 also for rows past the batch) and token
  // limit: holding them next to the output accumulators would push the kernel
  // into scratch memory.
  const uint8_t* q_operands = exchange + lane * 16u;
  // Scores are kept as t = int_dot * k_scale; the true score in log2 units is
  // t * q_scale, where q_scale (constant per query row, so maxima can be taken
  // over t) carries the query's quantisation step, 1/16 for the widened key
  // nibbles, 1/sqrt(D) and log2(e).

  // per-lane LDS addresses of the staged tile
  // K: lane (token = col, quad) takes 16 bytes of each sub-tile's K row
  // (they start in staging area 0 and change areas with every tile)
  uint32_t key_address = stage_k_lds + col * ROW + 16u * quad;
  // scales of tokens 16*st + 4*quad + i (i = 0..3)
  uint32_t scale_address = stage_s_lds + 8u * quad;
  // (the V scales lie CODES + 256 bytes past the K scales)
  // V: lane (col, quad) supplies LDS row 16*quad + col, i.e. token
  // 16*(col/4) + 4*quad + col%4 of the tile
  uint32_t value_address = stage_v_lds + (16u * quad + col) * ROW;
  uint32_t area = 0u;   // of the tile at hand: 0 or STAGE

  // ---- running state ---------------------------------------------------------
  float running_max[RT];   // in t units
  float running_sum[RT];
  f32x4 out[DT][RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    running_max[rt] = kMaskedMax;
    running_sum[rt] = 0.0f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) out[dt][rt][i] = 0.0f;
  }

  // Loads in flight at the top of an iteration, oldest first: this tile's
  // K+scales, this tile's V.
  for (uint32_t tile = tile_first; tile < tile_last; ++tile) {
    const uint32_t tile_begin = tile * 64u;
    const bool needs_mask = tile_begin + 64u > first_context_tokens;
    const bool has_next = tile + 1u < tile_last;
    // this tile's staging area, and whether the tile DEPTH ahead refills it
    const bool refills = tile + DEPTH < tile_last;
    const uint32_t ahead_units = DEPTH == 2 && has_next ? 2u : 0u;
    uint8_t* const stage_k = stage_base + area;

    // ---- K codes and scales out of LDS ----------------------------------------
    // in flight, oldest first: this tile's K, its V, the next tile's K and V
    vmem_wait_units<KS_LOADS>(1u + ahead_units);
    if constexpr (FUSED) {
      // the batch's own tokens inside this tile, [batch_first, batch_last):
      // their fresh records go over whatever the pages held, once the whole
      // tile has landed (a tile or two per launch pay this wait)
      const uint32_t batch_first = max(first_cache_position, tile_begin);
      const uint32_t batch_last =
          min(first_cache_position + args.rows, tile_begin + 64u);
      if (batch_first < batch_last) {
        vmem_wait<0>();
        const uint32_t lane_now = fresh_lane_index();
        uint8_t* stage_v = stage_k + CODES + 256;
        const uint32_t count = batch_last - batch_first;
#pragma clang loop vectorize(disable) unroll(disable)
        for (uint32_t piece = lane_now; piece < count * kParts; piece += 64u) {
          const uint32_t token = batch_first + piece / kParts;
          const uint32_t part = piece % kParts;
          const uint32_t t = token - tile_begin;
          const uint8_t* record = fresh + (token - first_cache_position) * RECORD;
          *reinterpret_cast<uint4*>(stage_k + t * ROW + part * 16u) =
              *reinterpret_cast<const uint4*>(record + part * 16u);
          // LDS row of token t in the V area: see stage_values
          const uint32_t lds_row = 16u * ((t >> 2) & 3u) + 4u * (t >> 4) + (t & 3u);
          *reinterpret_cast<uint4*>(stage_v + lds_row * ROW + part * 16u) =
              *reinterpret_cast<const uint4*>(record + ROW + part * 16u);
        }
#pragma clang loop vectorize(disable) unroll(disable)
        for (uint32_t index = lane_now; index < count; index += 64u) {
          const uint32_t token = batch_first + index;
          const uint8_t* record = fresh + (token - first_cache_position) * RECORD;
          *reinterpret_cast<uint16_t*>(stage_k + CODES + 2u * (token - tile_begin)) =
              *reinterpret_cast<const uint16_t*>(record + D);
          *reinterpret_cast<uint16_t*>(stage_v + CODES + 2u * (token - tile_begin)) =
              *reinterpret_cast<const uint16_t*>(record + D + 2);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      }
    }
    u32x4 key_raw[4 * (D / 128)];
    u32x2 scale_raw[4];  // K scales of sub-tile st
    [&]<int... I>(std::integer_sequence<int, I...>) {
      ((key_raw[I] = lds_read16<(I / (D / 128)) * 16 * ROW + (I % (D / 128)) * 64>(
            key_address)), ...);
    }(std::make_integer_sequence<int, 4 * (D / 128)>{});
    [&]<int... I>(std::integer_sequence<int, I...>) {
      ((scale_raw[I] = lds_read8<I * 32>(scale_address)), ...);
    }(std::make_integer_sequence<int, 4>{});
    lds_wait(key_raw);
    lds_wait(scale_raw);
    // that half of the staging area is free: fetch the K of the tile that
    // uses it next
    if (refills) stage_keys(tile + DEPTH, area);

    // K nibbles widened to int8 * 16 (sub-tile st, k-step h), scales of tokens
    // 16*st + 4*quad + i
    i32x4 key_operand[4][KSTEPS];
    float k_scale[4][4];
#pragma unroll
    for (int st = 0; st < 4; ++st) {
#pragma unroll
      for (int c = 0; c < D / 128; ++c) {
        const u32x4 x = key_raw[st * (D / 128) + c];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          i32x4 operand;
          operand[0] = static_cast<int>((x[2 * half] << 4) & 0xf0f0f0f0u);
          operand[1] = static_cast<int>(x[2 * half] & 0xf0f0f0f0u);
          operand[2] = static_cast<int>((x[2 * half + 1] << 4) & 0xf0f0f0f0u);
          operand[3] = static_cast<int>(x[2 * half + 1] & 0xf0f0f0f0u);
          key_operand[st][2 * c + half] = operand;
        }
      }
      k_scale[st][0] = f16_bits_to_f32(scale_raw[st][0] & 0xffffu);
      k_scale[st][1] = f16_bits_to_f32(scale_raw[st][0] >> 16);
      k_scale[st][2] = f16_bits_to_f32(scale_raw[st][1] & 0xffffu);
      k_scale[st][3] = f16_bits_to_f32(scale_raw[st][1] >> 16);
    }

    // V scales, folded into the probabilities: pair (u, c) =
    // (scale[token 16*(2u) + 4*quad + c], scale[token 16*(2u+1) + 4*quad + c])
    f16x2 v_scale[2][4];
    // P^T operands (probability times the token's V scale): k-step u covers
    // sub-tiles 2u, 2u+1; register c pairs the tokens (2u, i=c), (2u+1, i=c)
    f16x8 p_operand[RT][2];

    // One row tile at a time: scores, online softmax, probabilities.  A lane
    // owns query row `col` of the row tile and 16 of the 64 tokens.
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      // keeps the compiler from fetching the query operands of all row tiles
      // ahead of time (they would live across the whole tile)
      asm volatile("" ::: "memory");
      i32x4 q_high[KSTEPS], q_low[KSTEPS];
#pragma unroll
      for (int h = 0; h < KSTEPS; ++h) {
        q_high[h] = *reinterpret_cast<const i32x4*>(
            q_operands + ((rt * KSTEPS + h) * 2 + 0) * 1024);
        q_low[h] = *reinterpret_cast<const i32x4*>(
            q_operands + ((rt * KSTEPS + h) * 2 + 1) * 1024);
      }
      const float q_scale = exchange_scale[16 * rt + col];

      // ---- S = K . Q ----------------------------------------------------------
      float score[4][4];
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        i32x4 dot_high = {0, 0, 0, 0};
        i32x4 dot_low = {0, 0, 0, 0};
#pragma unroll
        for (int h = 0; h < KSTEPS; ++h) {
          dot_high = __builtin_amdgcn_mfma_i32_16x16x64_i8(
              key_operand[st][h], q_high[h], dot_high, 0, 0, 0);
          dot_low = __builtin_amdgcn_mfma_i32_16x16x64_i8(
              key_operand[st][h], q_low[h], dot_low, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int dot = (dot_high[i] << 7) + dot_low[i];
          score[st][i] = static_cast<float>(dot) * k_scale[st][i];
        }
      }
      if (needs_mask) {
        // only the tiles that reach past the first row's context get here
        const uint32_t lane_now = fresh_lane_index();
        const uint32_t first_token = tile_begin + 4u * (lane_now >> 4);
        const uint32_t limit = exchange_limit[16 * rt + (lane_now & 15u)];
#pragma unroll
        for (int st = 0; st < 4; ++st)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (first_token + 16u * st + i >= limit) score[st][i] = -INFINITY;
      }

      if (rt == 0) {
        // ---- V scales out of LDS ----------------------------------------------
        // in flight, oldest first: this tile's V, the next tile's K and V,
        // the K just asked for
        vmem_wait_units<KS_LOADS>(ahead_units + (refills ? 1u : 0u));
        u32x2 value_scale_raw[4];
        [&]<int... I>(std::integer_sequence<int, I...>) {
          ((value_scale_raw[I] = lds_read8<I * 32 + CODES + 256>(scale_address)), ...);
        }(std::make_integer_sequence<int, 4>{});
        lds_wait(value_scale_raw);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            uint32_t lo =
                (value_scale_raw[2 * u][c / 2] >> (16 * (c % 2))) & 0xffffu;
            uint32_t hi =
                (value_scale_raw[2 * u + 1][c / 2] >> (16 * (c % 2))) & 0xffffu;
            if (needs_mask) {
              // records no row can see may be uninitialised: keep their scale
              // (any bit pattern) away from the matrix core
              const uint32_t quad_now = fresh_lane_index() >> 4;
              if (tile_begin + 32u * u + 4u * quad_now + c >= last_context) lo = 0u;
              if (tile_begin + 32u * u + 16u + 4u * quad_now + c >= last_context)
                hi = 0u;
            }
            v_scale[u][c] = __builtin_bit_cast(f16x2, lo | (hi << 16));
          }
        }
      }

      // ---- online softmax -----------------------------------------------------
      // The running maximum only follows the tile maximum when that is more
      // than 8 (log2 units) ahead - probabilities then stay below 2^8, harmless
      // in F32 sums and binary16 operands - so the accumulators are rarely
      // rescaled; on a wave's first tile there is nothing to rescale yet.
      float tile_max = score[0][0];
#pragma unroll
      for (int st = 0; st < 4; ++st)
#pragma unroll
        for (int i = 0; i < 4; ++i) tile_max = fmaxf(tile_max, score[st][i]);
      tile_max = quad_row_max(tile_max);
      const bool grew = (tile_max - running_max[rt]) * q_scale > 8.0f;
      if (__builtin_amdgcn_ballot_w64(grew) != 0ull) {
        const float new_max = fmaxf(running_max[rt], tile_max);
        if (tile != tile_first) {
          const float factor =
              __builtin_amdgcn_exp2f((running_max[rt] - new_max) * q_scale);
          running_sum[rt] *= factor;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) out[dt][rt][i] *= factor;
        }
        running_max[rt] = new_max;
      }
      const float offset = -running_max[rt] * q_scale;
      float sum = 0.0f;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const float p0 =
              __builtin_amdgcn_exp2f(fmaf(score[2 * u][c], q_scale, offset));
          const float p1 =
              __builtin_amdgcn_exp2f(fmaf(score[2 * u + 1][c], q_scale, offset));
          sum += p0 + p1;
          f16x2 pair = {static_cast<_Float16>(p0), static_cast<_Float16>(p1)};
          pair *= v_scale[u][c];
          p_operand[rt][u][2 * c] = pair[0];
          p_operand[rt][u][2 * c + 1] = pair[1];
        }
      running_sum[rt] += sum;
    }

    // ---- V codes out of LDS, transposed to d-major ----------------------------
    u32x2 transposed[DT];
    [&]<int... I>(std::integer_sequence<int, I...>) {
      ((transposed[I] = lds_read8_transposed4<I * 8>(value_address)), ...);
    }(std::make_integer_sequence<int, DT>{});
    lds_wait(transposed);
    if (refills) stage_values(tile + DEPTH, area);
    if constexpr (DEPTH == 2) {
      // on to the other staging area
      const uint32_t step = area ? static_cast<uint32_t>(-STAGE) : STAGE;
      key_address += step;
      scale_address += step;
      value_address += step;
      area = STAGE - area;
    }

    // ---- O^T += V^T . P^T -------------------------------------------------------
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        // two's complement nibble -> u = code + 8 (one XOR per 8 nibbles),
        // inserted into the mantissa of a binary16 constant so that the bit
        // pattern is a small integer plus u exactly: 1024 + u for a nibble in
        // bits 0..3 (0x6400, ulp 1), 64 + u for one in bits 4..7 (0x5400, ulp
        // 1/16).  Subtracting the constant plus 8 leaves the signed code.
        const uint32_t x = transposed[dt][u] ^ 0x88888888u;
        const uint32_t y = x >> 8;
        const f16x2 bias_low = {static_cast<_Float16>(-1032.0f),
                                static_cast<_Float16>(-1032.0f)};
        const f16x2 bias_high = {static_cast<_Float16>(-72.0f),
                                 static_cast<_Float16>(-72.0f)};
        const f16x2 e0 = __builtin_bit_cast(
            f16x2, insert_bits(0x000f000fu, x, 0x64006400u)) + bias_low;
        const f16x2 e1 = __builtin_bit_cast(
            f16x2, insert_bits(0x00f000f0u, x, 0x54005400u)) + bias_high;
        const f16x2 e2 = __builtin_bit_cast(
            f16x2, insert_bits(0x000f000fu, y, 0x64006400u)) + bias_low;
        const f16x2 e3 = __builtin_bit_cast(
            f16x2, insert_bits(0x00f000f0u, y, 0x54005400u)) + bias_high;
        f16x8 v_operand;
        v_operand[0] = e0[0]; v_operand[1] = e0[1];
        v_operand[2] = e1[0]; v_operand[3] = e1[1];
        v_operand[4] = e2[0]; v_operand[5] = e2[1];
        v_operand[6] = e3[0]; v_operand[7] = e3[1];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          out[dt][rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
              v_operand, p_operand[rt][u], out[dt][rt], 0, 0, 0);
      }
    }
  }

  // each lane summed only its own tokens; maxima go to true log2 units
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    running_sum[rt] = quad_row_sum(running_sum[rt]);
    running_max[rt] = running_max[rt] > 0.5f * kMaskedMax
                          ? running_max[rt] * exchange_scale[16 * rt + col]
                          : kMaskedMax;
  }

  // ---- merge the eight wave states, write the split partial ------------------
  static_assert(kSplitWaves * kSplitWaves * 1024 <= kSplitWaves * STAGE,
                "merge pool does not fit the staging memory");
  static_assert(kSplitWaves * RT * 64 * 8 <= sizeof(exchange),
                "row summaries do not fit the exchange area");
  const PartialTarget target{args.partial_maxima, args.partial_sums,
                             args.partial_outputs, args.maximum_splits,
                             args.query_heads, kv_head, split, group,
                             matrix_rows};
  merge_wave_states<D, RT>(running_max, running_sum, out,
                           reinterpret_cast<float*>(stage),
                           reinterpret_cast<float2*>(exchange), wave, lane,
                           target);
}

// ---- prompt attention: eight row batches share every cache tile -------------
// A prompt chunk's row batches walk the same cache tiles, and the tile loop
// above is bound by vector instructions, a good part of them the nibble ->
// binary16 conversion of the tile's V codes and the scale handling.  Here a
// workgroup's eight waves each own one row batch (48 matrix rows: quantised
// queries, scores, softmax and accumulators as above), fetch every tile once
// for all of them and convert its V side once: the V operands of a tile lie in
// LDS in matrix-core order, the K scales as F32 and the V scales as the
// binary16 pairs the probabilities are multiplied with, and every wave reads
// them from there (the K codes stay raw: widening them is cheap, and LDS has
// no room for a second copy next to eight batches' query operands).
//
// Per tile t the workgroup meets one barrier.  Between two barriers a wave
//   1. sends its share of later tiles on their way, global -> LDS: waves 0..3
//      a quarter each of the V codes of tile t + 2 (waves 0 and 1 also its K
//      and V scales), waves 4..7 a quarter each of the K codes of tile t + 1,
//   2. converts its share of tile t + 1: V row tile `wave` from the raw codes
//      (read transposed), wave 6 the K scales, wave 7 the V scale pairs,
//   3. runs its batch over tile t.
// The tiles of the workgroup's longest context are dealt evenly over the grid's
// splits; a batch stops at its own last tile.  Every wave writes its batch's
// split partial itself - no states are merged.
constexpr int kPromptBatches = 8;

template <int D>
__global__ __launch_bounds__(kPromptBatches * 64) void q4h_prompt_attention_kernel(
    const SplitArgs args) {
  static_assert(D == 128, "LDS holds eight batches' query operands at 128 only");
  constexpr int RT = 3;
  constexpr int KSTEPS = D / 64;
  constexpr int DT = D / 16;
  constexpr int ROW = D / 2;
  constexpr int CODES = 64 * ROW;
  constexpr int Q_BYTES = RT * KSTEPS * 2 * 1024;   // query operands of a batch
  constexpr int RAW_V = CODES + 512;                // V codes | K scales | V scales
  constexpr int CONV_V = DT * 2 * 1024;             // V operands of a tile
  constexpr int CONV_KS = CONV_V;                   // K scales, F32 per token
  constexpr int CONV_VS = CONV_KS + 256;            // V scale pairs
  constexpr int CONV = CONV_VS + 128;
  __shared__ __attribute__((aligned(16))) uint8_t q_operands_all[kPromptBatches * Q_BYTES];
  __shared__ float q_scales[kPromptBatches * RT * 16];
  __shared__ uint32_t q_limits[kPromptBatches * RT * 16];
  __shared__ __attribute__((aligned(16))) uint8_t converted[2 * CONV];
  __shared__ __attribute__((aligned(16))) uint8_t raw_values[2 * RAW_V];
  __shared__ __attribute__((aligned(16))) uint8_t raw_keys[2 * CODES];

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t col = lane & 15u;
  const uint32_t quad = lane >> 4;
  const uint32_t kv_head = blockIdx.x;
  const uint32_t split = blockIdx.y;
  const uint32_t splits = gridDim.y;
  const uint32_t group = args.query_heads / args.kv_heads;

  // this wave's batch
  const uint32_t batches = (args.rows + args.batch_rows - 1u) / args.batch_rows;
  // (the workgroups with the longest contexts are dispatched first)
  const uint32_t first_batch = (gridDim.z - 1u - blockIdx.z) * kPromptBatches;
  const uint32_t batch = first_batch + wave;
  const bool live = batch < batches;
  const uint32_t first_row = live ? batch * args.batch_rows : 0u;
  const uint32_t batch_rows = live ? min(args.batch_rows, args.rows - first_row) : 0u;
  const uint32_t matrix_rows = batch_rows * group;
  const uint32_t first_context_tokens = args.first_context_tokens + first_row;
  const uint32_t batch_tiles =
      live ? (first_context_tokens + batch_rows - 1u + 63u) / 64u : 0u;
  // the workgroup's tiles: those of its last batch, cut by the grid's splits
  const uint32_t last_batch = min(first_batch + kPromptBatches, batches) - 1u;
  const uint32_t workgroup_context =
      args.first_context_tokens +
      min((last_batch + 1u) * args.batch_rows, args.rows) - 1u;
  const uint32_t workgroup_tiles = (workgroup_context + 63u) / 64u;
  const uint32_t quotient = workgroup_tiles / splits;
  const uint32_t remainder = workgroup_tiles - quotient * splits;
  const uint32_t tile_first = split * quotient + split * remainder / splits;
  const uint32_t tile_last =
      (split + 1u) * quotient + (split + 1u) * remainder / splits;
  // records from here on were never written: their scales stay away from the
  // matrix cores
  const uint32_t launch_context = args.first_context_tokens + args.rows - 1u;

  const uint32_t raw_values_lds =
      __builtin_amdgcn_readfirstlane(lds_address(raw_values));
  const uint32_t raw_keys_lds =
      __builtin_amdgcn_readfirstlane(lds_address(raw_keys));
  const uint32_t value_scale_distance =
      args.page_tokens * args.kv_heads * (ROW + 2u);

  // ---- a wave's share of fetching and converting a tile -----------------------
  // waves 0..3: V codes, LDS rows 16 wave .. + 15 of the permuted tile (row R
  // holds token 16 ((R / 4) % 4) + 4 (R / 16) + R % 4); waves 0 and 1 also the
  // tile's K and V scales (lanes 0..31 fetch tokens 2l, 2l + 1; the others
  // repeat them)
  const auto send_values = [&](uint32_t tile) {
    const uint32_t lane_now = fresh_lane_index();
    const uint32_t lane_row = lane_now >> 2;
    const uint32_t tile_begin = tile * 64u;
    const void* page = uniform_page(args.page_table, tile_begin / args.page_tokens);
    const Q4hPlanes planes =
        q4h_planes(page, args.layer, args.page_tokens, args.kv_heads, D);
    const size_t record0 = static_cast<size_t>(kv_head) * args.page_tokens +
                           tile_begin % args.page_tokens;
    const uint32_t target = raw_values_lds + (tile & 1u) * RAW_V;
    const uint8_t* rows = uniform_pointer(planes.value_codes +
                                          (record0 + 4u * wave) * ROW);
    copy16_to_lds(rows,
                  (16u * ((lane_row >> 2) & 3u) + (lane_row & 3u)) * ROW +
                      (lane_now & 3u) * 16u,
                  target + wave * 1024u);
    if (wave < 2u) {
      const uint8_t* scales = uniform_pointer(
          planes.key_scales + record0 * 2u + wave * value_scale_distance);
      copy4_to_lds(scales, 4u * (lane_now & 31u), target + CODES + wave * 256u);
    }
  };
  // waves 4..7: a quarter of the tile's K codes each
  const auto send_keys = [&](uint32_t tile) {
    const uint32_t lane_now = fresh_lane_index();
    const uint32_t tile_begin = tile * 64u;
    const void* page = uniform_page(args.page_table, tile_begin / args.page_tokens);
    const Q4hPlanes planes =
        q4h_planes(page, args.layer, args.page_tokens, args.kv_heads, D);
    const size_t record0 = static_cast<size_t>(kv_head) * args.page_tokens +
                           tile_begin % args.page_tokens;
    const uint8_t* rows = uniform_pointer(planes.key_codes + record0 * ROW +
                                          (wave - 4u) * 1024u);
    copy16_to_lds(rows, lane_now * 16u,
                  raw_keys_lds + (tile & 1u) * CODES + (wave - 4u) * 1024u);
  };
  const auto convert = [&](uint32_t tile) {
    uint8_t* target = converted + (tile & 1u) * CONV;
    const uint32_t source = raw_values_lds + (tile & 1u) * RAW_V;
    const uint32_t lane_now = fresh_lane_index();
    // V: row tile `wave` of head_dim, both halves of the 64 tokens
    u32x2 transposed;
    {
      const uint32_t address =
          source + (16u * (lane_now >> 4) + (lane_now & 15u)) * ROW + wave * 8u;
      asm volatile("ds_read_b64_tr_b4 %0, %1" : "=v"(transposed) : "v"(address));
    }
    uint32_t first_scale = 0u, second_scale = 0u;
    if (wave == 6u) {
      // K scale of token lane_now
      const uint32_t address = source + CODES + 2u * lane_now;
      asm volatile("ds_read_u16 %0, %1" : "=v"(first_scale) : "v"(address));
    } else if (wave == 7u) {
      // V scales of tokens (32 u + 4 q + c, + 16) for lane = 16 u + 4 q + c < 32
      const uint32_t low_token = 32u * ((lane_now >> 4) & 1u) + (lane_now & 15u);
      const uint32_t address = source + CODES + 256u + 2u * low_token;
      asm volatile("ds_read_u16 %0, %1" : "=v"(first_scale) : "v"(address));
      asm volatile("ds_read_u16 %0, %1 offset:32" : "=v"(second_scale) : "v"(address));
    }
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(transposed), "+v"(first_scale), "+v"(second_scale)
                 :: "memory");
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const uint32_t x = transposed[u] ^ 0x88888888u;
      const uint32_t y = x >> 8;
      const f16x2 bias_low = {static_cast<_Float16>(-1032.0f),
                              static_cast<_Float16>(-1032.0f)};
      const f16x2 bias_high = {static_cast<_Float16>(-72.0f),
                               static_cast<_Float16>(-72.0f)};
      const f16x2 e0 = __builtin_bit_cast(
          f16x2, insert_bits(0x000f000fu, x, 0x64006400u)) + bias_low;
      const f16x2 e1 = __builtin_bit_cast(
          f16x2, insert_bits(0x00f000f0u, x, 0x54005400u)) + bias_high;
      const f16x2 e2 = __builtin_bit_cast(
          f16x2, insert_bits(0x000f000fu, y, 0x64006400u)) + bias_low;
      const f16x2 e3 = __builtin_bit_cast(
          f16x2, insert_bits(0x00f000f0u, y, 0x54005400u)) + bias_high;
      u32x4 operand;
      operand[0] = __builtin_bit_cast(uint32_t, e0);
      operand[1] = __builtin_bit_cast(uint32_t, e1);
      operand[2] = __builtin_bit_cast(uint32_t, e2);
      operand[3] = __builtin_bit_cast(uint32_t, e3);
      *reinterpret_cast<u32x4*>(target + (wave * 2u + u) * 1024u + lane_now * 16u) =
          operand;
    }
    if (wave == 6u) {
      *reinterpret_cast<float*>(target + CONV_KS + lane_now * 4u) =
          f16_bits_to_f32(first_scale);
    } else if (wave == 7u && lane_now < 32u) {
      const uint32_t low_token = 32u * (lane_now >> 4) + (lane_now & 15u);
      const uint32_t tile_begin = tile * 64u;
      if (tile_begin + low_token >= launch_context) first_scale = 0u;
      if (tile_begin + low_token + 16u >= launch_context) second_scale = 0u;
      *reinterpret_cast<uint32_t*>(target + CONV_VS + lane_now * 4u) =
          first_scale | (second_scale << 16);
    }
  };

  // ---- the first tiles set out, the queries are quantised meanwhile -----------
  const bool any_tile = tile_first < tile_last;
  if (any_tile) {
    if (wave < 4u) send_values(tile_first);
    else send_keys(tile_first);
  }
  uint8_t* q_operands_mine = q_operands_all + wave * Q_BYTES;
  float* exchange_scale = q_scales + wave * RT * 16;
  uint32_t* exchange_limit = q_limits + wave * RT * 16;
  if (live) {
#pragma unroll 1
    for (uint32_t pair = 0; pair < static_cast<uint32_t>(RT * KSTEPS); ++pair) {
      // k-step pair % KSTEPS of row tile pair / KSTEPS, as in the split kernel
      const uint32_t rt = pair / KSTEPS;
      const uint32_t step = pair % KSTEPS;
      const uint32_t matrix_row = 16u * rt + col;
      const bool valid = matrix_row < matrix_rows;
      const uint32_t row = valid ? matrix_row / group : 0u;
      const uint32_t head = kv_head * group + (valid ? matrix_row % group : 0u);
      const size_t record =
          static_cast<size_t>(first_row + row) * args.query_heads + head;
      float values[16];
      float maximum = 0.0f;
#pragma unroll
      for (int h = 0; h < KSTEPS; ++h) {
        const uint32_t d0 = 128u * (h / 2) + 32u * quad + 16u * (h % 2);
#pragma unroll
        for (int piece = 0; piece < 4; ++piece) {
          float4 loaded = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
          if (valid)
            loaded = *reinterpret_cast<const float4*>(
                args.query + record * args.query_stride + d0 + 4u * piece);
          if (static_cast<uint32_t>(h) == step) {
            values[4 * piece + 0] = loaded.x;
            values[4 * piece + 1] = loaded.y;
            values[4 * piece + 2] = loaded.z;
            values[4 * piece + 3] = loaded.w;
          }
          maximum = fmaxf(maximum, fmaxf(fmaxf(fabsf(loaded.x), fabsf(loaded.y)),
                                         fmaxf(fabsf(loaded.z), fabsf(loaded.w))));
        }
      }
      maximum = quad_row_max(maximum);
      const float scale = fmaxf(maximum * (1.0f / 16319.0f), 0x1p-100f);
      const float inverse = 1.0f / scale;
      if (quad == 0u && step == 0u) {
        exchange_scale[16 * rt + col] =
            scale * (1.4426950408889634f / (16.0f * sqrtf(static_cast<float>(D))));
        exchange_limit[16 * rt + col] = first_context_tokens + row;
      }
      uint32_t high_bytes[16], low_bytes[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        int quantized = __float2int_rn(values[j] * inverse);
        quantized = max(-16319, min(16319, quantized));
        const int high = (quantized + 64) >> 7;
        const int low = quantized - (high << 7);
        high_bytes[j] = static_cast<uint32_t>(high) & 0xffu;
        low_bytes[j] = static_cast<uint32_t>(low) & 0xffu;
      }
      const int order[16] = {0, 2, 4, 6, 1, 3, 5, 7, 8, 10, 12, 14, 9, 11, 13, 15};
      i32x4 high_operand, low_operand;
#pragma unroll
      for (int word = 0; word < 4; ++word) {
        uint32_t high_word = 0u, low_word = 0u;
#pragma unroll
        for (int byte = 0; byte < 4; ++byte) {
          high_word |= high_bytes[order[4 * word + byte]] << (8 * byte);
          low_word |= low_bytes[order[4 * word + byte]] << (8 * byte);
        }
        high_operand[word] = static_cast<int>(high_word);
        low_operand[word] = static_cast<int>(low_word);
      }
      *reinterpret_cast<i32x4*>(q_operands_mine + (pair * 2u + 0u) * 1024u +
                                lane * 16u) = high_operand;
      *reinterpret_cast<i32x4*>(q_operands_mine + (pair * 2u + 1u) * 1024u +
                                lane * 16u) = low_operand;
    }
  }
  vmem_wait<0>();
  __syncthreads();   // the first tile's raw codes and scales are in LDS
  if (any_tile) {
    if (wave < 4u && tile_first + 1u < tile_last) send_values(tile_first + 1u);
    convert(tile_first);
  }
  vmem_wait<0>();
  __syncthreads();   // V operands of the first tile, raw V of the second

  const uint8_t* q_operands = q_operands_mine + lane * 16u;
  float running_max[RT];
  float running_sum[RT];
  f32x4 out[DT][RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    running_max[rt] = kMaskedMax;
    running_sum[rt] = 0.0f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) out[dt][rt][i] = 0.0f;
  }

  for (uint32_t tile = tile_first; tile < tile_last; ++tile) {
    if (wave < 4u) {
      if (tile + 2u < tile_last) send_values(tile + 2u);
    } else if (tile + 1u < tile_last) {
      send_keys(tile + 1u);
    }
    if (tile + 1u < tile_last) convert(tile + 1u);
    if (tile < batch_tiles) {
      const uint32_t tile_begin = tile * 64u;
      const bool needs_mask = tile_begin + 64u > first_context_tokens;
      const uint8_t* operands = converted + (tile & 1u) * CONV;
      // K codes out of LDS (raw), widened to int8 * 16
      u32x4 key_raw[4];
      {
        const uint32_t key_address =
            raw_keys_lds + (tile & 1u) * CODES + col * ROW + 16u * quad;
        key_raw[0] = lds_read16<0 * 16 * ROW>(key_address);
        key_raw[1] = lds_read16<1 * 16 * ROW>(key_address);
        key_raw[2] = lds_read16<2 * 16 * ROW>(key_address);
        key_raw[3] = lds_read16<3 * 16 * ROW>(key_address);
        lds_wait(key_raw);
      }
      i32x4 key_operand[4][KSTEPS];
      float k_scale[4][4];
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        const u32x4 x = key_raw[st];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          i32x4 operand;
          operand[0] = static_cast<int>((x[2 * half] << 4) & 0xf0f0f0f0u);
          operand[1] = static_cast<int>(x[2 * half] & 0xf0f0f0f0u);
          operand[2] = static_cast<int>((x[2 * half + 1] << 4) & 0xf0f0f0f0u);
          operand[3] = static_cast<int>(x[2 * half + 1] & 0xf0f0f0f0u);
          key_operand[st][half] = operand;
        }
        const float4 scales = *reinterpret_cast<const float4*>(
            operands + CONV_KS + (16u * st + 4u * quad) * 4u);
        k_scale[st][0] = scales.x; k_scale[st][1] = scales.y;
        k_scale[st][2] = scales.z; k_scale[st][3] = scales.w;
      }
      f16x2 v_scale[2][4];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const uint4 pairs = *reinterpret_cast<const uint4*>(
            operands + CONV_VS + (16u * u + 4u * quad) * 4u);
        v_scale[u][0] = __builtin_bit_cast(f16x2, pairs.x);
        v_scale[u][1] = __builtin_bit_cast(f16x2, pairs.y);
        v_scale[u][2] = __builtin_bit_cast(f16x2, pairs.z);
        v_scale[u][3] = __builtin_bit_cast(f16x2, pairs.w);
      }
      f16x8 p_operand[RT][2];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        asm volatile("" ::: "memory");
        i32x4 q_high[KSTEPS], q_low[KSTEPS];
#pragma unroll
        for (int h = 0; h < KSTEPS; ++h) {
          q_high[h] = *reinterpret_cast<const i32x4*>(
              q_operands + ((rt * KSTEPS + h) * 2 + 0) * 1024);
          q_low[h] = *reinterpret_cast<const i32x4*>(
              q_operands + ((rt * KSTEPS + h) * 2 + 1) * 1024);
        }
        const float q_scale = exchange_scale[16 * rt + col];
        float score[4][4];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
          i32x4 dot_high = {0, 0, 0, 0};
          i32x4 dot_low = {0, 0, 0, 0};
#pragma unroll
          for (int h = 0; h < KSTEPS; ++h) {
            dot_high = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                key_operand[st][h], q_high[h], dot_high, 0, 0, 0);
            dot_low = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                key_operand[st][h], q_low[h], dot_low, 0, 0, 0);
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int dot = (dot_high[i] << 7) + dot_low[i];
            score[st][i] = static_cast<float>(dot) * k_scale[st][i];
          }
        }
        if (needs_mask) {
          const uint32_t first_token = tile_begin + 4u * quad;
          const uint32_t limit = exchange_limit[16 * rt + col];
#pragma unroll
          for (int st = 0; st < 4; ++st)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (first_token + 16u * st + i >= limit) score[st][i] = -INFINITY;
        }
        // online softmax, as in the split kernel
        float tile_max = score[0][0];
#pragma unroll
        for (int st = 0; st < 4; ++st)
#pragma unroll
          for (int i = 0; i < 4; ++i) tile_max = fmaxf(tile_max, score[st][i]);
        tile_max = quad_row_max(tile_max);
        const bool grew = (tile_max - running_max[rt]) * q_scale > 8.0f;
        if (__builtin_amdgcn_ballot_w64(grew) != 0ull) {
          const float new_max = fmaxf(running_max[rt], tile_max);
          if (tile != tile_first) {
            const float factor =
                __builtin_amdgcn_exp2f((running_max[rt] - new_max) * q_scale);
            running_sum[rt] *= factor;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
              for (int i = 0; i < 4; ++i) out[dt][rt][i] *= factor;
          }
          running_max[rt] = new_max;
        }
        const float offset = -running_max[rt] * q_scale;
        float sum = 0.0f;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const float p0 =
                __builtin_amdgcn_exp2f(fmaf(score[2 * u][c], q_scale, offset));
            const float p1 =
                __builtin_amdgcn_exp2f(fmaf(score[2 * u + 1][c], q_scale, offset));
            sum += p0 + p1;
            f16x2 pair = {static_cast<_Float16>(p0), static_cast<_Float16>(p1)};
            pair *= v_scale[u][c];
            p_operand[rt][u][2 * c] = pair[0];
            p_operand[rt][u][2 * c + 1] = pair[1];
          }
        running_sum[rt] += sum;
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const f16x8 v_operand = *reinterpret_cast<const f16x8*>(
              operands + (dt * 2 + u) * 1024 + lane * 16u);
#pragma unroll
          for (int rt = 0; rt < RT; ++rt)
            out[dt][rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                v_operand, p_operand[rt][u], out[dt][rt], 0, 0, 0);
        }
      }
    }
    vmem_wait<0>();
    __syncthreads();
  }
  if (!live) return;

  // ---- the batch's split partial ------------------------------------------------
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    running_sum[rt] = quad_row_sum(running_sum[rt]);
    running_max[rt] = running_max[rt] > 0.5f * kMaskedMax
                          ? running_max[rt] * exchange_scale[16 * rt + col]
                          : kMaskedMax;
    const uint32_t matrix_row = 16u * rt + col;
    if (matrix_row >= matrix_rows) continue;
    const uint32_t row = first_row + matrix_row / group;
    const uint32_t head = kv_head * group + matrix_row % group;
    const size_t partial =
        (static_cast<size_t>(row) * args.maximum_splits + split) * args.query_heads +
        head;
    if (quad == 0u) {
      args.partial_maxima[partial] = running_max[rt];
      args.partial_sums[partial] = running_sum[rt];
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      *reinterpret_cast<f32x4*>(args.partial_outputs + partial * D + 16u * dt +
                                4u * quad) = out[dt][rt];
  }
}

// Split-K merge (maxima in log2 units), optional sigmoid output gate.
// One workgroup per (query head, row), one thread per output dimension.  The
// per-split weights exp2(m_s - M) are computed once, cooperatively, into LDS;
// the accumulation over splits then has independent loads that pipeline.
constexpr uint32_t kCombineSplitCapacity = 2048;

__global__ void attention_combine_kernel(
    const float* query, uint32_t query_stride, int output_gated,
    const float* partial_maxima, const float* partial_sums,
    const float* partial_outputs, void* output, uint32_t output_kind,
    uint32_t first_context_tokens, uint32_t maximum_splits,
    uint32_t split_tokens, uint32_t query_heads, uint32_t head_dim,
    const uint32_t* device_positions) {
  __shared__ float weights[kCombineSplitCapacity];
  __shared__ float scratch[4];
  if (device_positions)
    first_context_tokens = uniform_word(device_positions, 2u);
  const uint32_t head = blockIdx.x;
  const uint32_t row = blockIdx.y;
  const uint32_t dimension = threadIdx.x;
  // balanced launches (split_tokens == 0) use every split
  const uint32_t active =
      split_tokens ? (first_context_tokens + row + split_tokens - 1u) / split_tokens
                   : maximum_splits;
  const size_t first_partial =
      static_cast<size_t>(row) * maximum_splits * query_heads + head;
  // The first kCombinePrefetch partial outputs are fetched before anything
  // depends on them, so that they travel together with the maxima and sums.
  constexpr uint32_t kCombinePrefetch = 32;
  // (wave-uniform row address + the thread's dimension: the address arithmetic
  // stays on the scalar unit and no load waits for another)
  const float* partial_rows = partial_outputs + first_partial * head_dim;
  const uint32_t stride = query_heads * head_dim;
  const float* source = partial_rows + dimension;
  float fetched[kCombinePrefetch];
#pragma unroll
  for (uint32_t split = 0; split < kCombinePrefetch; ++split) {
    // past the last split: that split once more (finite), weighted by zero
    const float* row_of_split =
        partial_rows + static_cast<size_t>(min(split, active - 1u)) * stride;
    fetched[split] = row_of_split[dimension];
  }
  const size_t record = static_cast<size_t>(row) * query_heads + head;
  if (active <= kCombinePrefetch) {
    // Few splits: every wave takes one split per lane, so maximum, weights and
    // their sum come from lane exchanges alone and everything the result needs
    // is requested in one round trip.
    const uint32_t lane = threadIdx.x & 63u;
    const size_t partial = first_partial + static_cast<size_t>(lane) * query_heads;
    const float split_max = lane < active ? partial_maxima[partial] : kMaskedMax;
    const float split_sum = lane < active ? partial_sums[partial] : 0.0f;
    float gate = 0.0f;
    if (output_gated) gate = query[record * query_stride + head_dim + dimension];
    const float maximum = wave_max(split_max);
    const float weight = __builtin_amdgcn_exp2f(split_max - maximum);
    const float sum = wave_sum(split_sum * weight);
    float result = 0.0f;
#pragma unroll
    for (uint32_t split = 0; split < kCombinePrefetch; ++split)
      result = fmaf(fetched[split],
                    __uint_as_float(__builtin_amdgcn_readlane(
                        __float_as_uint(weight), split)),
                    result);
    result /= sum;
    if (output_gated) result *= 1.0f / (1.0f + expf(-gate));
    const size_t index = record * head_dim + dimension;
    if (output_kind == QLLM_OUT_BF16)
      static_cast<uint16_t*>(output)[index] =
          static_cast<uint16_t>(f32_to_bf16_bits(result));
    else
      static_cast<float*>(output)[index] = result;
    return;
  }
  float local_max = kMaskedMax;
  for (uint32_t split = threadIdx.x; split < active; split += blockDim.x)
    local_max = fmaxf(local_max,
                      partial_maxima[first_partial +
                                     static_cast<size_t>(split) * query_heads]);
  const float maximum = block_max(local_max, scratch);
  float local_sum = 0.0f;
  for (uint32_t split = threadIdx.x; split < active; split += blockDim.x) {
    const size_t partial = first_partial + static_cast<size_t>(split) * query_heads;
    const float weight =
        __builtin_amdgcn_exp2f(partial_maxima[partial] - maximum);
    weights[split] = weight;
    local_sum += partial_sums[partial] * weight;
  }
  const float sum = block_sum(local_sum, scratch);  // also publishes weights[]
  float result = 0.0f;
#pragma unroll
  for (uint32_t split = 0; split < kCombinePrefetch; ++split)
    if (split < active) result = fmaf(fetched[split], weights[split], result);
  for (uint32_t split = kCombinePrefetch; split < active; ++split)
    result = fmaf(source[static_cast<size_t>(split) * stride], weights[split], result);
  result /= sum;
  if (output_gated) {
    const float gate = query[record * query_stride + head_dim + dimension];
    result *= 1.0f / (1.0f + expf(-gate));
  }
  const size_t index = record * head_dim + dimension;
  if (output_kind == QLLM_OUT_BF16)
    static_cast<uint16_t*>(output)[index] =
        static_cast<uint16_t>(f32_to_bf16_bits(result));
  else
    static_cast<float*>(output)[index] = result;
}

// The combine of a launch with a single split (the prompt's chunks): the
// split's weight is one, so the result is its output over its sum - the same
// operations as above, four dimensions per thread and no per-split loads.
__global__ __launch_bounds__(256) void attention_single_split_kernel(
    const float* query, uint32_t query_stride, int output_gated,
    const float* partial_sums, const float* partial_outputs, void* output,
    uint32_t output_kind, uint32_t head_dim, size_t elements) {
  const size_t index =
      (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4u;
  if (index >= elements) return;
  const size_t record = index / head_dim;
  const uint32_t dimension = static_cast<uint32_t>(index - record * head_dim);
  const float4 partial = *reinterpret_cast<const float4*>(partial_outputs + index);
  const float sum = partial_sums[record];
  float result[4] = {partial.x / sum, partial.y / sum, partial.z / sum,
                     partial.w / sum};
  if (output_gated) {
    const float4 gate = *reinterpret_cast<const float4*>(
        query + record * query_stride + head_dim + dimension);
    result[0] *= 1.0f / (1.0f + expf(-gate.x));
    result[1] *= 1.0f / (1.0f + expf(-gate.y));
    result[2] *= 1.0f / (1.0f + expf(-gate.z));
    result[3] *= 1.0f / (1.0f + expf(-gate.w));
  }
  if (output_kind == QLLM_OUT_BF16) {
    uint2 packed;
    packed.x = f32_to_bf16_bits(result[0]) | (f32_to_bf16_bits(result[1]) << 16);
    packed.y = f32_to_bf16_bits(result[2]) | (f32_to_bf16_bits(result[3]) << 16);
    *reinterpret_cast<uint2*>(static_cast<uint16_t*>(output) + index) = packed;
  } else {
    *reinterpret_cast<float4*>(static_cast<float*>(output) + index) =
        make_float4(result[0], result[1], result[2], result[3]);
  }
}

// ---- K/V store ----------------------------------------------------------------

__global__ __launch_bounds__(64) void q4h_store_kernel(
    const float* key, const float* value, const void* const* page_table,
    uint32_t layer, uint32_t page_tokens, uint32_t first_cache_position,
    uint32_t kv_heads, uint32_t head_dim) {
  const uint32_t kv_head = blockIdx.x;
  const uint32_t row = blockIdx.y;
  const uint32_t lane = threadIdx.x;
  const uint32_t position = first_cache_position + row;
  uint8_t* page = static_cast<uint8_t*>(
      const_cast<void*>(page_table[position / page_tokens]));
  const Q4hPlanes planes =
      q4h_planes(page, layer, page_tokens, kv_heads, head_dim);
  const size_t record =
      static_cast<size_t>(kv_head) * page_tokens + position % page_tokens;
  const size_t source = (static_cast<size_t>(row) * kv_heads + kv_head) * head_dim;
  q4h_encode_record(key + source, head_dim,
                    const_cast<uint8_t*>(planes.key_codes) + record * (head_dim / 2u),
                    const_cast<uint8_t*>(planes.key_scales) + record * 2u, lane);
  q4h_encode_record(value + source, head_dim,
                    const_cast<uint8_t*>(planes.value_codes) + record * (head_dim / 2u),
                    const_cast<uint8_t*>(planes.value_scales) + record * 2u, lane);
}

// grid (query_heads + kv_heads, rows): blocks [0, query_heads) rotate a query
// head, the others rotate a key head and encode that K/V record.
__global__ __launch_bounds__(64) void qkv_rope_q4h_kernel(
    float* query, uint32_t query_stride, float* key, const float* value,
    const float* q_weight, const float* k_weight,
    const void* const* page_table, uint32_t layer, uint32_t page_tokens,
    uint32_t first_cache_position, uint32_t first_rotary_position,
    uint32_t query_heads, uint32_t kv_heads, uint32_t head_dim,
    uint32_t rotary_dim, float epsilon, float theta, bool bf16_activations,
    const uint32_t* device_positions, const float* partials,
    uint32_t partial_count, uint32_t rows, uint8_t* operands,
    float* operand_scales, const void* const* q8_page_table = nullptr,
    size_t q8_page_offset = 0u) {
  __shared__ float shared[256];
  __shared__ float rotated[256];
  if (device_positions) {
    first_cache_position = uniform_word(device_positions, 0u);
    first_rotary_position = uniform_word(device_positions, 1u);
  }
  // grid layer y takes rows y, y + gridDim.y, ... (one row each for a verify
  // step; a prompt chunk's thousands of rows go eight to a block)
  const auto process = [&](const uint32_t row) {
  const uint32_t lane = threadIdx.x;
  if (partials) {
    // The projection arrived as K-split partials f32 [partial_count][rows]
    // [q rows | k rows | v rows]: this block's slice of query (with its gate
    // half, if any), or of key and value, is summed in index order first.
    const uint32_t query_rows = query_heads * query_stride;
    const uint32_t kv_rows = kv_heads * head_dim;
    const size_t width = static_cast<size_t>(query_rows) + 2u * kv_rows;
    const size_t slab = static_cast<size_t>(rows) * width;
    const float* source = partials + static_cast<size_t>(row) * width;
    if (blockIdx.x < query_heads) {
      const uint32_t first = blockIdx.x * query_stride;
      float* q = query + static_cast<size_t>(row) * query_rows + first;
      for (uint32_t index = lane; index < query_stride; index += 64u) {
        float sum = source[first + index];
        for (uint32_t part = 1; part < partial_count; ++part)
          sum += source[part * slab + first + index];
        q[index] = sum;
      }
    } else {
      const uint32_t first = (blockIdx.x - query_heads) * head_dim;
      float* k = key + static_cast<size_t>(row) * kv_rows + first;
      float* v = const_cast<float*>(value) + static_cast<size_t>(row) * kv_rows + first;
      for (uint32_t index = lane; index < head_dim; index += 64u) {
        float k_sum = source[query_rows + first + index];
        float v_sum = source[query_rows + kv_rows + first + index];
        for (uint32_t part = 1; part < partial_count; ++part) {
          k_sum += source[part * slab + query_rows + first + index];
          v_sum += source[part * slab + query_rows + kv_rows + first + index];
        }
        k[index] = k_sum;
        v[index] = v_sum;
      }
    }
    __syncthreads();   // one wave: its stores are visible to all its lanes
  }
  const uint32_t rotary_position = first_rotary_position + row;
  if (blockIdx.x < query_heads) {
    const uint32_t head = blockIdx.x;
    float* q =
        query + (static_cast<size_t>(row) * query_heads + head) * query_stride;
    head_norm_rope(q, q_weight, head_dim, rotary_dim, rotary_position, epsilon,
                   theta, bf16_activations, shared, rotated, lane);
    if (!operands) return;
    // The attention kernel's query operands (same arithmetic as its own
    // quantisation): 15 bits against the row's largest magnitude, split into
    // a high and a low int8 plane, each byte dropped where the matrix core
    // wants it.  Element d of the row belongs to k-step h = 2 (d / 128) +
    // (d % 32) / 16, lane quad (d % 128) / 32, and inside the lane's 16 bytes
    // to slot (j < 8: even j first, then odd j; likewise for j >= 8), j = d % 16.
    const uint32_t group = query_heads / kv_heads;
    const uint32_t matrix_row = row * group + head % group;
    const uint32_t row_tile = matrix_row / 16u;
    const uint32_t column = matrix_row % 16u;
    const uint32_t k_steps = head_dim / 64u;
    const uint32_t row_tiles = q4h_row_tiles(rows, group);
    float maximum = 0.0f;
    for (uint32_t index = lane; index < head_dim; index += 64u)
      maximum = fmaxf(maximum, fabsf(rotated[index]));
    maximum = wave_max(maximum);
    const float scale = fmaxf(maximum * (1.0f / 16319.0f), 0x1p-100f);
    const float inverse = 1.0f / scale;
    uint8_t* planes = operands + (head / group) *
                                     q4h_operand_plane_bytes(row_tiles, head_dim);
    for (uint32_t index = lane; index < head_dim; index += 64u) {
      int quantized = __float2int_rn(rotated[index] * inverse);
      quantized = max(-16319, min(16319, quantized));
      const int high = (quantized + 64) >> 7;  // floor((v + 64) / 128)
      const int low = quantized - (high << 7);
      const uint32_t within = index % 128u;
      const uint32_t step = 2u * (index / 128u) + (within % 32u) / 16u;
      const uint32_t quad = within / 32u;
      const uint32_t j = index % 16u;
      const uint32_t slot = (j & 8u) + ((j & 1u) << 2) + ((j & 7u) >> 1);
      uint8_t* piece = planes +
                       static_cast<size_t>(row_tile * k_steps + step) * 2048u +
                       (16u * quad + column) * 16u + slot;
      piece[0] = static_cast<uint8_t>(high);
      piece[1024] = static_cast<uint8_t>(low);
    }
    if (lane == 0u)
      operand_scales[(head / group) * row_tiles * 16u + matrix_row] =
          scale * (1.4426950408889634f /
                   (16.0f * sqrtf(static_cast<float>(head_dim))));
    return;
  }
  const uint32_t head = blockIdx.x - query_heads;
  float* k = key + (static_cast<size_t>(row) * kv_heads + head) * head_dim;
  head_norm_rope(k, k_weight, head_dim, rotary_dim, rotary_position, epsilon,
                 theta, bf16_activations, shared, rotated, lane);
  if (q8_page_table) {
    // the proposer's Q8 cache: the rotated key and the value of this (row, kv
    // head) as Q8 records, what a separate store launch would write
    const uint32_t position = first_cache_position + row;
    uint8_t* layer_base = static_cast<uint8_t*>(const_cast<void*>(
                              q8_page_table[position / page_tokens])) + q8_page_offset;
    __syncthreads();   // `rotated` is complete (one wave)
    q8_encode_record(rotated, head_dim, layer_base, 0u, position % page_tokens, head,
                     kv_heads, page_tokens, lane);
    q8_encode_record(value + (static_cast<size_t>(row) * kv_heads + head) * head_dim,
                     head_dim, layer_base, 1u, position % page_tokens, head, kv_heads,
                     page_tokens, lane);
    return;
  }
  if (!page_table) return;  // rotary only; the caller stores K/V itself
  const uint32_t position = first_cache_position + row;
  uint8_t* page = static_cast<uint8_t*>(
      const_cast<void*>(page_table[position / page_tokens]));
  const Q4hPlanes planes =
      q4h_planes(page, layer, page_tokens, kv_heads, head_dim);
  const size_t record =
      static_cast<size_t>(head) * page_tokens + position % page_tokens;
  q4h_encode_record(rotated, head_dim,
                    const_cast<uint8_t*>(planes.key_codes) + record * (head_dim / 2u),
                    const_cast<uint8_t*>(planes.key_scales) + record * 2u, lane);
  q4h_encode_record(value + (static_cast<size_t>(row) * kv_heads + head) * head_dim,
                    head_dim,
                    const_cast<uint8_t*>(planes.value_codes) + record * (head_dim / 2u),
                    const_cast<uint8_t*>(planes.value_scales) + record * 2u, lane);
  };
  for (uint32_t row = blockIdx.y; row < rows; row += gridDim.y) {
    process(row);
    __syncthreads();   // the scratch rows are free again
  }
}

// transformer_kernels.cu:4391-4416
__global__ __launch_bounds__(64) void quantize_queries_q8_kernel(
    const float* query, uint32_t query_stride, int8_t* q8, float* scales,
    uint32_t query_heads, uint32_t head_dim) {
  const uint32_t head = blockIdx.x;
  const uint32_t row = blockIdx.y;
  const uint32_t lane = threadIdx.x;
  const size_t record = static_cast<size_t>(row) * query_heads + head;
  const float* source = query + record * query_stride;
  float maximum = 0.0f;
  for (uint32_t index = lane; index < head_dim; index += 64u)
    maximum = fmaxf(maximum, fabsf(source[index]));
  maximum = wave_max(maximum);
  const float scale = fmaxf(__fdiv_rn(maximum, 127.0f), 0x1p-24f);
  if (lane == 0u) scales[record] = scale;
  for (uint32_t index = lane; index < head_dim; index += 64u) {
    const int quantized =
        max(-127, min(127, __float2int_rn(__fdiv_rn(source[index], scale))));
    q8[record * head_dim + index] = static_cast<int8_t>(quantized);
  }
}

template <int D, bool FUSED = false>
int32_t launch_split(const SplitArgs& args, uint32_t row_tiles, dim3 grid,
                     hipStream_t stream) {
  const size_t lds = 0;  // all LDS of the split kernel is static
  switch (row_tiles) {
    case 1:
      q4h_attention_split_kernel<D, 1, FUSED>
          <<<grid, kSplitWaves * 64, lds, stream>>>(args);
      break;
    case 2:
      q4h_attention_split_kernel<D, 2, FUSED>
          <<<grid, kSplitWaves * 64, lds, stream>>>(args);
      break;
    default:
      if constexpr (D == 128) {
        q4h_attention_split_kernel<D, 3, FUSED>
            <<<grid, kSplitWaves * 64, lds, stream>>>(args);
        break;
      } else {
        return fail(QLLM_INVALID_ARGUMENT,
                    "Q4H attention: three row tiles need head_dim 128");
      }
  }
  return launched("Q4H attention split");
}

}  // namespace

// shared with the exact-F16 path
int32_t launch_attention_combine(const float* query, uint32_t query_stride,
                                 int output_gated, const float* partial_maxima,
                                 const float* partial_sums,
                                 const float* partial_outputs, void* output,
                                 uint32_t output_kind,
                                 uint32_t first_context_tokens,
                                 uint32_t maximum_splits, uint32_t split_tokens,
                                 uint32_t rows, uint32_t query_heads,
                                 uint32_t head_dim,
                                 const uint32_t* device_positions,
                                 hipStream_t stream) {
  if (maximum_splits == 1u && !split_tokens && head_dim % 4u == 0u &&
      query_stride % 4u == 0u && !(reinterpret_cast<uintptr_t>(query) & 15u)) {
    const size_t elements = static_cast<size_t>(rows) * query_heads * head_dim;
    attention_single_split_kernel<<<static_cast<unsigned>((elements / 4u + 255u) / 256u),
                                    256, 0, stream>>>(
        query, query_stride, output_gated, partial_sums, partial_outputs, output,
        output_kind, head_dim, elements);
    return launched("attention single-split combine");
  }
  const dim3 grid(query_heads, rows);
  attention_combine_kernel<<<grid, head_dim, 0, stream>>>(
      query, query_stride, output_gated, partial_maxima, partial_sums,
      partial_outputs, output, output_kind, first_context_tokens,
      maximum_splits, split_tokens, query_heads, head_dim, device_positions);
  return launched("attention split combine");
}

// grid layers of the rotary kernels: a block per row up to 64 rows, beyond
// that eight rows per block (a block is one wave; hundreds of thousands of
// them cost more to dispatch than to run)
inline uint32_t rope_grid_rows(uint32_t rows) {
  return rows <= 64u ? rows : (rows + 7u) / 8u;
}

}  // namespace qllm

using namespace qllm;

extern "C" size_t qllm_q4h_layer_bytes(uint32_t page_tokens, uint32_t kv_heads,
                                       uint32_t head_dim) {
  return q4h_layer_bytes(page_tokens, kv_heads, head_dim);
}

extern "C" int32_t qllm_store_kv_paged_q4h_batch(
    const float* key, const float* value, const void* const* page_table,
    uint32_t full_attention_layer, uint32_t page_tokens,
    uint32_t first_cache_position, uint32_t rows, uint32_t kv_heads,
    uint32_t head_dim, void* stream) {
  if (!key || !value || !page_table || !page_tokens || !rows || !kv_heads ||
      !head_dim || head_dim % 2u || head_dim > 256u ||
      first_cache_position > 0xffffffffu - (rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid Q4H K/V store");
  q4h_store_kernel<<<dim3(kv_heads, rows), 64, 0, as_stream(stream)>>>(
      key, value, page_table, full_attention_layer, page_tokens,
      first_cache_position, kv_heads, head_dim);
  return launched("Q4H K/V store");
}

extern "C" int32_t qllm_qkv_rope_cache_paged_q4h_batch(
    float* query, uint32_t query_stride, float* key, const float* value,
    const float* q_norm_weight, const float* k_norm_weight,
    const void* const* page_table, uint32_t full_attention_layer,
    uint32_t page_tokens, uint32_t first_cache_position,
    uint32_t first_rotary_position, uint32_t rows, uint32_t query_heads,
    uint32_t kv_heads, uint32_t head_dim, uint32_t rotary_dim, float epsilon,
    float rope_theta, int32_t bf16_activations, void* stream) {
  if (!query || !key || !value || !page_table || !page_tokens || !rows ||
      !query_heads || !kv_heads || query_heads < kv_heads ||
      query_heads % kv_heads || !head_dim || head_dim > 256u || head_dim % 2u ||
      query_stride < head_dim || !rotary_dim || rotary_dim > head_dim ||
      rotary_dim % 2u || !(epsilon > 0.0f) || !(rope_theta > 0.0f) ||
      first_cache_position > 0xffffffffu - (rows - 1u) ||
      first_rotary_position > 0xffffffffu - (rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid Q4H QKV rope cache batch");
  qkv_rope_q4h_kernel<<<dim3(query_heads + kv_heads, rope_grid_rows(rows)), 64, 0,
                        as_stream(stream)>>>(
      query, query_stride, key, value, q_norm_weight, k_norm_weight, page_table,
      full_attention_layer, page_tokens, first_cache_position,
      first_rotary_position, query_heads, kv_heads, head_dim, rotary_dim,
      epsilon, rope_theta, bf16_activations != 0, nullptr, nullptr, 0u, rows,
      nullptr, nullptr);
  return launched("Q4H QKV rope cache batch");
}

extern "C" int32_t qllm_qkv_rope_cache_paged_q4h_batch_deferred(
    float* query, uint32_t query_stride, float* key, const float* value,
    const float* q_norm_weight, const float* k_norm_weight,
    const void* const* page_table, uint32_t full_attention_layer,
    uint32_t page_tokens, const uint32_t* device_positions, uint32_t rows,
    uint32_t query_heads, uint32_t kv_heads, uint32_t head_dim,
    uint32_t rotary_dim, float epsilon, float rope_theta,
    int32_t bf16_activations, void* stream) {
  if (!query || !key || !value || !page_table || !page_tokens ||
      !device_positions || !rows || !query_heads || !kv_heads ||
      query_heads < kv_heads || query_heads % kv_heads || !head_dim ||
      head_dim > 256u || head_dim % 2u || query_stride < head_dim ||
      !rotary_dim || rotary_dim > head_dim || rotary_dim % 2u ||
      !(epsilon > 0.0f) || !(rope_theta > 0.0f))
    return fail(QLLM_INVALID_ARGUMENT,
                "invalid deferred Q4H QKV rope cache batch");
  qkv_rope_q4h_kernel<<<dim3(query_heads + kv_heads, rope_grid_rows(rows)), 64, 0,
                        as_stream(stream)>>>(
      query, query_stride, key, value, q_norm_weight, k_norm_weight, page_table,
      full_attention_layer, page_tokens, 0u, 0u, query_heads, kv_heads,
      head_dim, rotary_dim, epsilon, rope_theta, bf16_activations != 0,
      device_positions, nullptr, 0u, rows, nullptr, nullptr);
  return launched("deferred Q4H QKV rope cache batch");
}

extern "C" int32_t qllm_qkv_rope_cache_paged_q4h_from_partials(
    const float* partials, uint32_t partial_count, float* query,
    uint32_t query_stride, float* key, float* value,
    const float* q_norm_weight, const float* k_norm_weight,
    const void* const* page_table, uint32_t full_attention_layer,
    uint32_t page_tokens, uint32_t first_cache_position,
    uint32_t first_rotary_position, const uint32_t* device_positions,
    uint32_t rows, uint32_t query_heads, uint32_t kv_heads, uint32_t head_dim,
    uint32_t rotary_dim, float epsilon, float rope_theta,
    int32_t bf16_activations, void* stream) {
  if (!partials || !partial_count || partial_count > 16u || !query || !key ||
      !value || !page_table || !page_tokens || !rows || !query_heads ||
      !kv_heads || query_heads < kv_heads || query_heads % kv_heads ||
      !head_dim || head_dim > 256u || head_dim % 2u ||
      query_stride < head_dim || !rotary_dim || rotary_dim > head_dim ||
      rotary_dim % 2u || !(epsilon > 0.0f) || !(rope_theta > 0.0f) ||
      (!device_positions &&
       (first_cache_position > 0xffffffffu - (rows - 1u) ||
        first_rotary_position > 0xffffffffu - (rows - 1u))))
    return fail(QLLM_INVALID_ARGUMENT,
                "invalid Q4H QKV rope cache batch from partials");
  qkv_rope_q4h_kernel<<<dim3(query_heads + kv_heads, rope_grid_rows(rows)), 64, 0,
                        as_stream(stream)>>>(
      query, query_stride, key, value, q_norm_weight, k_norm_weight, page_table,
      full_attention_layer, page_tokens, first_cache_position,
      first_rotary_position, query_heads, kv_heads, head_dim, rotary_dim,
      epsilon, rope_theta, bf16_activations != 0, device_positions, partials,
      partial_count, rows, nullptr, nullptr);
  return launched("Q4H QKV rope cache batch from partials");
}

extern "C" size_t qllm_q4h_query_operand_bytes(uint32_t rows,
                                               uint32_t query_heads,
                                               uint32_t kv_heads,
                                               uint32_t head_dim) {
  if (!rows || !kv_heads || !query_heads || query_heads % kv_heads ||
      (head_dim != 128u && head_dim != 256u))
    return 0;
  return kv_heads *
         q4h_operand_plane_bytes(q4h_row_tiles(rows, query_heads / kv_heads),
                                 head_dim);
}

extern "C" int32_t qllm_qkv_rope_cache_paged_q4h_prepared(
    const float* partials, uint32_t partial_count, float* query,
    uint32_t query_stride, float* key, float* value,
    const float* q_norm_weight, const float* k_norm_weight,
    const void* const* page_table, uint32_t full_attention_layer,
    uint32_t page_tokens, uint32_t first_cache_position,
    uint32_t first_rotary_position, const uint32_t* device_positions,
    uint32_t rows, uint32_t query_heads, uint32_t kv_heads, uint32_t head_dim,
    uint32_t rotary_dim, float epsilon, float rope_theta,
    int32_t bf16_activations, int8_t* query_operands,
    float* query_operand_scales, void* stream) {
  if ((partials && (!partial_count || partial_count > 16u)) || !query || !key ||
      !value || !page_table || !page_tokens || !rows || !query_heads ||
      !kv_heads || query_heads < kv_heads || query_heads % kv_heads ||
      (head_dim != 128u && head_dim != 256u) || query_stride < head_dim ||
      !rotary_dim || rotary_dim > head_dim || rotary_dim % 2u ||
      !(epsilon > 0.0f) || !(rope_theta > 0.0f) || !query_operands ||
      !query_operand_scales ||
      (reinterpret_cast<uintptr_t>(query_operands) & 15u) ||
      (!device_positions &&
       (first_cache_position > 0xffffffffu - (rows - 1u) ||
        first_rotary_position > 0xffffffffu - (rows - 1u))))
    return fail(QLLM_INVALID_ARGUMENT,
                "invalid Q4H QKV rope cache batch with query operands");
  const uint32_t row_tiles = q4h_row_tiles(rows, query_heads / kv_heads);
  if (row_tiles > 3u || (head_dim == 256u && row_tiles > 2u))
    return fail(QLLM_INVALID_ARGUMENT,
                "Q4H query operands: rows * (query_heads/kv_heads) exceeds 48 "
                "(32 at head_dim 256)");
  qkv_rope_q4h_kernel<<<dim3(query_heads + kv_heads, rope_grid_rows(rows)), 64, 0,
                        as_stream(stream)>>>(
      query, query_stride, key, value, q_norm_weight, k_norm_weight, page_table,
      full_attention_layer, page_tokens, first_cache_position,
      first_rotary_position, query_heads, kv_heads, head_dim, rotary_dim,
      epsilon, rope_theta, bf16_activations != 0, device_positions, partials,
      partials ? partial_count : 0u, rows,
      reinterpret_cast<uint8_t*>(query_operands), query_operand_scales);
  return launched("Q4H QKV rope cache batch with query operands");
}

extern "C" int32_t qllm_qkv_rope_batch(
    float* query, uint32_t query_stride, float* key,
    const float* q_norm_weight, const float* k_norm_weight,
    uint32_t first_rotary_position, uint32_t rows, uint32_t query_heads,
    uint32_t kv_heads, uint32_t head_dim, uint32_t rotary_dim, float epsilon,
    float rope_theta, int32_t bf16_activations, void* stream) {
  if (!query || !key || !rows || !query_heads || !kv_heads ||
      query_heads < kv_heads || query_heads % kv_heads || !head_dim ||
      head_dim > 256u || head_dim % 2u || query_stride < head_dim ||
      !rotary_dim || rotary_dim > head_dim || rotary_dim % 2u ||
      !(epsilon > 0.0f) || !(rope_theta > 0.0f) ||
      first_rotary_position > 0xffffffffu - (rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid QKV rope batch");
  qkv_rope_q4h_kernel<<<dim3(query_heads + kv_heads, rope_grid_rows(rows)), 64, 0,
                        as_stream(stream)>>>(
      query, query_stride, key, nullptr, q_norm_weight, k_norm_weight, nullptr,
      0u, 1u, 0u, first_rotary_position, query_heads, kv_heads, head_dim,
      rotary_dim, epsilon, rope_theta, bf16_activations != 0, nullptr, nullptr,
      0u, rows, nullptr, nullptr);
  return launched("QKV rope batch");
}

extern "C" int32_t qllm_qkv_rope_batch_deferred(
    float* query, uint32_t query_stride, float* key,
    const float* q_norm_weight, const float* k_norm_weight,
    const uint32_t* device_positions, uint32_t rows, uint32_t query_heads,
    uint32_t kv_heads, uint32_t head_dim, uint32_t rotary_dim, float epsilon,
    float rope_theta, int32_t bf16_activations, void* stream) {
  if (!query || !key || !device_positions || !rows || !query_heads ||
      !kv_heads || query_heads < kv_heads || query_heads % kv_heads ||
      !head_dim || head_dim > 256u || head_dim % 2u ||
      query_stride < head_dim || !rotary_dim || rotary_dim > head_dim ||
      rotary_dim % 2u || !(epsilon > 0.0f) || !(rope_theta > 0.0f))
    return fail(QLLM_INVALID_ARGUMENT, "invalid deferred QKV rope batch");
  qkv_rope_q4h_kernel<<<dim3(query_heads + kv_heads, rope_grid_rows(rows)), 64, 0,
                        as_stream(stream)>>>(
      query, query_stride, key, nullptr, q_norm_weight, k_norm_weight, nullptr,
      0u, 1u, 0u, 0u, query_heads, kv_heads, head_dim, rotary_dim, epsilon,
      rope_theta, bf16_activations != 0, device_positions, nullptr, 0u, rows,
      nullptr, nullptr);
  return launched("deferred QKV rope batch");
}

// Rotary (and per-head norm) of a batch's queries and keys plus the K/V store
// into the proposer's Q8 cache, in one launch; device_positions (optional):
// word 0 the first cache position, word 1 the first rotary position.
extern "C" int32_t qllm_qkv_rope_store_q8_batch(
    float* query, uint32_t query_stride, float* key, const float* value,
    const float* q_norm_weight, const float* k_norm_weight,
    const void* const* page_table, size_t page_offset_bytes, uint32_t page_tokens,
    uint32_t first_cache_position, uint32_t first_rotary_position,
    const uint32_t* device_positions, uint32_t rows, uint32_t query_heads,
    uint32_t kv_heads, uint32_t head_dim, uint32_t rotary_dim, float epsilon,
    float rope_theta, int32_t bf16_activations, void* stream) {
  if (!query || !key || !value || !page_table || !page_tokens || !rows ||
      !query_heads || !kv_heads || query_heads < kv_heads ||
      query_heads % kv_heads || !head_dim || head_dim > 256u || head_dim % 2u ||
      query_stride < head_dim || !rotary_dim || rotary_dim > head_dim ||
      rotary_dim % 2u || !(epsilon > 0.0f) || !(rope_theta > 0.0f) ||
      page_offset_bytes % 16u ||
      (!device_positions &&
       (first_cache_position > 0xffffffffu - (rows - 1u) ||
        first_rotary_position > 0xffffffffu - (rows - 1u))))
    return fail(QLLM_INVALID_ARGUMENT, "invalid QKV rope + Q8 store batch");
  qkv_rope_q4h_kernel<<<dim3(query_heads + kv_heads, rope_grid_rows(rows)), 64, 0,
                        as_stream(stream)>>>(
      query, query_stride, key, value, q_norm_weight, k_norm_weight, nullptr, 0u,
      page_tokens, first_cache_position, first_rotary_position, query_heads,
      kv_heads, head_dim, rotary_dim, epsilon, rope_theta, bf16_activations != 0,
      device_positions, nullptr, 0u, rows, nullptr, nullptr, page_table,
      page_offset_bytes);
  return launched("QKV rope + Q8 store batch");
}

extern "C" int32_t qllm_quantize_gqa_queries_q8(
    const float* query, uint32_t query_stride, int8_t* q8, float* query_scales,
    uint32_t rows, uint32_t query_heads, uint32_t head_dim, void* stream) {
  if (!query || !q8 || !query_scales || !rows || !query_heads || !head_dim ||
      query_stride < head_dim)
    return fail(QLLM_INVALID_ARGUMENT, "invalid GQA query Q8 quantization");
  quantize_queries_q8_kernel<<<dim3(query_heads, rows), 64, 0,
                               as_stream(stream)>>>(
      query, query_stride, q8, query_scales, query_heads, head_dim);
  return launched("GQA query Q8 quantization");
}

extern "C" int32_t qllm_attention_paged_q4h_batched(
    const qllm_q4h_attention_launch* launch, uint32_t batch_rows) {
  if (!launch || !launch->query || !launch->page_table || !launch->output ||
      (reinterpret_cast<uintptr_t>(launch->query) & 15u) ||
      launch->query_stride % 4u || !launch->partial_maxima ||
      !launch->partial_sums || !launch->partial_outputs ||
      !launch->first_context_tokens || !launch->rows || !batch_rows ||
      launch->device_positions || !launch->page_tokens ||
      launch->page_tokens % 64u || !launch->query_heads || !launch->kv_heads ||
      launch->query_heads % launch->kv_heads ||
      (launch->head_dim != 128u && launch->head_dim != 256u) ||
      launch->split_tokens % 64u || !launch->maximum_splits ||
      launch->maximum_splits > kCombineSplitCapacity ||
      launch->query_stride <
          (launch->output_gated ? 2u : 1u) * launch->head_dim ||
      (launch->output_kind != QLLM_OUT_F32 &&
       launch->output_kind != QLLM_OUT_BF16) ||
      launch->rows > 65535u ||
      launch->first_context_tokens > 0xffffffffu - (launch->rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid batched Q4H paged attention");
  const uint32_t group = launch->query_heads / launch->kv_heads;
  const uint32_t row_tiles = (std::min(batch_rows, launch->rows) * group + 15u) / 16u;
  if (row_tiles > 3u || (launch->head_dim == 256u && row_tiles > 2u))
    return fail(QLLM_INVALID_ARGUMENT,
                "batched Q4H paged attention: batch_rows * (query_heads/kv_heads) "
                "exceeds 48 (32 at head_dim 256)");
  const uint32_t batches = (launch->rows + batch_rows - 1u) / batch_rows;
  const uint32_t last_context = launch->first_context_tokens + launch->rows - 1u;
  const uint32_t splits =
      !launch->split_tokens
          ? launch->maximum_splits
          : (last_context + launch->split_tokens - 1u) / launch->split_tokens;
  if (splits > launch->maximum_splits)
    return fail(QLLM_INVALID_ARGUMENT,
                "batched Q4H paged attention: context needs more splits than "
                "maximum_splits");
  SplitArgs args{};
  args.query = launch->query;
  args.query_stride = launch->query_stride;
  args.page_table = launch->page_table;
  args.partial_maxima = launch->partial_maxima;
  args.partial_sums = launch->partial_sums;
  args.partial_outputs = launch->partial_outputs;
  args.first_context_tokens = launch->first_context_tokens;
  args.rows = launch->rows;
  args.layer = launch->full_attention_layer;
  args.page_tokens = launch->page_tokens;
  args.query_heads = launch->query_heads;
  args.kv_heads = launch->kv_heads;
  args.split_tokens = launch->split_tokens;
  args.maximum_splits = launch->maximum_splits;
  args.batch_rows = batch_rows;
  const dim3 grid(launch->kv_heads, splits, batches);
  const hipStream_t stream = as_stream(launch->stream);
  int32_t status = launch->head_dim == 128u
                       ? launch_split<128>(args, row_tiles, grid, stream)
                       : launch_split<256>(args, row_tiles, grid, stream);
  if (status != QLLM_OK) return status;
  // partials are laid out by global row, which is what the combine indexes
  return launch_attention_combine(
      launch->query, launch->query_stride, launch->output_gated,
      launch->partial_maxima, launch->partial_sums, launch->partial_outputs,
      launch->output, launch->output_kind, launch->first_context_tokens,
      launch->maximum_splits, launch->split_tokens, launch->rows,
      launch->query_heads, launch->head_dim, nullptr, stream);
}

extern "C" int32_t qllm_attention_paged_q4h_prompt(
    const qllm_q4h_attention_launch* launch, uint32_t batch_rows) {
  if (!launch || !launch->query || !launch->page_table || !launch->output ||
      (reinterpret_cast<uintptr_t>(launch->query) & 15u) ||
      launch->query_stride % 4u || !launch->partial_maxima ||
      !launch->partial_sums || !launch->partial_outputs ||
      !launch->first_context_tokens || !launch->rows || !batch_rows ||
      launch->device_positions || !launch->page_tokens ||
      launch->page_tokens % 64u || !launch->query_heads || !launch->kv_heads ||
      launch->query_heads % launch->kv_heads || launch->head_dim != 128u ||
      launch->split_tokens || !launch->maximum_splits ||
      launch->maximum_splits > kCombineSplitCapacity ||
      launch->query_stride <
          (launch->output_gated ? 2u : 1u) * launch->head_dim ||
      (launch->output_kind != QLLM_OUT_F32 &&
       launch->output_kind != QLLM_OUT_BF16) ||
      launch->rows > 65535u * kPromptBatches ||
      launch->first_context_tokens > 0xffffffffu - (launch->rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid Q4H prompt attention");
  const uint32_t group = launch->query_heads / launch->kv_heads;
  if (std::min(batch_rows, launch->rows) * group > 48u)
    return fail(QLLM_INVALID_ARGUMENT,
                "Q4H prompt attention: batch_rows * (query_heads/kv_heads) "
                "exceeds 48");
  const uint32_t batches = (launch->rows + batch_rows - 1u) / batch_rows;
  SplitArgs args{};
  args.query = launch->query;
  args.query_stride = launch->query_stride;
  args.page_table = launch->page_table;
  args.partial_maxima = launch->partial_maxima;
  args.partial_sums = launch->partial_sums;
  args.partial_outputs = launch->partial_outputs;
  args.first_context_tokens = launch->first_context_tokens;
  args.rows = launch->rows;
  args.layer = launch->full_attention_layer;
  args.page_tokens = launch->page_tokens;
  args.query_heads = launch->query_heads;
  args.kv_heads = launch->kv_heads;
  args.maximum_splits = launch->maximum_splits;
  args.batch_rows = batch_rows;
  const dim3 grid(launch->kv_heads, launch->maximum_splits,
                  (batches + kPromptBatches - 1u) / kPromptBatches);
  const hipStream_t stream = as_stream(launch->stream);
  q4h_prompt_attention_kernel<128><<<grid, kPromptBatches * 64, 0, stream>>>(args);
  const int32_t status = launched("Q4H prompt attention");
  if (status != QLLM_OK) return status;
  return launch_attention_combine(
      launch->query, launch->query_stride, launch->output_gated,
      launch->partial_maxima, launch->partial_sums, launch->partial_outputs,
      launch->output, launch->output_kind, launch->first_context_tokens,
      launch->maximum_splits, 0u, launch->rows, launch->query_heads,
      launch->head_dim, nullptr, stream);
}

namespace {
int32_t launch_q4h_attention(const qllm_q4h_attention_launch* launch,
                             const qllm_q4h_fused_rope* rope) {
  if (!launch || !launch->query || !launch->page_table || !launch->output ||
      (reinterpret_cast<uintptr_t>(launch->query) & 15u) ||
      launch->query_stride % 4u ||
      !launch->partial_maxima || !launch->partial_sums ||
      !launch->partial_outputs || !launch->first_context_tokens ||
      !launch->rows || !launch->page_tokens || launch->page_tokens % 64u ||
      !launch->query_heads || !launch->kv_heads ||
      launch->query_heads % launch->kv_heads ||
      (launch->head_dim != 128u && launch->head_dim != 256u) ||
      launch->split_tokens % 64u || !launch->maximum_splits ||
      launch->maximum_splits > kCombineSplitCapacity ||
      launch->query_stride <
          (launch->output_gated ? 2u : 1u) * launch->head_dim ||
      (launch->output_kind != QLLM_OUT_F32 &&
       launch->output_kind != QLLM_OUT_BF16) ||
      launch->first_context_tokens > 0xffffffffu - (launch->rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid Q4H paged attention");
  const uint32_t group = launch->query_heads / launch->kv_heads;
  const uint32_t matrix_rows = launch->rows * group;
  const uint32_t row_tiles = (matrix_rows + 15u) / 16u;
  if (row_tiles > 3u || (launch->head_dim == 256u && row_tiles > 2u))
    return fail(QLLM_INVALID_ARGUMENT,
                "Q4H paged attention: rows * (query_heads/kv_heads) exceeds "
                "48 (32 at head_dim 256)");
  const uint32_t last_context = launch->first_context_tokens + launch->rows - 1u;
  // with device-side positions the context is not known here: cover every
  // split (workgroups past the context write neutral partials)
  const uint32_t splits =
      launch->device_positions || !launch->split_tokens
          ? launch->maximum_splits
          : (last_context + launch->split_tokens - 1u) / launch->split_tokens;
  if (splits > launch->maximum_splits)
    return fail(QLLM_INVALID_ARGUMENT,
                "Q4H paged attention: context needs more splits than "
                "maximum_splits");
  SplitArgs args{};
  args.query = launch->query;
  if (launch->q8_queries && launch->query_scales) {
    if (reinterpret_cast<uintptr_t>(launch->q8_queries) & 15u)
      return fail(QLLM_INVALID_ARGUMENT,
                  "Q4H paged attention: query operands must be 16-byte aligned");
    args.query_operands = reinterpret_cast<const uint8_t*>(launch->q8_queries);
    args.query_operand_scales = launch->query_scales;
  }
  args.query_stride = launch->query_stride;
  args.page_table = launch->page_table;
  args.partial_maxima = launch->partial_maxima;
  args.partial_sums = launch->partial_sums;
  args.partial_outputs = launch->partial_outputs;
  args.first_context_tokens = launch->first_context_tokens;
  args.rows = launch->rows;
  args.layer = launch->full_attention_layer;
  args.page_tokens = launch->page_tokens;
  args.query_heads = launch->query_heads;
  args.kv_heads = launch->kv_heads;
  args.split_tokens = launch->split_tokens;
  args.maximum_splits = launch->maximum_splits;
  args.device_positions = launch->device_positions;
  const dim3 grid(launch->kv_heads, splits);
  const hipStream_t stream = as_stream(launch->stream);
  int32_t status;
  if (rope) {
    if (!rope->key || !rope->value || !rope->rope_table || !rope->rotary_dim ||
        launch->rows > 16u ||
        rope->rotary_dim > launch->head_dim || rope->rotary_dim % 2u ||
        !(rope->epsilon > 0.0f) ||
        (!launch->device_positions &&
         rope->first_cache_position + 1u != launch->first_context_tokens))
      return fail(QLLM_INVALID_ARGUMENT, "invalid fused rotary inputs");
    args.query_operands = nullptr;
    args.raw_key = rope->key;
    args.raw_value = rope->value;
    args.q_weight = rope->q_norm_weight;
    args.k_weight = rope->k_norm_weight;
    args.rope_table = reinterpret_cast<const float2*>(rope->rope_table);
    args.rotary_dim = rope->rotary_dim;
    args.epsilon = rope->epsilon;
    args.first_cache_position = rope->first_cache_position;
    args.bf16_activations = rope->bf16_activations != 0 ? 1u : 0u;
    status = launch->head_dim == 128u
                 ? launch_split<128, true>(args, row_tiles, grid, stream)
                 : launch_split<256, true>(args, row_tiles, grid, stream);
  } else {
    status = launch->head_dim == 128u
                 ? launch_split<128>(args, row_tiles, grid, stream)
                 : launch_split<256>(args, row_tiles, grid, stream);
  }
  if (status != QLLM_OK) return status;
  return launch_attention_combine(
      launch->query, launch->query_stride, launch->output_gated,
      launch->partial_maxima, launch->partial_sums, launch->partial_outputs,
      launch->output, launch->output_kind, launch->first_context_tokens,
      launch->maximum_splits, launch->split_tokens, launch->rows,
      launch->query_heads, launch->head_dim, launch->device_positions, stream);
}
}  // namespace

extern "C" int32_t qllm_attention_paged_q4h(
    const qllm_q4h_attention_launch* launch) {
  return launch_q4h_attention(launch, nullptr);
}

extern "C" int32_t qllm_attention_paged_q4h_fused(
    const qllm_q4h_attention_launch* launch, const qllm_q4h_fused_rope* rope) {
  if (!rope) return fail(QLLM_INVALID_ARGUMENT, "invalid fused rotary inputs");
  return launch_q4h_attention(launch, rope);
}

extern "C" int32_t qllm_rope_table(float* table, uint32_t rows,
                                   uint32_t rotary_dim,
                                   uint32_t first_rotary_position,
                                   float rope_theta, int32_t bf16_activations,
                                   const uint32_t* device_positions,
                                   void* stream) {
  if (!table || !rows || !rotary_dim || rotary_dim % 2u || rotary_dim > 256u ||
      !(rope_theta > 0.0f) ||
      (!device_positions && first_rotary_position > 0xffffffffu - (rows - 1u)))
    return fail(QLLM_INVALID_ARGUMENT, "invalid rotary table request");
  rope_table_kernel<<<rows, 128, 0, as_stream(stream)>>>(
      reinterpret_cast<float2*>(table), rotary_dim, first_rotary_position,
      rope_theta, bf16_activations != 0, device_positions);
  return launched("rotary table");
}
