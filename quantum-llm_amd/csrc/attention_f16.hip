// Exact-F16 and Q8 paged KV caches: K/V store and decode attention.
//
// Replaces, from runtime/src/cuda/transformer_kernels.cu of the reference:
//   store_gqa_kv_fp16_to_paged                                  :4208
//   gated_gqa_attention_staged_fp16_impl and its kernels        :10214-10476,
//                                                               :6517-6665, :7023-7057
// The reference walks its context splits one after the other and keeps one
// running softmax state; here the splits run in parallel, each workgroup
// leaves an (max, sum, unnormalised output) partial and the split combine
// shared with the Q4H path merges them.  Arithmetic follows the reference:
// the query is rounded to binary16, scores are F32 sums of binary16
// products, probabilities are rounded to binary16 before they weigh V and
// before they enter the denominator.
//
// The same kernel, instantiated for the proposer's Q8 cache (int8 codes, one
// binary16 scale per record; reference encoder :601-625, attention
// gated_gqa_attention_microbatch_paged_q8_tensor_core :9732): codes become
// exact binary16 integers on the way into the matrix cores, the K scale
// multiplies the score and the V scale the probability.
#include "attention_common.hpp"

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


// Q8 layout inside a page, `page_offset` bytes in:  K codes
// [page_tokens][kv_heads][head_dim] int8, V codes likewise, K scales
// [kv_heads][page_tokens] binary16, V scales likewise - the reference's
// records (codes followed by their scale, :5093-5101) with codes and scales in
// separate planes, which keeps every row 16-byte aligned; the bytes per layer
// are the same, page_tokens * kv_heads * 2 * (head_dim + 2).
// One wave per (token, kv head); scale = f16(max(absmax/127, 2^-24)),
// code = clamp(rn(x / scale), -127, 127)  (:601-625).
__global__ __launch_bounds__(64) void q8_store_kernel(
    const float* key, const float* value, const void* const* page_table,
    size_t page_offset, uint32_t page_tokens, uint32_t first_cache_position,
    uint32_t kv_heads, uint32_t head_dim, const uint32_t* device_positions) {
  const uint32_t lane = threadIdx.x;
  const uint32_t kv_head = blockIdx.x;
  const uint32_t row = blockIdx.y;
  if (device_positions)
    first_cache_position = uniform_word(device_positions, 0u);
  const uint32_t position = first_cache_position + row;
  uint8_t* page = static_cast<uint8_t*>(const_cast<void*>(
                      page_table[position / page_tokens])) + page_offset;
  const uint32_t slot = position % page_tokens;
#pragma unroll
  for (uint32_t kind = 0; kind < 2u; ++kind)
    q8_encode_record((kind ? value : key) +
                         (static_cast<size_t>(row) * kv_heads + kv_head) * head_dim,
                     head_dim, page, kind, slot, kv_head, kv_heads, page_tokens, lane);
}

// 8 int8 codes -> 8 exact binary16 values: code + 128 becomes the low mantissa
// byte of 1024.0 (bit pattern 0x6400 + u = 1024 + u exactly), minus 1152.
__device__ __forceinline__ f16x8 int8x8_to_f16(uint2 codes) {
  const uint32_t low = codes.x ^ 0x80808080u;
  const uint32_t high = codes.y ^ 0x80808080u;
  const f16x2 bias = {static_cast<_Float16>(-1152.0f), static_cast<_Float16>(-1152.0f)};
  const f16x2 e0 = __builtin_bit_cast(
      f16x2, __builtin_amdgcn_perm(0x64646464u, low, 0x04010400u)) + bias;
  const f16x2 e1 = __builtin_bit_cast(
      f16x2, __builtin_amdgcn_perm(0x64646464u, low, 0x04030402u)) + bias;
  const f16x2 e2 = __builtin_bit_cast(
      f16x2, __builtin_amdgcn_perm(0x64646464u, high, 0x04010400u)) + bias;
  const f16x2 e3 = __builtin_bit_cast(
      f16x2, __builtin_amdgcn_perm(0x64646464u, high, 0x04030402u)) + bias;
  f16x8 result;
  result[0] = e0[0]; result[1] = e0[1]; result[2] = e1[0]; result[3] = e1[1];
  result[4] = e2[0]; result[5] = e2[1]; result[6] = e3[0]; result[7] = e3[1];
  return result;
}

struct F16SplitArgs {
  const float* query;
  uint32_t query_stride;
  const void* const* pages;
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
  size_t page_offset;   // Q8: byte offset of the layer inside a page
  const uint32_t* device_positions;  // optional: [2] = first_context_tokens
  // Batched launch (prompt prefill): grid layer z takes rows
  // [z * batch_rows, +batch_rows) of `rows`.  0 = one batch holds all rows.
  uint32_t batch_rows;
};

constexpr uint32_t kF16Tile = 32;  // tokens per wave step

// One workgroup (8 waves) per (kv head, context split); a wave walks 32-token
// tiles with its own online-softmax state:
//   scores  S[tok][row] = K . Q     v_mfma_f32_16x16x32_f16; K rows come
//           straight from the page as A operands (16 bytes per lane), the
//           binary16 query sits in LDS in B-operand order
//   output  O^T[d][row] += V^T . P^T   v_mfma_f32_16x16x16_f16; the V tile is
//           staged in LDS, rows swizzled so that the transposing read
//           (ds_read_b64_tr_b16: 4 tokens x 16 dims per lane group) is free
//           of bank conflicts, and the score registers of a 16-token sub-tile
//           are already the B operand.
// D = head_dim (128 or 256), RT = 16-row tiles of rows*group query rows,
// Q8 = the cache holds int8 codes and per-record scales instead of binary16.
template <int D, int RT, bool Q8>
__global__ __launch_bounds__(kSplitWaves * 64) void f16_attention_split_kernel(
    const F16SplitArgs launch_args) {
  // a batched launch narrows the arguments to the batch of this grid layer
  F16SplitArgs args = launch_args;
  if (launch_args.batch_rows) {
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
  constexpr int KSTEPS = D / 32;  // k-steps of the score MFMA over head_dim
  constexpr int DT = D / 16;      // 16-wide tiles of head_dim
  constexpr int GR = D / 8;       // 16-byte granules per V row
  constexpr int STAGE = kF16Tile * D * 2;  // V tile of a wave (bytes)
  constexpr int UNITS = RT * KSTEPS;       // query operands of 1 KiB
  constexpr int POOL = kSplitWaves * kSplitWaves * 1024;  // merge needs 64 KiB
  constexpr int EXCHANGE_Q = UNITS * 1024 + RT * 64;
  constexpr int EXCHANGE_MERGE = kSplitWaves * RT * 512;
  __shared__ __attribute__((aligned(16)))
  uint8_t stage[kSplitWaves * STAGE > POOL ? kSplitWaves * STAGE : POOL];
  __shared__ __attribute__((aligned(16)))
  uint8_t exchange[EXCHANGE_Q > EXCHANGE_MERGE ? EXCHANGE_Q : EXCHANGE_MERGE];

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t col = lane & 15u;
  const uint32_t quad = lane >> 4;
  const uint32_t kv_head = blockIdx.x;
  const uint32_t split = blockIdx.y;
  const uint32_t group = args.query_heads / args.kv_heads;
  const uint32_t matrix_rows = args.rows * group;
  const uint32_t first_context_tokens =
      args.device_positions ? uniform_word(args.device_positions, 2u)
                            : args.first_context_tokens;
  const uint32_t last_context = first_context_tokens + args.rows - 1u;
  const uint32_t context_tiles = (last_context + kF16Tile - 1u) / kF16Tile;
  uint32_t tile_first, tile_last;
  wave_tile_range(context_tiles, kF16Tile, args.split_tokens, split, gridDim.y,
                  wave, tile_first, tile_last);

  // ---- query operands (B side of S = K.Q) in binary16, built once -------------
  uint32_t* exchange_limit = reinterpret_cast<uint32_t*>(exchange + UNITS * 1024);
  for (uint32_t unit = wave; unit < static_cast<uint32_t>(UNITS);
       unit += kSplitWaves) {
    const uint32_t rt = unit / KSTEPS;
    const uint32_t step = unit % KSTEPS;
    const uint32_t matrix_row = 16u * rt + col;
    const bool valid = matrix_row < matrix_rows;
    const uint32_t row = valid ? matrix_row / group : 0u;
    const uint32_t head = kv_head * group + (valid ? matrix_row % group : 0u);
    const float* source =
        args.query +
        (static_cast<size_t>(row) * args.query_heads + head) * args.query_stride +
        32u * step + 8u * quad;
    f16x8 operand;
#pragma unroll
    for (int piece = 0; piece < 2; ++piece) {
      float4 loaded = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if (valid) loaded = *reinterpret_cast<const float4*>(source + 4 * piece);
      operand[4 * piece + 0] = static_cast<_Float16>(loaded.x);
      operand[4 * piece + 1] = static_cast<_Float16>(loaded.y);
      operand[4 * piece + 2] = static_cast<_Float16>(loaded.z);
      operand[4 * piece + 3] = static_cast<_Float16>(loaded.w);
    }
    *reinterpret_cast<f16x8*>(exchange + unit * 1024u + lane * 16u) = operand;
    if (step == 0u && quad == 0u)
      exchange_limit[16u * rt + col] = first_context_tokens + row;
  }
  __syncthreads();
  const uint8_t* q_operands = exchange + lane * 16u;
  const float score_unit =
      1.4426950408889634f / sqrtf(static_cast<float>(D));  // log2 units

  // ---- page geometry ------------------------------------------------------------
  const size_t page_values =
      static_cast<size_t>(args.page_tokens) * args.kv_heads * D;
  const size_t layer_offset = static_cast<size_t>(args.layer) * 2u * page_values;
  const uint32_t row_stride = args.kv_heads * D;  // elements between tokens
  uint8_t* stage_v = stage + wave * STAGE;
  // transposing read: lane (quad, col = 4*r + j) supplies the 8 bytes of token
  // 4*quad + r (of the 16-token sub-tile), halves 16*dt + 4*j .. +3.  Granule
  // (16 bytes) p of token t lives at granule p ^ (2 * (t & 7)) of its row.
  const uint32_t read_token = 4u * quad + (col >> 2);
  const uint32_t read_swizzle = read_token & 7u;
  const uint32_t read_base =
      read_token * (GR * 16u) + ((col >> 1) & 1u) * 16u + (col & 1u) * 8u;

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

  // Q8 cache: a tile's codes and scales as the lanes fetch them - V granules
  // (8 codes) pass * 64 + lane, the K operand rows, the scales of the lane's
  // tokens.  The next tile's are asked for before the tile at hand is worked on,
  // so a wave always has one tile in flight (the binary16 cache at head_dim 128
  // has the kernel below for that) - where the registers hold a second tile.
  constexpr bool AHEAD = Q8 && D == 128 && RT <= 2;
  constexpr int V_PASSES = kF16Tile * GR / 64;
  struct Q8Tile {
    uint2 value[V_PASSES];
    uint2 key[2][KSTEPS];
    uint2 key_scale[2];
    uint2 value_scale[2];
  };
  const auto fetch_q8_tile = [&](uint32_t tile, Q8Tile& loaded) {
    const uint32_t tile_begin = tile * kF16Tile;
    const void* page_base = uniform_page(args.pages, tile_begin / args.page_tokens);
    const uint32_t tile_slot = tile_begin % args.page_tokens;
    // code planes, then scale planes [kv_heads][page_tokens]
    const uint8_t* keys8 = static_cast<const uint8_t*>(page_base) + args.page_offset +
                           static_cast<size_t>(tile_slot) * row_stride + kv_head * D;
    const uint8_t* values8 = keys8 + page_values;
    const uint16_t* key_scales =
        reinterpret_cast<const uint16_t*>(static_cast<const uint8_t*>(page_base) +
                                          args.page_offset + 2u * page_values) +
        static_cast<size_t>(kv_head) * args.page_tokens + tile_slot;
    const uint16_t* value_scales =
        key_scales + static_cast<size_t>(args.kv_heads) * args.page_tokens;
#pragma unroll
    for (int pass = 0; pass < V_PASSES; ++pass) {
      const uint32_t piece = pass * 64u + lane;
      loaded.value[pass] = *reinterpret_cast<const uint2*>(
          values8 + static_cast<size_t>(piece / GR) * row_stride + (piece % GR) * 8u);
    }
#pragma unroll
    for (int st = 0; st < 2; ++st) {
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        loaded.key[st][ks] = *reinterpret_cast<const uint2*>(
            keys8 + static_cast<size_t>(16u * st + col) * row_stride + 32u * ks +
            8u * quad);
      loaded.key_scale[st] =
          *reinterpret_cast<const uint2*>(key_scales + 16u * st + 4u * quad);
      loaded.value_scale[st] =
          *reinterpret_cast<const uint2*>(value_scales + 16u * st + 4u * quad);
    }
  };
  Q8Tile q8_tile{}, q8_next{};
  if constexpr (AHEAD)
    if (tile_first < tile_last) fetch_q8_tile(tile_first, q8_tile);

  for (uint32_t tile = tile_first; tile < tile_last; ++tile) {
    const uint32_t tile_begin = tile * kF16Tile;
    const bool needs_mask = tile_begin + kF16Tile > first_context_tokens;
    if constexpr (AHEAD) {
      if (tile + 1u < tile_last) fetch_q8_tile(tile + 1u, q8_next);
    } else if constexpr (Q8) {
      fetch_q8_tile(tile, q8_tile);
    }
    // binary16 cache
    const uint16_t* keys = nullptr;
    const uint16_t* values = nullptr;
    if constexpr (!Q8) {
      const void* page_base = uniform_page(args.pages, tile_begin / args.page_tokens);
      const uint32_t tile_slot = tile_begin % args.page_tokens;
      keys = static_cast<const uint16_t*>(page_base) + layer_offset +
             static_cast<size_t>(tile_slot) * row_stride + kv_head * D;
      values = keys + page_values;
    }

    // ---- V tile -> LDS (swizzled rows) ----------------------------------------
#pragma unroll
    for (int pass = 0; pass < kF16Tile * GR / 64; ++pass) {
      const uint32_t piece = pass * 64u + lane;
      const uint32_t token = piece / GR;
      const uint32_t part = piece % GR;
      uint4 value;
      if constexpr (Q8)
        value = __builtin_bit_cast(uint4, int8x8_to_f16(q8_tile.value[pass]));
      else
        value = *reinterpret_cast<const uint4*>(
            values + static_cast<size_t>(token) * row_stride + part * 8u);
      // records no row can see may be uninitialised: a NaN there would
      // survive its zero probability
      if (needs_mask && tile_begin + token >= last_context)
        value = make_uint4(0u, 0u, 0u, 0u);
      *reinterpret_cast<uint4*>(stage_v + (token * GR + (part ^ (2u * (token & 7u)))) *
                                              16u) = value;
    }

    // ---- S = K . Q, online softmax, probabilities per row tile ------------------
    f16x4 p_operand[RT][2];
    f16x8 key_operand[2][KSTEPS];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        if constexpr (Q8)
          key_operand[st][ks] = int8x8_to_f16(q8_tile.key[st][ks]);
        else
          key_operand[st][ks] = *reinterpret_cast<const f16x8*>(
              keys + static_cast<size_t>(16u * st + col) * row_stride + 32u * ks +
              8u * quad);
      }
    // Q8: scales of the lane's tokens 16*st + 4*quad + i; the K scale goes into
    // the score, the V scale into the probability.  Records no row can see
    // may be uninitialised: their V scale (any bit pattern) is replaced by 0.
    float key_scale[2][4];
    f16x4 value_scale[2];
    if constexpr (Q8) {
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const uint2 k = q8_tile.key_scale[st];
        uint2 v = q8_tile.value_scale[st];
        key_scale[st][0] = f16_bits_to_f32(k.x & 0xffffu) * score_unit;
        key_scale[st][1] = f16_bits_to_f32(k.x >> 16) * score_unit;
        key_scale[st][2] = f16_bits_to_f32(k.y & 0xffffu) * score_unit;
        key_scale[st][3] = f16_bits_to_f32(k.y >> 16) * score_unit;
        if (needs_mask) {
          const uint32_t first_token = tile_begin + 16u * st + 4u * quad;
          if (first_token + 0u >= last_context) v.x &= 0xffff0000u;
          if (first_token + 1u >= last_context) v.x &= 0x0000ffffu;
          if (first_token + 2u >= last_context) v.y &= 0xffff0000u;
          if (first_token + 3u >= last_context) v.y &= 0x0000ffffu;
        }
        value_scale[st] = __builtin_bit_cast(f16x4, v);
      }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      asm volatile("" ::: "memory");  // one row tile's query operands at a time
      float score[2][4];
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        f32x4 dot = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const f16x8 q = *reinterpret_cast<const f16x8*>(
              q_operands + (rt * KSTEPS + ks) * 1024);
          dot = __builtin_amdgcn_mfma_f32_16x16x32_f16(key_operand[st][ks], q,
                                                       dot, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
          score[st][i] = dot[i] * (Q8 ? key_scale[st][i] : score_unit);
      }
      if (needs_mask) {
        const uint32_t first_token = tile_begin + 4u * quad;
        const uint32_t limit = exchange_limit[16 * rt + col];
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (first_token + 16u * st + i >= limit) score[st][i] = -INFINITY;
      }
      // the running maximum follows the tile maximum only when that is more
      // than 8 (log2 units) ahead: probabilities stay below 2^8
      float tile_max = score[0][0];
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int i = 0; i < 4; ++i) tile_max = fmaxf(tile_max, score[st][i]);
      tile_max = quad_row_max(tile_max);
      const bool grew = tile_max - running_max[rt] > 8.0f;
      if (__builtin_amdgcn_ballot_w64(grew) != 0ull) {
        const float new_max = fmaxf(running_max[rt], tile_max);
        if (tile != tile_first) {
          const float factor = __builtin_amdgcn_exp2f(running_max[rt] - new_max);
          running_sum[rt] *= factor;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) out[dt][rt][i] *= factor;
        }
        running_max[rt] = new_max;
      }
      float sum = 0.0f;
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const _Float16 p = static_cast<_Float16>(
              __builtin_amdgcn_exp2f(score[st][i] - running_max[rt]));
          p_operand[rt][st][i] = p;
          sum += static_cast<float>(p);
        }
      if constexpr (Q8) {
#pragma unroll
        for (int st = 0; st < 2; ++st) p_operand[rt][st] *= value_scale[st];
      }
      running_sum[rt] += sum;
    }

    // ---- O^T += V^T . P^T -------------------------------------------------------
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int st = 0; st < 2; ++st) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        // granule 2*dt + (j >> 1) of the row, swizzled; (j >> 1) and the byte
        // offset of (j & 1) are already in read_base
        const uint32_t address = st * 16u * (GR * 16u) + read_base +
                                 ((2u * dt) ^ (2u * read_swizzle)) * 16u;
        typedef short i16x4 __attribute__((ext_vector_type(4)));
        const f16x4 v = __builtin_bit_cast(
            f16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                       (__attribute__((address_space(3))) i16x4*)(stage_v +
                                                                  address)));
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          out[dt][rt] = __builtin_amdgcn_mfma_f32_16x16x16f16(
              v, p_operand[rt][st], out[dt][rt], 0, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();
    if constexpr (AHEAD) q8_tile = q8_next;
  }

#pragma unroll
  for (int rt = 0; rt < RT; ++rt) running_sum[rt] = quad_row_sum(running_sum[rt]);

  static_assert(kSplitWaves * RT * 512 <= sizeof(exchange), "summaries fit");
  const PartialTarget target{args.partial_maxima, args.partial_sums,
                             args.partial_outputs, args.maximum_splits,
                             args.query_heads, kv_head, split, group,
                             matrix_rows};
  merge_wave_states<D, RT>(running_max, running_sum, out,
                           reinterpret_cast<float*>(stage),
                           reinterpret_cast<float2*>(exchange), wave, lane,
                           target);
}

// The binary16 cache at head_dim 128, software-pipelined: the kernel above
// asks for a tile when it needs it and so leaves the memory system idle while
// it computes.  Here a tile's K rows and V rows travel global -> LDS with
// direct loads (no registers) into wave-private staging areas, and each area is
// refilled with the next tile as soon as the current one has been read out of
// it, so a wave always has a K or a V tile in flight.  Arithmetic, tile size and
// the order of every sum are those of the kernel above: results are bit-equal.
//
// LDS granules (16 bytes) are swizzled against bank conflicts on the way in, by
// the choice of which global granule a lane fetches for its LDS slot: K row r
// keeps granule g at g ^ (r & 15) (the A-operand read takes one granule from
// each of 16 consecutive rows), V row t at g ^ (2 * (t & 7)) as above.
template <int RT>
__global__ __launch_bounds__(kSplitWaves * 64) void f16_attention_split_d128_kernel(
    const F16SplitArgs args) {
  constexpr int D = 128;
  constexpr int KSTEPS = D / 32;
  constexpr int DT = D / 16;
  constexpr int GR = D / 8;                    // 16-byte granules per row
  constexpr int TILE_BYTES = kF16Tile * D * 2;  // K (or V) rows of a tile
  constexpr int STAGE = 2 * TILE_BYTES;        // a wave's K area, then its V area
  constexpr int LOADS = TILE_BYTES / 1024;     // direct loads per area and tile
  constexpr int UNITS = RT * KSTEPS;
  constexpr int EXCHANGE_Q = UNITS * 1024 + RT * 64;
  constexpr int EXCHANGE_MERGE = kSplitWaves * RT * 512;
  static_assert(kSplitWaves * STAGE >= kSplitWaves * kSplitWaves * 1024,
                "the merge pool fits the staging memory");
  __shared__ __attribute__((aligned(16))) uint8_t stage[kSplitWaves * STAGE];
  __shared__ __attribute__((aligned(16)))
  uint8_t exchange[EXCHANGE_Q > EXCHANGE_MERGE ? EXCHANGE_Q : EXCHANGE_MERGE];

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t col = lane & 15u;
  const uint32_t quad = lane >> 4;
  const uint32_t kv_head = blockIdx.x;
  const uint32_t split = blockIdx.y;
  const uint32_t group = args.query_heads / args.kv_heads;
  const uint32_t matrix_rows = args.rows * group;
  const uint32_t first_context_tokens =
      args.device_positions ? uniform_word(args.device_positions, 2u)
                            : args.first_context_tokens;
  const uint32_t last_context = first_context_tokens + args.rows - 1u;
  const uint32_t context_tiles = (last_context + kF16Tile - 1u) / kF16Tile;
  uint32_t tile_first, tile_last;
  wave_tile_range(context_tiles, kF16Tile, args.split_tokens, split, gridDim.y,
                  wave, tile_first, tile_last);

  uint8_t* stage_k = stage + wave * STAGE;
  uint8_t* stage_v = stage_k + TILE_BYTES;
  const uint32_t stage_k_lds =
      __builtin_amdgcn_readfirstlane(lds_address(stage_k));
  const uint32_t stage_v_lds = stage_k_lds + TILE_BYTES;
  const uint32_t row_bytes = args.kv_heads * D * 2u;   // bytes between tokens
  const size_t page_bytes =
      static_cast<size_t>(args.page_tokens) * row_bytes;   // K (or V) of a layer

  // Load `pass` of an area fills LDS slots [64 * pass, +64): lane l holds row
  // 4 * pass + l / 16, slot granule l % 16, and fetches the global granule that
  // the swizzle puts there.  The lane's share of the address depends on
  // pass % 4 (K) or pass % 2 (V) only.
  auto stage_rows = [&](uint32_t tile, bool values) {
    const uint32_t lane_now = fresh_lane_index();
    const uint32_t lane_row = lane_now >> 4;
    const uint32_t granule = lane_now & 15u;
    const uint32_t tile_begin = tile * kF16Tile;
    const uint8_t* page = static_cast<const uint8_t*>(
        uniform_page(args.pages, tile_begin / args.page_tokens));
    const uint8_t* rows = uniform_pointer(
        page + (static_cast<size_t>(args.layer) * 2u + (values ? 1u : 0u)) * page_bytes +
        static_cast<size_t>(tile_begin % args.page_tokens) * row_bytes +
        kv_head * (D * 2u));
    const uint32_t target = values ? stage_v_lds : stage_k_lds;
#pragma unroll
    for (int pass = 0; pass < LOADS; ++pass) {
      const uint32_t row = 4u * (pass % 4) + lane_row;   // row & 15
      const uint32_t source_granule =
          values ? granule ^ (2u * (row & 7u)) : granule ^ row;
      copy16_to_lds(rows + static_cast<size_t>(4 * pass) * row_bytes,
                    lane_row * row_bytes + source_granule * 16u,
                    target + pass * 1024);
    }
  };
  // the wave's first tile sets out before the query work below
  if (tile_first < tile_last) {
    stage_rows(tile_first, false);
    stage_rows(tile_first, true);
  }

  // ---- query operands (B side of S = K.Q) in binary16, built once -------------
  uint32_t* exchange_limit = reinterpret_cast<uint32_t*>(exchange + UNITS * 1024);
  for (uint32_t unit = wave; unit < static_cast<uint32_t>(UNITS);
       unit += kSplitWaves) {
    const uint32_t rt = unit / KSTEPS;
    const uint32_t step = unit % KSTEPS;
    const uint32_t matrix_row = 16u * rt + col;
    const bool valid = matrix_row < matrix_rows;
    const uint32_t row = valid ? matrix_row / group : 0u;
    const uint32_t head = kv_head * group + (valid ? matrix_row % group : 0u);
    const float* source =
        args.query +
        (static_cast<size_t>(row) * args.query_heads + head) * args.query_stride +
        32u * step + 8u * quad;
    f16x8 operand;
#pragma unroll
    for (int piece = 0; piece < 2; ++piece) {
      float4 loaded = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if (valid) loaded = *reinterpret_cast<const float4*>(source + 4 * piece);
      operand[4 * piece + 0] = static_cast<_Float16>(loaded.x);
      operand[4 * piece + 1] = static_cast<_Float16>(loaded.y);
      operand[4 * piece + 2] = static_cast<_Float16>(loaded.z);
      operand[4 * piece + 3] = static_cast<_Float16>(loaded.w);
    }
    *reinterpret_cast<f16x8*>(exchange + unit * 1024u + lane * 16u) = operand;
    if (step == 0u && quad == 0u)
      exchange_limit[16u * rt + col] = first_context_tokens + row;
  }
  __syncthreads();
  const uint8_t* q_operands = exchange + lane * 16u;
  const float score_unit =
      1.4426950408889634f / sqrtf(static_cast<float>(D));  // log2 units

  // K operand of (st, ks): row 16 * st + col, granule 4 * ks + quad
  const uint8_t* key_read = stage_k + col * (GR * 16u);
  // V, transposing read: see the kernel above
  const uint32_t read_token = 4u * quad + (col >> 2);
  const uint32_t read_swizzle = read_token & 7u;
  const uint32_t read_base =
      read_token * (GR * 16u) + ((col >> 1) & 1u) * 16u + (col & 1u) * 8u;

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

  // Loads in flight at the top of an iteration, oldest first: this tile's K,
  // this tile's V.
  for (uint32_t tile = tile_first; tile < tile_last; ++tile) {
    const uint32_t tile_begin = tile * kF16Tile;
    const bool needs_mask = tile_begin + kF16Tile > first_context_tokens;
    const bool has_next = tile + 1u < tile_last;

    // ---- K rows out of LDS, the next tile's K on its way ------------------------
    vmem_wait<LOADS>();
    f16x8 key_operand[2][KSTEPS];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        key_operand[st][ks] = *reinterpret_cast<const f16x8*>(
            key_read + st * 16 * (GR * 16) + (((4u * ks + quad) ^ col) * 16u));
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (has_next) stage_rows(tile + 1u, false);

    // ---- S = K . Q, online softmax, probabilities per row tile ------------------
    f16x4 p_operand[RT][2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      asm volatile("" ::: "memory");  // one row tile's query operands at a time
      float score[2][4];
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        f32x4 dot = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const f16x8 q = *reinterpret_cast<const f16x8*>(
              q_operands + (rt * KSTEPS + ks) * 1024);
          dot = __builtin_amdgcn_mfma_f32_16x16x32_f16(key_operand[st][ks], q,
                                                       dot, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) score[st][i] = dot[i] * score_unit;
      }
      if (needs_mask) {
        const uint32_t first_token = tile_begin + 4u * quad;
        const uint32_t limit = exchange_limit[16 * rt + col];
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (first_token + 16u * st + i >= limit) score[st][i] = -INFINITY;
      }
      float tile_max = score[0][0];
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int i = 0; i < 4; ++i) tile_max = fmaxf(tile_max, score[st][i]);
      tile_max = quad_row_max(tile_max);
      const bool grew = tile_max - running_max[rt] > 8.0f;
      if (__builtin_amdgcn_ballot_w64(grew) != 0ull) {
        const float new_max = fmaxf(running_max[rt], tile_max);
        if (tile != tile_first) {
          const float factor = __builtin_amdgcn_exp2f(running_max[rt] - new_max);
          running_sum[rt] *= factor;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) out[dt][rt][i] *= factor;
        }
        running_max[rt] = new_max;
      }
      float sum = 0.0f;
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const _Float16 p = static_cast<_Float16>(
              __builtin_amdgcn_exp2f(score[st][i] - running_max[rt]));
          p_operand[rt][st][i] = p;
          sum += static_cast<float>(p);
        }
      running_sum[rt] += sum;
    }

    // ---- V rows have arrived; O^T += V^T . P^T ----------------------------------
    // in flight, oldest first: this tile's V, the next tile's K
    if (has_next)
      vmem_wait<LOADS>();
    else
      vmem_wait<0>();
    if (needs_mask) {
      // records no row can see may be uninitialised: a NaN there would
      // survive its zero probability
#pragma unroll
      for (int pass = 0; pass < LOADS; ++pass) {
        const uint32_t token = 4u * pass + quad;
        if (tile_begin + token >= last_context)
          *reinterpret_cast<uint4*>(stage_v + (pass * 64u + lane) * 16u) =
              make_uint4(0u, 0u, 0u, 0u);
      }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int st = 0; st < 2; ++st) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const uint32_t address = st * 16u * (GR * 16u) + read_base +
                                 ((2u * dt) ^ (2u * read_swizzle)) * 16u;
        typedef short i16x4 __attribute__((ext_vector_type(4)));
        const f16x4 v = __builtin_bit_cast(
            f16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                       (__attribute__((address_space(3))) i16x4*)(stage_v +
                                                                  address)));
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          out[dt][rt] = __builtin_amdgcn_mfma_f32_16x16x16f16(
              v, p_operand[rt][st], out[dt][rt], 0, 0, 0);
      }
    }
    // every V read has returned before the area is refilled
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (has_next) stage_rows(tile + 1u, true);
  }

#pragma unroll
  for (int rt = 0; rt < RT; ++rt) running_sum[rt] = quad_row_sum(running_sum[rt]);

  const PartialTarget target{args.partial_maxima, args.partial_sums,
                             args.partial_outputs, args.maximum_splits,
                             args.query_heads, kv_head, split, group,
                             matrix_rows};
  merge_wave_states<D, RT>(running_max, running_sum, out,
                           reinterpret_cast<float*>(stage),
                           reinterpret_cast<float2*>(exchange), wave, lane,
                           target);
}

int32_t launch_f16_split_d128(const F16SplitArgs& args, uint32_t row_tiles,
                              dim3 grid, hipStream_t stream) {
  switch (row_tiles) {
    case 1:
      f16_attention_split_d128_kernel<1><<<grid, kSplitWaves * 64, 0, stream>>>(args);
      break;
    case 2:
      f16_attention_split_d128_kernel<2><<<grid, kSplitWaves * 64, 0, stream>>>(args);
      break;
    default:
      f16_attention_split_d128_kernel<3><<<grid, kSplitWaves * 64, 0, stream>>>(args);
      break;
  }
  return launched("F16 attention split");
}

template <int D, bool Q8 = false>
int32_t launch_f16_split(const F16SplitArgs& args, uint32_t row_tiles, dim3 grid,
                         hipStream_t stream) {
  switch (row_tiles) {
    case 1:
      f16_attention_split_kernel<D, 1, Q8>
          <<<grid, kSplitWaves * 64, 0, stream>>>(args);
      break;
    case 2:
      f16_attention_split_kernel<D, 2, Q8>
          <<<grid, kSplitWaves * 64, 0, stream>>>(args);
      break;
    default:
      if constexpr (D == 128) {
        f16_attention_split_kernel<D, 3, Q8>
            <<<grid, kSplitWaves * 64, 0, stream>>>(args);
        break;
      } else {
        return fail(QLLM_INVALID_ARGUMENT,
                    "F16 attention: three row tiles need head_dim 128");
      }
  }
  return launched("F16 attention split");
}

}  // namespace

// defined with the Q4H kernels
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
                                 hipStream_t stream);
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
  if (!launch || !launch->query || !launch->device_pages || !launch->output ||
      (reinterpret_cast<uintptr_t>(launch->query) & 15u) ||
      launch->query_stride % 4u || !launch->partial_maxima ||
      !launch->partial_sums || !launch->partial_outputs ||
      !launch->first_context_tokens || !launch->rows ||
      !launch->device_page_tokens || launch->device_page_tokens % kF16Tile ||
      !launch->query_heads || !launch->kv_heads ||
      launch->query_heads % launch->kv_heads ||
      (launch->head_dim != 128u && launch->head_dim != 256u) ||
      launch->split_tokens % kF16Tile || !launch->maximum_splits ||
      launch->maximum_splits > 2048u ||
      launch->query_stride <
          (launch->output_gated ? 2u : 1u) * launch->head_dim ||
      (launch->output_kind != QLLM_OUT_F32 &&
       launch->output_kind != QLLM_OUT_BF16) ||
      launch->first_context_tokens > 0xffffffffu - (launch->rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid F16 paged attention");
  const uint32_t group = launch->query_heads / launch->kv_heads;
  const uint32_t row_tiles = (launch->rows * group + 15u) / 16u;
  if (row_tiles > 3u || (launch->head_dim == 256u && row_tiles > 2u))
    return fail(QLLM_INVALID_ARGUMENT,
                "F16 paged attention: rows * (query_heads/kv_heads) exceeds "
                "48 (32 at head_dim 256)");
  const uint32_t last_context = launch->first_context_tokens + launch->rows - 1u;
  const uint32_t splits =
      launch->split_tokens
          ? (last_context + launch->split_tokens - 1u) / launch->split_tokens
          : launch->maximum_splits;
  if (splits > launch->maximum_splits)
    return fail(QLLM_INVALID_ARGUMENT,
                "F16 paged attention: context needs more splits than "
                "maximum_splits");
  F16SplitArgs args{};
  args.query = launch->query;
  args.query_stride = launch->query_stride;
  args.pages = launch->device_pages;
  args.partial_maxima = launch->partial_maxima;
  args.partial_sums = launch->partial_sums;
  args.partial_outputs = launch->partial_outputs;
  args.first_context_tokens = launch->first_context_tokens;
  args.rows = launch->rows;
  args.layer = launch->device_page_layer;
  args.page_tokens = launch->device_page_tokens;
  args.query_heads = launch->query_heads;
  args.kv_heads = launch->kv_heads;
  args.split_tokens = launch->split_tokens;
  args.maximum_splits = launch->maximum_splits;
  const dim3 grid(launch->kv_heads, splits);
  const hipStream_t stream = as_stream(launch->stream);
  const int32_t status =
      launch->head_dim == 128u
          ? launch_f16_split_d128(args, row_tiles, grid, stream)
          : launch_f16_split<256>(args, row_tiles, grid, stream);
  if (status != QLLM_OK) return status;
  return launch_attention_combine(
      launch->query, launch->query_stride, launch->output_gated,
      launch->partial_maxima, launch->partial_sums, launch->partial_outputs,
      launch->output, launch->output_kind, launch->first_context_tokens,
      launch->maximum_splits, launch->split_tokens, launch->rows,
      launch->query_heads, launch->head_dim, nullptr, stream);
}

extern "C" int32_t qllm_attention_paged_f16_batched(
    const qllm_f16_attention_launch* launch, uint32_t batch_rows) {
  if (!launch || !launch->query || !launch->device_pages || !launch->output ||
      (reinterpret_cast<uintptr_t>(launch->query) & 15u) ||
      launch->query_stride % 4u || !launch->partial_maxima ||
      !launch->partial_sums || !launch->partial_outputs ||
      !launch->first_context_tokens || !launch->rows || !batch_rows ||
      !launch->device_page_tokens || launch->device_page_tokens % kF16Tile ||
      !launch->query_heads || !launch->kv_heads ||
      launch->query_heads % launch->kv_heads ||
      (launch->head_dim != 128u && launch->head_dim != 256u) ||
      launch->split_tokens % kF16Tile || !launch->maximum_splits ||
      launch->maximum_splits > 2048u ||
      launch->query_stride <
          (launch->output_gated ? 2u : 1u) * launch->head_dim ||
      (launch->output_kind != QLLM_OUT_F32 &&
       launch->output_kind != QLLM_OUT_BF16) ||
      launch->rows > 65535u ||
      launch->first_context_tokens > 0xffffffffu - (launch->rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid batched F16 paged attention");
  const uint32_t group = launch->query_heads / launch->kv_heads;
  const uint32_t row_tiles =
      ((batch_rows < launch->rows ? batch_rows : launch->rows) * group + 15u) / 16u;
  if (row_tiles > 3u || (launch->head_dim == 256u && row_tiles > 2u))
    return fail(QLLM_INVALID_ARGUMENT,
                "batched F16 paged attention: batch_rows * (query_heads/kv_heads) "
                "exceeds 48 (32 at head_dim 256)");
  const uint32_t batches = (launch->rows + batch_rows - 1u) / batch_rows;
  const uint32_t last_context = launch->first_context_tokens + launch->rows - 1u;
  const uint32_t splits =
      launch->split_tokens
          ? (last_context + launch->split_tokens - 1u) / launch->split_tokens
          : launch->maximum_splits;
  if (splits > launch->maximum_splits)
    return fail(QLLM_INVALID_ARGUMENT,
                "batched F16 paged attention: context needs more splits than "
                "maximum_splits");
  F16SplitArgs args{};
  args.query = launch->query;
  args.query_stride = launch->query_stride;
  args.pages = launch->device_pages;
  args.partial_maxima = launch->partial_maxima;
  args.partial_sums = launch->partial_sums;
  args.partial_outputs = launch->partial_outputs;
  args.first_context_tokens = launch->first_context_tokens;
  args.rows = launch->rows;
  args.layer = launch->device_page_layer;
  args.page_tokens = launch->device_page_tokens;
  args.query_heads = launch->query_heads;
  args.kv_heads = launch->kv_heads;
  args.split_tokens = launch->split_tokens;
  args.maximum_splits = launch->maximum_splits;
  args.batch_rows = batch_rows;
  const dim3 grid(launch->kv_heads, splits, batches);
  const hipStream_t stream = as_stream(launch->stream);
  const int32_t status =
      launch->head_dim == 128u ? launch_f16_split<128>(args, row_tiles, grid, stream)
                               : launch_f16_split<256>(args, row_tiles, grid, stream);
  if (status != QLLM_OK) return status;
  return launch_attention_combine(
      launch->query, launch->query_stride, launch->output_gated,
      launch->partial_maxima, launch->partial_sums, launch->partial_outputs,
      launch->output, launch->output_kind, launch->first_context_tokens,
      launch->maximum_splits, launch->split_tokens, launch->rows,
      launch->query_heads, launch->head_dim, nullptr, stream);
}

extern "C" size_t qllm_q8_layer_bytes(uint32_t page_tokens, uint32_t kv_heads,
                                      uint32_t head_dim) {
  return static_cast<size_t>(page_tokens) * kv_heads * 2u * (head_dim + 2u);
}

extern "C" int32_t qllm_store_kv_paged_q8_batch(
    const float* key, const float* value, const void* const* page_table,
    size_t page_offset_bytes, uint32_t page_tokens,
    uint32_t first_cache_position, uint32_t rows, uint32_t kv_heads,
    uint32_t head_dim, void* stream) {
  if (!key || !value || !page_table || !page_tokens || !rows || !kv_heads ||
      !head_dim || page_offset_bytes % 16u ||
      first_cache_position > 0xffffffffu - (rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid Q8 K/V store");
  q8_store_kernel<<<dim3(kv_heads, rows), 64, 0, as_stream(stream)>>>(
      key, value, page_table, page_offset_bytes, page_tokens,
      first_cache_position, kv_heads, head_dim, nullptr);
  return launched("Q8 K/V store");
}

extern "C" int32_t qllm_store_kv_paged_q8_batch_deferred(
    const float* key, const float* value, const void* const* page_table,
    size_t page_offset_bytes, uint32_t page_tokens,
    const uint32_t* device_positions, uint32_t rows, uint32_t kv_heads,
    uint32_t head_dim, void* stream) {
  if (!key || !value || !page_table || !page_tokens || !device_positions ||
      !rows || !kv_heads || !head_dim || page_offset_bytes % 16u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid deferred Q8 K/V store");
  q8_store_kernel<<<dim3(kv_heads, rows), 64, 0, as_stream(stream)>>>(
      key, value, page_table, page_offset_bytes, page_tokens, 0u, kv_heads,
      head_dim, device_positions);
  return launched("deferred Q8 K/V store");
}

extern "C" int32_t qllm_attention_paged_q8(const qllm_q8_attention_launch* launch) {
  if (!launch || !launch->query || !launch->device_pages || !launch->output ||
      (reinterpret_cast<uintptr_t>(launch->query) & 15u) ||
      launch->query_stride % 4u || !launch->partial_maxima ||
      !launch->partial_sums || !launch->partial_outputs ||
      (!launch->device_positions && !launch->first_context_tokens) ||
      !launch->rows ||
      !launch->page_tokens || launch->page_tokens % kF16Tile ||
      launch->page_offset_bytes % 16u || !launch->query_heads ||
      !launch->kv_heads || launch->query_heads % launch->kv_heads ||
      (launch->head_dim != 128u && launch->head_dim != 256u) ||
      launch->split_tokens % kF16Tile || !launch->maximum_splits ||
      launch->maximum_splits > 2048u ||
      launch->query_stride <
          (launch->output_gated ? 2u : 1u) * launch->head_dim ||
      (launch->output_kind != QLLM_OUT_F32 &&
       launch->output_kind != QLLM_OUT_BF16) ||
      launch->first_context_tokens > 0xffffffffu - (launch->rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid Q8 paged attention");
  const uint32_t group = launch->query_heads / launch->kv_heads;
  const uint32_t row_tiles = (launch->rows * group + 15u) / 16u;
  if (row_tiles > 3u || (launch->head_dim == 256u && row_tiles > 2u))
    return fail(QLLM_INVALID_ARGUMENT,
                "Q8 paged attention: rows * (query_heads/kv_heads) exceeds "
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
                "Q8 paged attention: context needs more splits than "
                "maximum_splits");
  F16SplitArgs args{};
  args.query = launch->query;
  args.query_stride = launch->query_stride;
  args.pages = launch->device_pages;
  args.partial_maxima = launch->partial_maxima;
  args.partial_sums = launch->partial_sums;
  args.partial_outputs = launch->partial_outputs;
  args.first_context_tokens = launch->first_context_tokens;
  args.rows = launch->rows;
  args.page_tokens = launch->page_tokens;
  args.query_heads = launch->query_heads;
  args.kv_heads = launch->kv_heads;
  args.split_tokens = launch->split_tokens;
  args.maximum_splits = launch->maximum_splits;
  args.page_offset = launch->page_offset_bytes;
  args.device_positions = launch->device_positions;
  const dim3 grid(launch->kv_heads, splits);
  const hipStream_t stream = as_stream(launch->stream);
  const int32_t status =
      launch->head_dim == 128u
          ? launch_f16_split<128, true>(args, row_tiles, grid, stream)
          : launch_f16_split<256, true>(args, row_tiles, grid, stream);
  if (status != QLLM_OK) return status;
  return launch_attention_combine(
      launch->query, launch->query_stride, launch->output_gated,
      launch->partial_maxima, launch->partial_sums, launch->partial_outputs,
      launch->output, launch->output_kind, launch->first_context_tokens,
      launch->maximum_splits, launch->split_tokens, launch->rows,
      launch->query_heads, launch->head_dim, launch->device_positions, stream);
}

extern "C" int32_t qllm_attention_paged_q8_batched(
    const qllm_q8_attention_launch* launch, uint32_t batch_rows) {
  if (!launch || !launch->query || !launch->device_pages || !launch->output ||
      (reinterpret_cast<uintptr_t>(launch->query) & 15u) ||
      launch->query_stride % 4u || !launch->partial_maxima ||
      !launch->partial_sums || !launch->partial_outputs ||
      launch->device_positions || !launch->first_context_tokens ||
      !launch->rows || !batch_rows || launch->rows > 65535u ||
      !launch->page_tokens || launch->page_tokens % kF16Tile ||
      launch->page_offset_bytes % 16u || !launch->query_heads ||
      !launch->kv_heads || launch->query_heads % launch->kv_heads ||
      (launch->head_dim != 128u && launch->head_dim != 256u) ||
      launch->split_tokens % kF16Tile || !launch->maximum_splits ||
      launch->maximum_splits > 2048u ||
      launch->query_stride <
          (launch->output_gated ? 2u : 1u) * launch->head_dim ||
      (launch->output_kind != QLLM_OUT_F32 &&
       launch->output_kind != QLLM_OUT_BF16) ||
      launch->first_context_tokens > 0xffffffffu - (launch->rows - 1u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid batched Q8 paged attention");
  const uint32_t group = launch->query_heads / launch->kv_heads;
  const uint32_t row_tiles =
      ((batch_rows < launch->rows ? batch_rows : launch->rows) * group + 15u) / 16u;
  if (row_tiles > 3u || (launch->head_dim == 256u && row_tiles > 2u))
    return fail(QLLM_INVALID_ARGUMENT,
                "batched Q8 paged attention: batch_rows * (query_heads/kv_heads) "
                "exceeds 48 (32 at head_dim 256)");
  const uint32_t batches = (launch->rows + batch_rows - 1u) / batch_rows;
  const uint32_t last_context = launch->first_context_tokens + launch->rows - 1u;
  const uint32_t splits =
      launch->split_tokens
          ? (last_context + launch->split_tokens - 1u) / launch->split_tokens
          : launch->maximum_splits;
  if (splits > launch->maximum_splits)
    return fail(QLLM_INVALID_ARGUMENT,
                "batched Q8 paged attention: context needs more splits than "
                "maximum_splits");
  F16SplitArgs args{};
  args.query = launch->query;
  args.query_stride = launch->query_stride;
  args.pages = launch->device_pages;
  args.partial_maxima = launch->partial_maxima;
  args.partial_sums = launch->partial_sums;
  args.partial_outputs = launch->partial_outputs;
  args.first_context_tokens = launch->first_context_tokens;
  args.rows = launch->rows;
  args.page_tokens = launch->page_tokens;
  args.query_heads = launch->query_heads;
  args.kv_heads = launch->kv_heads;
  args.split_tokens = launch->split_tokens;
  args.maximum_splits = launch->maximum_splits;
  args.page_offset = launch->page_offset_bytes;
  args.batch_rows = batch_rows;
  const dim3 grid(launch->kv_heads, splits, batches);
  const hipStream_t stream = as_stream(launch->stream);
  const int32_t status =
      launch->head_dim == 128u
          ? launch_f16_split<128, true>(args, row_tiles, grid, stream)
          : launch_f16_split<256, true>(args, row_tiles, grid, stream);
  if (status != QLLM_OK) return status;
  return launch_attention_combine(
      launch->query, launch->query_stride, launch->output_gated,
      launch->partial_maxima, launch->partial_sums, launch->partial_outputs,
      launch->output, launch->output_kind, launch->first_context_tokens,
      launch->maximum_splits, launch->split_tokens, launch->rows,
      launch->query_heads, launch->head_dim, nullptr, stream);
}
