// FP4 (E2M1, block-scaled) weight GEMM for small batches (M <= 8 rows).
//
// Replaces fp4_gemv_q8_batch_weight_reuse / fp4_gemv_q8_batch5_tensor_core_kernel
// and fp4_gemm_bf16_block32 of the reference
// (runtime/src/cuda/transformer_kernels.cu:1025-1275, 1436-1541, 7400-7593).
//
// Two kernels:
//  * fp4_gemm_mfma_kernel  - the hot path.  At M=5 a verify step needs
//    16 flop per weight byte; at HBM speed that is ~130 TFLOP/s, above what
//    the vector ALUs deliver, so the contraction runs on the matrix cores,
//    on v_mfma_f32_16x16x32_bf16: 16 weight rows on the N side, 32 columns of
//    K - two 16-blocks with scales of their own - which are kept apart on the
//    M side (MFMA rows 0..7 carry the batch for the first block, rows 8..15
//    for the second), so that each block sum is scaled by its own scale before
//    the halves are added.  Packed nibbles stream from HBM with one 16-byte
//    load per lane (one contiguous KiB per wave in the tiled layout), are
//    expanded in registers by v_cvt_scalef32_pk_bf16_fp4 (exact), and the
//    activations of a chunk ride along through a wave-private LDS ring; a
//    workgroup's waves interleave over the 64-column chunks of K and meet in
//    LDS once, after the loop.
//  * fp4_gemv_generic_kernel - any shape/scheme/activation type (the Q8
//    integer form of the reference included), one wave per output row; used
//    for shapes the MFMA kernel does not take.  The provider never selects it
//    for a K that is a multiple of 64.
#include "common.hpp"

#include <algorithm>
#include <cstdlib>

namespace qllm {
namespace {

constexpr int kSchemeUe8m0 = QLLM_SCALE_UE8M0_BLOCK32;
constexpr int kSchemeF16 = QLLM_SCALE_F16_BLOCK16;

constexpr uint32_t kChunk = 64;            // K elements per wave step

// eight int8 codes -> the same integers as bf16 (exact: seven bits)
__device__ __forceinline__ bf16x8 q8x8_to_bf16(uint2 bytes) {
  const uint32_t word[2] = {bytes.x, bytes.y};
  bf16x8 result;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int32_t code =
        static_cast<int32_t>(word[k >> 2] << (24 - 8 * (k & 3))) >> 24;
    const uint32_t bits = __builtin_bit_cast(uint32_t, static_cast<float>(code));
    result[k] = __builtin_bit_cast(__bf16, static_cast<uint16_t>(bits >> 16));
  }
  return result;
}

__device__ __forceinline__ bf16x8 expand_fp4x8(uint32_t packed, float scale) {
  const bf16x2 p0 = fp4x2_to_bf16<0>(packed, scale);
  const bf16x2 p1 = fp4x2_to_bf16<1>(packed, scale);
  const bf16x2 p2 = fp4x2_to_bf16<2>(packed, scale);
  const bf16x2 p3 = fp4x2_to_bf16<3>(packed, scale);
  bf16x8 result;
  result[0] = p0[0]; result[1] = p0[1];
  result[2] = p1[0]; result[3] = p1[1];
  result[4] = p2[0]; result[5] = p2[1];
  result[6] = p3[0]; result[7] = p3[1];
  return result;
}

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

// Streaming (non-temporal) loads: weights are read once per step.
__device__ __forceinline__ uint4 load_stream16(const uint8_t* address) {
  const u32x4 v =
      __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(address));
  return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint2 load_stream8(const uint8_t* address) {
  const u32x2 v =
      __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(address));
  return make_uint2(v[0], v[1]);
}

struct GemmTile {
  const uint8_t* weights;
  const uint8_t* scales;
};

struct GemmArgs {
  GemmTile tile[2];
  const uint16_t* activations;  // bf16 [batch, padded_columns]; Q8: int8
  // Q8 kernels: the scale of every activation row, applied to its sums
  const float* activation_scales;
  void* output;
  const float* residual;
  uint32_t rows;
  uint32_t padded_columns;
  uint32_t output_kind;
  uint32_t tile_rows;           // weight rows per tile: even, 8..32
  // Optional split of the output rows over up to three buffers (the q, k and
  // v projections stored as one matrix): segment s takes the next
  // segment_rows[s] rows.  segments == 0: everything goes to `output`.
  // Cut of K over several workgroups per tile: workgroup (tile, split) sums the
  // split's share of the 64-column chunks and writes an F32 partial to
  // output + split * batch * rows (no residual, no segments); the consumer
  // adds the partials.  0 or 1: one workgroup per tile.
  uint32_t k_splits;
  uint32_t segments;
  uint32_t segment_rows[3];
  uint32_t segment_kind[3];
  void* segment_output[3];
  // Balanced tail: a launch whose tile count is not a multiple of the CU
  // count leaves a few CUs with one workgroup more than the rest, and the
  // launch lasts as long as they do.  With balance_splits > 1 the tiles from
  // balance_first_tile on are cut along K over balance_splits small
  // workgroups each (grid = balance_first_tile + extra tiles * splits), so
  // that every CU gets the same share.  A small workgroup leaves its sums in
  // balance_partials [extra tile][split][TILES][items] (write-through stores)
  // and bumps the tile's counter; the one that finds it at splits - 1 adds the
  // partials in split order, whichever workgroup it is, runs the epilogue and
  // puts the counter back to zero.  Nobody waits for anybody.
  uint32_t balance_first_tile;
  uint32_t balance_splits;
  float* balance_partials;
  uint32_t* balance_counters;
  // Stage 1 of the arg-max over the output rows (a head's logits), taken from
  // the epilogue: with argmax_values (TILES == 1, F32 output, one workgroup
  // per tile) the tile's best (value, output row) of every batch row goes to
  // argmax_values / argmax_indices [batch][tiles] - larger value first, equal
  // values by lower row, NaN never - and a one-block launch picks the winner.
  float* argmax_values;
  uint32_t* argmax_indices;
};

// Epilogue store of one value.
__device__ __forceinline__ void store_output(void* output, uint32_t kind,
                                             size_t index, float value) {
  if (kind == QLLM_OUT_BF16)
    static_cast<uint16_t*>(output)[index] =
        static_cast<uint16_t>(f32_to_bf16_bits(value));
  else if (kind == QLLM_OUT_F32_BF16_ROUNDED)
    static_cast<float*>(output)[index] = bf16_round(value);
  else
    static_cast<float*>(output)[index] = value;
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

// Balanced tail (GemmArgs::balance_*): most small workgroups per cut tile, and
// the layout of the workspace that serves it - one counter per cut tile, then
// the partials.
constexpr uint32_t kMaxBalanceSplits = 8;
constexpr uint32_t kMaxBalanceTiles = 1024;   // one counter each
constexpr size_t kBalanceCounterBytes = 4096;
constexpr size_t kBalanceWorkspaceBytes = size_t{4} << 20;
// floats of one small workgroup's hand-over: a slot per tile of the pair
constexpr size_t balance_slot_floats(bool pair) { return (pair ? 2u : 1u) * 256u; }

bool balance_workspace_ok(const void* workspace, size_t bytes) {
  return workspace && bytes >= kBalanceWorkspaceBytes &&
         reinterpret_cast<uintptr_t>(workspace) % 16u == 0u;
}

// 4x4 transpose of dwords across the four 16-lane rows of a wave: on return
// register d of row c holds what register c of row d held.
__device__ __forceinline__ void transpose_rows4(uint32_t (&v)[4]) {
  const auto a = __builtin_amdgcn_permlane32_swap(v[0], v[2], false, false);
  const auto b = __builtin_amdgcn_permlane32_swap(v[1], v[3], false, false);
  const auto c = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);
  const auto d = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
  v[0] = c[0]; v[1] = c[1]; v[2] = d[0]; v[3] = d[1];
}

// Workgroup = WAVES waves, one tile of h = tile_rows weight rows (for the fused
// SwiGLU pair: the gate tile and the up tile of the same rows).  Its waves
// interleave over 64-column chunks of K (wave w takes chunks w, w+WAVES, ...).
//
// The contraction runs on v_mfma_f32_16x16x32_bf16.  One instruction takes 16
// weight rows (N side) and 32 columns of K, i.e. two 16-blocks that carry
// different binary16 scales.  The M side has 16 rows and the batch at most 8,
// so the two blocks are kept apart there: MFMA rows 0..7 see the activations
// of the first block and zeros for the second, rows 8..15 the opposite.  The
// result then holds the two per-block partial sums in different lanes (row
// groups 0,1 / 2,3), each is scaled in F32 by its own block scale, and the two
// halves are added once after the K loop.  A chunk of one tile is four such
// instructions (j = first / second half of the tile's rows, s = columns 0..31 /
// 32..63); a half has h/2 <= 16 rows, lanes n >= h/2 repeat the last row and
// are ignored.
//
// Lane (n = lane%16, g = lane/16) supplies to instruction (j, s) the 8 weights
// (4 bytes) of row j*h/2 + n, columns 32s+8g..+8, and needs the scale of block
// 2s + g/2 of that row.  TILED selects the provider's streaming layout (see
// qllm_fp4_prepack): the 64 sixteen-byte pieces a wave loads for one (tile,
// chunk) are contiguous (one 1 KiB burst) and hold the lane's four dwords in
// (j, s) order, scales likewise.  With the row-major layout lane (n, g) loads
// the 16 bytes of row 16(g/2)+n at byte chunk*32 + (g%2)*16 and a 4x4 dword
// transpose across the four lane rows regroups them (h is 32 there).
//
// Activations travel with the weights: together with the weight pieces of a
// chunk a wave prefetches the batch x 64 activation values of that chunk
// (8*batch sixteen-byte pieces, one per lane), drops them into a small
// wave-private LDS ring and reads the two A fragments back; lanes whose MFMA
// row belongs to the other block (or to no batch row) read a zero piece kept
// in the same ring slot.  Nothing is staged per workgroup, so there is no
// barrier in the K loop and any K that is a multiple of 64 is handled alike.
//
// Batches of up to 6 rows sit in MFMA rows {0,1,2,4,5,6} of each half: those
// are accumulator registers 0..2 of both row groups, one FMA fewer than rows
// 0..5 would cost.
//
// Q8: the activations are the reference's per-row Q8 (int8 codes and one F32
// scale per row, quantize_q8_batch_kernel, transformer_kernels.cu:912-946) and
// the result is its integer statement (fp4_gemv_q8_batch5_tensor_core_kernel,
// :1162-1275): out = 0.5 * s_m * sum over 32-blocks of 2^(e - 127) * (integer
// block sum).  The codes enter the same matrix instruction as exact bf16
// integers (|q| <= 127), the weights as exact bf16 (E2M1 value times a power of
// two): every product and every block sum is exact in F32, the blocks are
// accumulated in F32 as the reference accumulates them, the row scale is
// applied in the epilogue.  A chunk's codes are 4 * batch sixteen-byte pieces
// (16 columns each); a lane's fragment is eight consecutive bytes of a piece.
template <int SCHEME, int BATCH, int TILES, int WAVES, bool TILED, bool Q8 = false>
__global__ __launch_bounds__(WAVES * 64) void fp4_gemm_mfma_kernel(
    const GemmArgs args) {
  constexpr int PF = 4;                // chunks in flight per lane
  constexpr int PIECES = (Q8 ? 4 : 8) * BATCH;   // activation pieces per chunk
  constexpr bool COMPACT = BATCH <= 6;
  constexpr int REGS = COMPACT ? 3 : 4;  // accumulator registers in use
  constexpr int kZeroPiece = 64;
  constexpr bool F16 = SCHEME == kSchemeF16;
  // scale registers per (slot, tile): tiled = the lane's four scales;
  // row-major = the chunk's scales of rows n and 16+n
  constexpr int SCALE_WORDS = TILED ? (F16 ? 2 : 1) : (F16 ? 4 : 2);
  __shared__ __attribute__((aligned(16))) uint4 ring[WAVES][2][kZeroPiece + 1];
  __shared__ float reduce[WAVES][TILES][2][REGS][32];

  const uint32_t lane = threadIdx.x & 63u;
  // wave index as a scalar, so everything derived from it (chunk counts,
  // loop bounds, addresses) is uniform
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t n = lane & 15u;
  const uint32_t g = lane >> 4;
  const uint32_t K = args.padded_columns;
  const uint32_t row_bytes = K / 2u;
  const uint32_t scale_row_bytes = F16 ? K / 8u : K / 32u;
  constexpr uint32_t kScaleChunk = F16 ? 8u : 2u;   // scale bytes per row, chunk
  const uint32_t h = args.tile_rows;
  const uint32_t half_rows = h / 2u;
  const uint32_t tile_lane = n < half_rows ? n : half_rows - 1u;
  const bool balanced =
      args.balance_splits > 1u && blockIdx.x >= args.balance_first_tile;
  const uint32_t splits =
      balanced ? args.balance_splits : (args.k_splits > 1u ? args.k_splits : 1u);
  const uint32_t extra_index =
      balanced ? (blockIdx.x - args.balance_first_tile) / splits : 0u;
  const uint32_t tile_index =
      balanced ? args.balance_first_tile + extra_index : blockIdx.x / splits;
  const uint32_t split =
      balanced ? blockIdx.x - args.balance_first_tile - extra_index * splits
               : blockIdx.x - tile_index * splits;
  const uint32_t first_row = tile_index * h;

  // Weight and scale streams: wave-uniform start of the tile's stream plus a
  // 32-bit lane offset; consecutive chunks are weight_step / scale_step apart.
  const uint32_t weight_step = TILED ? 32u * h : 32u;
  const uint32_t scale_step = TILED ? h * kScaleChunk : kScaleChunk;
  const uint8_t* weight_base[TILES];
  const uint8_t* scale_base[TILES];
  uint32_t weight_lane, scale_lane[2];
  if (TILED) {
    weight_lane = (g * half_rows + tile_lane) * 16u;
    scale_lane[0] = F16 ? ((g >> 1) * half_rows + tile_lane) * 8u : tile_lane * 4u;
    scale_lane[1] = scale_lane[0];
  } else {
    const uint32_t last = args.rows - 1u - first_row;   // rows past the end repeat it
    weight_lane = min((g >> 1) * 16u + n, last) * row_bytes + (g & 1u) * 16u;
    scale_lane[0] = min(n, last) * scale_row_bytes;
    scale_lane[1] = min(16u + n, last) * scale_row_bytes;
  }
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    if (TILED) {
      const size_t first_chunk = static_cast<size_t>(tile_index) * (K / kChunk);
      weight_base[t] = args.tile[t].weights + first_chunk * weight_step;
      scale_base[t] = args.tile[t].scales + first_chunk * scale_step;
    } else {
      weight_base[t] =
          args.tile[t].weights + static_cast<size_t>(first_row) * row_bytes;
      scale_base[t] =
          args.tile[t].scales + static_cast<size_t>(first_row) * scale_row_bytes;
    }
  }
  // activation piece this lane fetches per chunk: piece p = octet*BATCH + m
  //   ->  act[m][chunk*64 + octet*8 .. +8]
  const uint32_t piece = lane < PIECES ? lane : PIECES - 1u;
  const uint32_t activation_lane =
      Q8 ? (piece % BATCH) * K + (piece / BATCH) * 16u
         : ((piece % BATCH) * K + (piece / BATCH) * 8u) * 2u;
  constexpr uint32_t kActivationChunkBytes = Q8 ? kChunk : kChunk * 2u;
  const uint8_t* activation_base =
      reinterpret_cast<const uint8_t*>(args.activations);
  // A fragment of span s: MFMA row n carries batch row m of block n/8; lane
  // (n, g) holds columns 8g..8g+7 of the span, i.e. octet 4s+g, which belongs
  // to block g/2.
  uint32_t fragment_piece[2];
  {
    const uint32_t r = n & 7u;
    const uint32_t m = COMPACT ? (r >> 2) * 3u + (r & 3u) : r;
    const bool live =
        m < BATCH && (!COMPACT || (r & 3u) < 3u) && (g >> 1) == (n >> 3);
    if (Q8) {
      // byte offsets into the ring slot: columns 32s + 8g .. + 8 of row m
      fragment_piece[0] = live ? ((g >> 1) * BATCH + m) * 16u + (g & 1u) * 8u
                               : kZeroPiece * 16u;
      fragment_piece[1] = live ? ((2u + (g >> 1)) * BATCH + m) * 16u + (g & 1u) * 8u
                               : kZeroPiece * 16u;
    } else {
      fragment_piece[0] = live ? g * BATCH + m : kZeroPiece;
      fragment_piece[1] = live ? (4u + g) * BATCH + m : kZeroPiece;
    }
  }
  if (lane < 2u) ring[wave][lane][kZeroPiece] = make_uint4(0u, 0u, 0u, 0u);

  // Output item of this thread (see the epilogue); its residual is fetched
  // now, so that the value is there when the K loop ends.
  constexpr uint32_t kItems = 2u * REGS * 32u;
  static_assert(kItems <= WAVES * 64u, "one output item per thread");
  const uint32_t item_lane = threadIdx.x & 31u;
  const uint32_t item_reg = (threadIdx.x >> 5) % REGS;
  const uint32_t item_half = (threadIdx.x >> 5) / REGS;         // j
  const uint32_t item_batch = (COMPACT ? 3u : 4u) * (item_lane >> 4) + item_reg;
  const uint32_t item_row = first_row + item_half * half_rows + (item_lane & 15u);
  const bool item_valid = threadIdx.x < kItems && item_batch < BATCH &&
                          (item_lane & 15u) < half_rows && item_row < args.rows;
  const size_t item_index = static_cast<size_t>(item_batch) * args.rows + item_row;
  float residual_value = 0.0f;
  if constexpr (TILES == 1) {
    if (args.residual && !args.segments && item_valid)
      residual_value = args.residual[item_index];
  }

  float acc[TILES][2][REGS];
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < REGS; ++i) acc[t][j][i] = 0.0f;

  // this workgroup's chunks: [first_chunk_of_split, + chunks)
  const uint32_t all_chunks = K / kChunk;
  const uint32_t first_chunk_of_split = split * all_chunks / splits;
  const uint32_t chunks = (split + 1u) * all_chunks / splits - first_chunk_of_split;
  const uint32_t my_chunks =
      chunks > wave ? (chunks - wave + WAVES - 1u) / WAVES : 0u;
  // Prefetch is unconditional, which keeps the load/wait pattern of the
  // unrolled ring static: an index past the wave's last chunk fetches the
  // first 16 bytes of the activations instead, in every lane (one line that
  // every workgroup keeps in L2; the value is ignored).  Fetching the last
  // chunk again would go back to HBM for it: streamed lines do not stay.
  const uint32_t last_index = my_chunks ? my_chunks - 1u : 0u;

  uint4 codes[PF][TILES];
  uint32_t scales[PF][TILES][SCALE_WORDS];
  uint4 activation[PF];
  auto issue = [&](int slot, uint32_t index) {
    const bool past = index > last_index;                                 // uniform
    const uint32_t chunk =
        first_chunk_of_split + wave + min(index, last_index) * WAVES;     // uniform
    const uint32_t weight_offset = past ? 0u : weight_lane;
    const uint32_t scale_offset[2] = {past ? 0u : scale_lane[0],
                                      past ? 0u : scale_lane[1]};
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      const uint8_t* weight_chunk =
          past ? activation_base
               : weight_base[t] + static_cast<size_t>(chunk) * weight_step;
      codes[slot][t] = load_stream16(weight_chunk + weight_offset);
      const uint8_t* scale_chunk =
          past ? activation_base
               : scale_base[t] + static_cast<size_t>(chunk) * scale_step;
      if constexpr (TILED && F16) {
        const uint2 v = load_stream8(scale_chunk + scale_offset[0]);
        scales[slot][t][0] = v.x;
        scales[slot][t][1] = v.y;
      } else if constexpr (TILED) {
        scales[slot][t][0] =
            *reinterpret_cast<const uint32_t*>(scale_chunk + scale_offset[0]);
      } else if constexpr (F16) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const uint2 v = load_stream8(scale_chunk + scale_offset[j]);
          scales[slot][t][2 * j] = v.x;
          scales[slot][t][2 * j + 1] = v.y;
        }
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j)
          scales[slot][t][j] =
              *reinterpret_cast<const uint16_t*>(scale_chunk + scale_offset[j]);
      }
    }
    activation[slot] = *reinterpret_cast<const uint4*>(
        activation_base + chunk * kActivationChunkBytes + activation_lane);
  };

  if (my_chunks) {
#pragma unroll
    for (int slot = 0; slot < PF; ++slot) issue(slot, static_cast<uint32_t>(slot));

    for (uint32_t base = 0; base < my_chunks; base += PF) {
#pragma unroll
      for (int slot = 0; slot < PF; ++slot) {
        const uint32_t index = base + slot;
        uint4 q[TILES];
        uint32_t s[TILES][SCALE_WORDS];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
          q[t] = codes[slot][t];
#pragma unroll
          for (int w = 0; w < SCALE_WORDS; ++w) s[t][w] = scales[slot][t][w];
        }
        const uint4 x = activation[slot];
        issue(slot, index + PF);
        if (index >= my_chunks) continue;

        // activation pieces -> wave-private ring -> A fragments
        uint4* stage = ring[wave][slot & 1];
        stage[lane] = x;
        __builtin_amdgcn_wave_barrier();
        bf16x8 a[2];
#pragma unroll
        for (int span = 0; span < 2; ++span) {
          if constexpr (Q8) {
            const uint2 bytes = *reinterpret_cast<const uint2*>(
                reinterpret_cast<const uint8_t*>(stage) + fragment_piece[span]);
            a[span] = q8x8_to_bf16(bytes);
          } else {
            a[span] = __builtin_bit_cast(bf16x8, stage[fragment_piece[span]]);
          }
        }
        __builtin_amdgcn_wave_barrier();

#pragma unroll
        for (int t = 0; t < TILES; ++t) {
          // packed[2j+s] = the lane's 8 weights for instruction (j, s);
          // scale / fold [2j+s] likewise
          uint32_t packed[4] = {q[t].x, q[t].y, q[t].z, q[t].w};
          if (!TILED) transpose_rows4(packed);
          float scale[4];
          float fold[4];
          if constexpr (F16) {
            // binary16 scale applied in F32 after the block's MFMA
            uint32_t pair[2];   // scales of (j, 0), (j, 1) as two halves
            if constexpr (TILED) {
              pair[0] = s[t][0];
              pair[1] = s[t][1];
            } else {
              // row j holds blocks 0..3 in two words; this lane wants blocks
              // g/2 and 2 + g/2
#pragma unroll
              for (int j = 0; j < 2; ++j)
                pair[j] = (g >> 1) ? (s[t][2 * j] >> 16) | (s[t][2 * j + 1] & 0xffff0000u)
                                   : (s[t][2 * j] & 0xffffu) | (s[t][2 * j + 1] << 16);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              scale[2 * j] = f16_bits_to_f32(pair[j] & 0xffffu);
              scale[2 * j + 1] = f16_bits_to_f32(pair[j] >> 16);
            }
            fold[0] = fold[1] = fold[2] = fold[3] = 1.0f;
          } else {
            // power-of-two scale folded into the nibble->bf16 conversion
            uint32_t bytes = s[t][0];
            if constexpr (!TILED) bytes |= s[t][1] << 16;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              fold[k] = ue8m0_to_f32((bytes >> (8 * k)) & 0xffu);
              scale[k] = 1.0f;
            }
          }
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            f32x4 d[2];
#pragma unroll
            for (int span = 0; span < 2; ++span) {
              const bf16x8 w = expand_fp4x8(packed[2 * j + span], fold[2 * j + span]);
              const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
              d[span] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[span], w, zero,
                                                                0, 0, 0);
            }
#pragma unroll
            for (int span = 0; span < 2; ++span)
#pragma unroll
              for (int i = 0; i < REGS; ++i)
                acc[t][j][i] = fmaf(d[span][i], scale[2 * j + span], acc[t][j][i]);
          }
        }
      }
    }
  }

  // The two blocks of a span sit in lanes 32 apart: add them, then reduce
  // across waves through LDS.  Lane (n, g < 2) register i now holds batch row
  // (COMPACT ? 3 : 4) * g + i of weight row j*h/2 + n.
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < REGS; ++i) {
        const float total = acc[t][j][i] + __shfl_xor(acc[t][j][i], 32, kWave);
        if (lane < 32u) reduce[wave][t][j][i][lane] = total;
      }
  __syncthreads();

  float total = 0.0f;
  float up = 0.0f;   // tile 1 is the up projection of the same rows
  if (threadIdx.x < kItems) {
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      total += reduce[w][0][item_half][item_reg][item_lane];
      if (TILES == 2) up += reduce[w][TILES - 1][item_half][item_reg][item_lane];
    }
  }
  if (balanced) {
    // hand the sums over; the last of the tile's workgroups finishes it
    float* const slot = args.balance_partials +
                        static_cast<size_t>(extra_index) * splits * TILES * 256u;
    if (threadIdx.x < kItems) {
      float* const mine = slot + static_cast<size_t>(split) * TILES * 256u;
      __hip_atomic_store(mine + threadIdx.x, total, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
      if (TILES == 2)
        __hip_atomic_store(mine + 256u + threadIdx.x, up, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    // the stores have reached memory before the counter moves
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    __shared__ uint32_t arrived;
    if (threadIdx.x == 0u) {
      arrived = __hip_atomic_fetch_add(args.balance_counters + extra_index, 1u,
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (arrived == splits - 1u)
        __hip_atomic_store(args.balance_counters + extra_index, 0u, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (arrived != splits - 1u) return;
    // every partial is requested before the first is used: one round trip
    float part[kMaxBalanceSplits][TILES];
    if (threadIdx.x < kItems) {
#pragma unroll
      for (uint32_t s = 0; s < kMaxBalanceSplits; ++s) {
        const float* theirs = slot + static_cast<size_t>(s) * TILES * 256u;
#pragma unroll
        for (int t = 0; t < TILES; ++t)
          part[s][t] = s < splits
                           ? __hip_atomic_load(theirs + t * 256u + threadIdx.x,
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                           : 0.0f;
      }
      total = 0.0f;
      up = 0.0f;
#pragma unroll
      for (uint32_t s = 0; s < kMaxBalanceSplits; ++s) {
        total += part[s][0];
        if (TILES == 2) up += part[s][TILES - 1];
      }
    }
  }
  if constexpr (Q8) {
    if (item_valid) {
      const float row_scale = args.activation_scales[item_batch];
      total *= row_scale;
      up *= row_scale;
    }
  }
  if constexpr (TILES == 1) {
    if (args.argmax_values != nullptr) {
      // the tile's best logit per batch row, on the values that are stored
      const float value = total + residual_value;
      __syncthreads();   // every wave has read its sums out of `reduce`
      float* const best_values = &reduce[0][0][0][0][0];
      uint32_t* const best_rows = reinterpret_cast<uint32_t*>(best_values) + kItems;
      if (threadIdx.x < kItems) {
        best_values[threadIdx.x] = item_valid ? value : -INFINITY;
        best_rows[threadIdx.x] = item_valid ? item_row : 0xffffffffu;
      }
      __syncthreads();
      if (threadIdx.x < BATCH) {
        const uint32_t m = threadIdx.x;
        const uint32_t group = m / (COMPACT ? 3u : 4u);
        const uint32_t reg = m % (COMPACT ? 3u : 4u);
        float best = -INFINITY;
        uint32_t best_row = 0xffffffffu;
        for (uint32_t half = 0; half < 2u; ++half)
          for (uint32_t k = 0; k < 16u; ++k) {
            const uint32_t slot = (half * REGS + reg) * 32u + group * 16u + k;
            const float candidate = best_values[slot];
            const uint32_t candidate_row = best_rows[slot];
            if (candidate > best || (candidate == best && candidate_row < best_row)) {
              best = candidate;
              best_row = candidate_row;
            }
          }
        args.argmax_values[m * gridDim.x + blockIdx.x] = best;
        args.argmax_indices[m * gridDim.x + blockIdx.x] = best_row;
      }
    }
  }
  if (!item_valid) return;
  if (TILES == 2) {
    if (args.output_kind == QLLM_OUT_F32) {
      // F32 activations (silu_product_kernel without bf16 rounding,
      // transformer_kernels.cu:2774-2783)
      static_cast<float*>(args.output)[item_index] =
          total / (1.0f + __expf(-total)) * up;
      return;
    }
    const float activated = bf16_round(total / (1.0f + __expf(-total)));
    static_cast<uint16_t*>(args.output)[item_index] =
        static_cast<uint16_t>(f32_to_bf16_bits(activated * up));
  } else if (args.segments) {
    uint32_t local = item_row;
    uint32_t segment = 0;
    while (segment + 1u < args.segments && local >= args.segment_rows[segment]) {
      local -= args.segment_rows[segment];
      ++segment;
    }
    store_output(args.segment_output[segment], args.segment_kind[segment],
                 static_cast<size_t>(item_batch) * args.segment_rows[segment] + local,
                 total);
  } else if (splits > 1u && !balanced) {
    static_cast<float*>(args.output)[static_cast<size_t>(split) * BATCH * args.rows +
                                     item_index] = total;
  } else {
    store_output(args.output, args.output_kind, item_index, total + residual_value);
  }
}

// ---- generic fallback: one wave per output row -------------------------------

template <int SCHEME, bool Q8>
__global__ __launch_bounds__(256) void fp4_gemv_generic_kernel(
    const uint8_t* __restrict__ weights, const uint8_t* __restrict__ scales,
    const void* __restrict__ activations, const float* __restrict__ act_scales,
    void* output, const float* residual, uint32_t rows,
    uint32_t padded_columns, uint32_t batch, uint32_t output_kind) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (row >= rows) return;
  const uint32_t K = padded_columns;
  const uint8_t* row_codes = weights + static_cast<size_t>(row) * (K / 2u);
  const uint8_t* row_scales =
      scales + static_cast<size_t>(row) *
                   (SCHEME == kSchemeF16 ? K / 8u : K / 32u);
  float totals[8];
#pragma unroll
  for (int m = 0; m < 8; ++m) totals[m] = 0.0f;

  for (uint32_t chunk = lane; chunk < K / 32u; chunk += 64u) {
    const uint4 packed4 =
        *reinterpret_cast<const uint4*>(row_codes + chunk * 16u);
    const uint32_t packed[4] = {packed4.x, packed4.y, packed4.z, packed4.w};
    float scale[2];
    if (SCHEME == kSchemeF16) {
      const uint32_t pair =
          *reinterpret_cast<const uint32_t*>(row_scales + chunk * 4u);
      scale[0] = f16_bits_to_f32(pair & 0xffffu);
      scale[1] = f16_bits_to_f32(pair >> 16);
    } else {
      scale[0] = scale[1] = ue8m0_to_f32(row_scales[chunk]);
    }
    // decode 32 weights (value * 2 as exact small floats)
    float w[32];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t code = (packed[d] >> (4 * j)) & 0xfu;
        const uint32_t index = code & 7u;
        const float magnitude = index <= 4u ? static_cast<float>(index)
                                : index == 5u ? 6.0f
                                : index == 6u ? 8.0f
                                              : 12.0f;
        w[d * 8 + j] = (code & 8u) ? -magnitude : magnitude;
      }
    }
    for (uint32_t m = 0; m < batch; ++m) {
      float partial[2] = {0.0f, 0.0f};
      if (Q8) {
        const int8_t* x =
            static_cast<const int8_t*>(activations) +
            static_cast<size_t>(m) * K + chunk * 32u;
        int32_t dot[2] = {0, 0};
#pragma unroll
        for (int j = 0; j < 32; ++j)
          dot[j / 16] += static_cast<int32_t>(w[j]) * static_cast<int32_t>(x[j]);
        partial[0] = static_cast<float>(dot[0]);
        partial[1] = static_cast<float>(dot[1]);
      } else {
        const uint16_t* x =
            static_cast<const uint16_t*>(activations) +
            static_cast<size_t>(m) * K + chunk * 32u;
#pragma unroll
        for (int j = 0; j < 32; ++j)
          partial[j / 16] = fmaf(w[j], bf16_bits_to_f32(x[j]), partial[j / 16]);
      }
      totals[m] = fmaf(partial[0], scale[0], totals[m]);
      totals[m] = fmaf(partial[1], scale[1], totals[m]);
    }
  }
  for (uint32_t m = 0; m < batch; ++m) {
    float total = wave_sum(totals[m]) * 0.5f;
    if (Q8) total *= act_scales[m];
    if (lane == 0u) {
      const size_t index = static_cast<size_t>(m) * rows + row;
      if (residual) total += residual[index];
      store_output(output, output_kind, index, total);
    }
  }
}

// Tile heights of the streaming layout: even, 8..32; 0 stands for 32.
bool tile_rows_ok(uint32_t tile_rows) {
  return tile_rows == 0u ||
         (tile_rows >= 8u && tile_rows <= 32u && tile_rows % 2u == 0u);
}

uint32_t matrix_tile_rows(const qllm_fp4_matrix* matrix) {
  return matrix->layout == QLLM_LAYOUT_TILED && matrix->tile_rows
             ? matrix->tile_rows
             : 32u;
}

bool matrix_ok(const qllm_fp4_matrix* m) {
  return m && m->weights && m->scales && m->rows && m->columns &&
         m->padded_columns >= m->columns && m->padded_columns % 32u == 0u &&
         (m->scale_scheme == QLLM_SCALE_UE8M0_BLOCK32 ||
          m->scale_scheme == QLLM_SCALE_F16_BLOCK16) &&
         (m->layout == QLLM_LAYOUT_ROW_MAJOR ||
          (m->layout == QLLM_LAYOUT_TILED && m->padded_columns % kChunk == 0u &&
           tile_rows_ok(m->tile_rows)));
}

template <int SCHEME, int BATCH, int TILES, bool TILED, bool Q8>
int32_t launch_mfma_waves(const GemmArgs& args, uint32_t grid, uint32_t waves,
                          hipStream_t stream) {
  if (waves == 4u)
    fp4_gemm_mfma_kernel<SCHEME, BATCH, TILES, 4, TILED, Q8>
        <<<grid, 256, 0, stream>>>(args);
  else
    fp4_gemm_mfma_kernel<SCHEME, BATCH, TILES, 8, TILED, Q8>
        <<<grid, 512, 0, stream>>>(args);
  return launched(Q8 ? "FP4 x Q8 MFMA GEMM" : "FP4 MFMA GEMM");
}

template <int SCHEME, int TILES, bool TILED, bool Q8 = false>
int32_t launch_mfma_batch(const GemmArgs& args, uint32_t batch, uint32_t grid,
                          uint32_t waves, hipStream_t stream) {
  switch (batch) {
    case 1: return launch_mfma_waves<SCHEME, 1, TILES, TILED, Q8>(args, grid, waves, stream);
    case 2: return launch_mfma_waves<SCHEME, 2, TILES, TILED, Q8>(args, grid, waves, stream);
    case 3: return launch_mfma_waves<SCHEME, 3, TILES, TILED, Q8>(args, grid, waves, stream);
    case 4: return launch_mfma_waves<SCHEME, 4, TILES, TILED, Q8>(args, grid, waves, stream);
    case 5: return launch_mfma_waves<SCHEME, 5, TILES, TILED, Q8>(args, grid, waves, stream);
    case 6: return launch_mfma_waves<SCHEME, 6, TILES, TILED, Q8>(args, grid, waves, stream);
    case 7: return launch_mfma_waves<SCHEME, 7, TILES, TILED, Q8>(args, grid, waves, stream);
    default: return launch_mfma_waves<SCHEME, 8, TILES, TILED, Q8>(args, grid, waves, stream);
  }
}

// One tile per workgroup (a gate tile and its up tile for the fused SwiGLU
// pair), or k_splits workgroups per tile; four waves split K, eight when the
// launch has too few workgroups to give every CU one.
uint32_t compute_units() {
  static const uint32_t count = [] {
    int device = 0, units = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount,
                              device) != hipSuccess ||
        units <= 0)
      return 256u;
    return static_cast<uint32_t>(units);
  }();
  return count;
}

int32_t launch_mfma(GemmArgs args, int scheme, bool tiled, uint32_t batch,
                    bool swiglu, hipStream_t stream, void* balance_workspace = nullptr) {
  const uint32_t splits = args.k_splits > 1u ? args.k_splits : 1u;
  uint32_t tiles =
      (args.rows + args.tile_rows - 1u) / args.tile_rows * splits;
  const size_t partial_capacity =
      (kBalanceWorkspaceBytes - kBalanceCounterBytes) / sizeof(float);
  if (balance_workspace && splits == 1u) {
    // the tiles past the last full round over the CUs, cut so that their
    // pieces make one more, equal, round
    const uint32_t units = compute_units();
    const uint32_t extra = tiles > units ? tiles % units : 0u;
    const uint32_t cut =
        extra ? std::min({units / extra, kMaxBalanceSplits,
                          args.padded_columns / kChunk})
              : 0u;
    if (cut >= 2u && extra <= kMaxBalanceTiles &&
        size_t{extra} * cut * balance_slot_floats(swiglu) <= partial_capacity) {
      args.balance_first_tile = tiles - extra;
      args.balance_splits = cut;
      args.balance_counters = static_cast<uint32_t*>(balance_workspace);
      args.balance_partials = reinterpret_cast<float*>(
          static_cast<uint8_t*>(balance_workspace) + kBalanceCounterBytes);
      tiles = args.balance_first_tile + extra * cut;
    }
  }
  // four waves split K, eight when the launch has too few workgroups to give
  // every CU one
  const uint32_t waves = tiles <= 256u && !swiglu ? 8u : 4u;
#define QLLM_LAUNCH(SCHEME_, TILES_, TILED_)                                  \
  return launch_mfma_batch<SCHEME_, TILES_, TILED_>(args, batch, tiles, waves, \
                                                    stream)
  if (args.activation_scales) {
    // Q8 activations: block-32 UE8M0 matrices in the streaming layout
    if (scheme != kSchemeUe8m0 || !tiled)
      return fail(QLLM_INVALID_ARGUMENT,
                  "the Q8 matrix-core GEMM takes tiled block-32 UE8M0 matrices");
    if (swiglu)
      return launch_mfma_batch<kSchemeUe8m0, 2, true, true>(args, batch, tiles,
                                                           waves, stream);
    return launch_mfma_batch<kSchemeUe8m0, 1, true, true>(args, batch, tiles, waves,
                                                         stream);
  }
  if (scheme == kSchemeF16) {
    if (tiled) {
      if (swiglu) QLLM_LAUNCH(kSchemeF16, 2, true);
      QLLM_LAUNCH(kSchemeF16, 1, true);
    }
    if (swiglu) QLLM_LAUNCH(kSchemeF16, 2, false);
    QLLM_LAUNCH(kSchemeF16, 1, false);
  }
  if (tiled) {
    if (swiglu) QLLM_LAUNCH(kSchemeUe8m0, 2, true);
    QLLM_LAUNCH(kSchemeUe8m0, 1, true);
  }
  if (swiglu) QLLM_LAUNCH(kSchemeUe8m0, 2, false);
  QLLM_LAUNCH(kSchemeUe8m0, 1, false);
#undef QLLM_LAUNCH
}

// Row-major -> streaming layout with tiles of h rows (even).  The block of
// (tile, chunk) holds 2h pieces of 16 bytes, piece g*h/2 + n = four dwords in
// (j, s) order, dword 2j+s = the 8 weights of row h*tile + j*h/2 + n, columns
// 64*chunk + 32s + 8g..+8: exactly what lane 16g + n feeds to the four
// instructions of the chunk, and one contiguous burst per wave-level load.
// Rows past the matrix are zero.  Scales follow per (tile, chunk): binary16 as
// h entries of 8 bytes, entry p*h/2 + n = the scales of blocks 2s + p of rows
// j*h/2 + n in (j, s) order; UE8M0 as h/2 entries of 4 bytes, entry n = the
// scales of 32-blocks s of rows j*h/2 + n in (j, s) order.
__global__ void fp4_prepack_kernel(const uint8_t* weights,
                                   const uint8_t* scales, uint8_t* out_weights,
                                   uint8_t* out_scales, uint32_t rows,
                                   uint32_t padded_columns, uint32_t f16_scales,
                                   uint32_t h) {
  const uint32_t chunks = padded_columns / kChunk;
  const uint32_t tiles = (rows + h - 1u) / h;
  const uint32_t half_rows = h / 2u;
  const size_t pieces = static_cast<size_t>(tiles) * chunks * 2u * h;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  const uint32_t scale_chunk_bytes = f16_scales ? 8u : 2u;
  const uint32_t scale_entries = f16_scales ? h : half_rows;
  for (size_t piece = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
       piece < pieces; piece += stride) {
    const uint32_t within = static_cast<uint32_t>(piece % (2u * h));
    const size_t block = piece / (2u * h);
    const uint32_t g = within / half_rows;
    const uint32_t n = within % half_rows;
    const uint32_t chunk = static_cast<uint32_t>(block % chunks);
    const uint32_t tile = static_cast<uint32_t>(block / chunks);
    uint32_t value[4];
    for (uint32_t j = 0; j < 2u; ++j)
      for (uint32_t s = 0; s < 2u; ++s) {
        const uint32_t row = tile * h + j * half_rows + n;
        value[2u * j + s] =
            row < rows ? *reinterpret_cast<const uint32_t*>(
                             weights + static_cast<size_t>(row) * (padded_columns / 2u) +
                             chunk * 32u + s * 16u + g * 4u)
                       : 0u;
      }
    *reinterpret_cast<uint4*>(out_weights + piece * 16u) =
        make_uint4(value[0], value[1], value[2], value[3]);
    // the first pieces of a (tile, chunk) also write its scale entries
    if (within >= scale_entries) continue;
    const uint32_t p = within / half_rows;   // block parity (binary16 only)
    for (uint32_t j = 0; j < 2u; ++j)
      for (uint32_t s = 0; s < 2u; ++s) {
        const uint32_t row = tile * h + j * half_rows + n;
        const uint8_t* source =
            scales + static_cast<size_t>(row) * (chunks * scale_chunk_bytes) +
            chunk * scale_chunk_bytes;
        if (f16_scales) {
          uint16_t* target = reinterpret_cast<uint16_t*>(
              out_scales + (block * h + within) * 8u);
          target[2u * j + s] =
              row < rows ? reinterpret_cast<const uint16_t*>(source)[2u * s + p] : 0u;
        } else {
          uint8_t* target = out_scales + (block * half_rows + within) * 4u;
          target[2u * j + s] = row < rows ? source[s] : 0u;
        }
      }
  }
}

// The inverse of fp4_prepack_kernel for rows [first_row, first_row + count):
// every piece of the tiles that overlap the range puts its four dwords back
// where the row-major layout has them.
__global__ void fp4_unpack_kernel(const uint8_t* tiled_weights,
                                  const uint8_t* tiled_scales,
                                  uint8_t* out_weights, uint8_t* out_scales,
                                  uint32_t first_row, uint32_t count,
                                  uint32_t padded_columns, uint32_t f16_scales,
                                  uint32_t h) {
  const uint32_t chunks = padded_columns / kChunk;
  const uint32_t half_rows = h / 2u;
  const uint32_t first_tile = first_row / h;
  const uint32_t last_tile = (first_row + count - 1u) / h;
  const size_t pieces =
      static_cast<size_t>(last_tile - first_tile + 1u) * chunks * 2u * h;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  const uint32_t scale_chunk_bytes = f16_scales ? 8u : 2u;
  const uint32_t scale_entries = f16_scales ? h : half_rows;
  for (size_t local = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
       local < pieces; local += stride) {
    const size_t piece =
        local + static_cast<size_t>(first_tile) * chunks * 2u * h;
    const uint32_t within = static_cast<uint32_t>(piece % (2u * h));
    const size_t block = piece / (2u * h);
    const uint32_t g = within / half_rows;
    const uint32_t n = within % half_rows;
    const uint32_t chunk = static_cast<uint32_t>(block % chunks);
    const uint32_t tile = static_cast<uint32_t>(block / chunks);
    const uint4 packed = *reinterpret_cast<const uint4*>(tiled_weights + piece * 16u);
    const uint32_t value[4] = {packed.x, packed.y, packed.z, packed.w};
    for (uint32_t j = 0; j < 2u; ++j)
      for (uint32_t s = 0; s < 2u; ++s) {
        const uint32_t row = tile * h + j * half_rows + n;
        if (row < first_row || row >= first_row + count) continue;
        *reinterpret_cast<uint32_t*>(
            out_weights +
            static_cast<size_t>(row - first_row) * (padded_columns / 2u) +
            chunk * 32u + s * 16u + g * 4u) = value[2u * j + s];
      }
    if (within >= scale_entries) continue;
    const uint32_t p = within / half_rows;
    for (uint32_t j = 0; j < 2u; ++j)
      for (uint32_t s = 0; s < 2u; ++s) {
        const uint32_t row = tile * h + j * half_rows + n;
        if (row < first_row || row >= first_row + count) continue;
        uint8_t* target =
            out_scales +
            static_cast<size_t>(row - first_row) * (chunks * scale_chunk_bytes) +
            chunk * scale_chunk_bytes;
        if (f16_scales)
          reinterpret_cast<uint16_t*>(target)[2u * s + p] =
              reinterpret_cast<const uint16_t*>(
                  tiled_scales + (block * h + within) * 8u)[2u * j + s];
        else
          target[s] = (tiled_scales + (block * half_rows + within) * 4u)[2u * j + s];
      }
  }
}

}  // namespace
}  // namespace qllm

using namespace qllm;

extern "C" int32_t qllm_fp4_unpack_rows(const qllm_fp4_matrix* matrix,
                                        uint32_t first_row, uint32_t row_count,
                                        void* weights, void* scales,
                                        void* stream) {
  if (!matrix_ok(matrix) || !row_count || first_row >= matrix->rows ||
      row_count > matrix->rows - first_row || !weights || !scales)
    return fail(QLLM_INVALID_ARGUMENT, "invalid FP4 row read-back");
  const bool f16 = matrix->scale_scheme == QLLM_SCALE_F16_BLOCK16;
  const size_t row_bytes = matrix->padded_columns / 2u;
  const size_t scale_row_bytes =
      f16 ? matrix->padded_columns / 8u : matrix->padded_columns / 32u;
  if (matrix->layout == QLLM_LAYOUT_ROW_MAJOR) {
    if (const int32_t status = checked(
            hipMemcpyAsync(weights, matrix->weights + first_row * row_bytes,
                           row_count * row_bytes, hipMemcpyDeviceToDevice,
                           as_stream(stream)),
            "copy FP4 rows"))
      return status;
    return checked(
        hipMemcpyAsync(scales,
                       static_cast<const uint8_t*>(matrix->scales) +
                           first_row * scale_row_bytes,
                       row_count * scale_row_bytes, hipMemcpyDeviceToDevice,
                       as_stream(stream)),
        "copy FP4 row scales");
  }
  if (matrix->padded_columns % kChunk != 0u)
    return fail(QLLM_INVALID_ARGUMENT, "tiled FP4 matrix needs K % 64 == 0");
  const uint32_t h = matrix_tile_rows(matrix);
  const size_t tiles = (first_row + row_count - 1u) / h - first_row / h + 1u;
  const size_t pieces = tiles * (matrix->padded_columns / kChunk) * 2u * h;
  const uint32_t grid =
      static_cast<uint32_t>(pieces / 256u < 16384u ? pieces / 256u + 1u : 16384u);
  fp4_unpack_kernel<<<grid, 256, 0, as_stream(stream)>>>(
      matrix->weights, static_cast<const uint8_t*>(matrix->scales),
      static_cast<uint8_t*>(weights), static_cast<uint8_t*>(scales), first_row,
      row_count, matrix->padded_columns, f16 ? 1u : 0u, h);
  return launched("FP4 row read-back");
}

extern "C" int32_t qllm_fp4_gemm_bf16(const qllm_fp4_matrix* matrix,
                                      const void* input, size_t input_bytes,
                                      void* output, uint32_t output_kind,
                                      const float* residual, uint32_t batch,
                                      void* stream) {
  if (!matrix_ok(matrix) || !input || !output || !batch || batch > 8u ||
      output_kind > QLLM_OUT_BF16 ||
      input_bytes <
          static_cast<size_t>(batch) * matrix->padded_columns * 2u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid FP4 BF16 GEMM");
  if (residual && output_kind == QLLM_OUT_BF16 &&
      static_cast<const void*>(residual) == output)
    return fail(QLLM_INVALID_ARGUMENT,
                "FP4 BF16 GEMM: bf16 output cannot alias the f32 residual");
  if (matrix->padded_columns % kChunk == 0u) {
    GemmArgs args{};
    args.tile[0] = {matrix->weights,
                    static_cast<const uint8_t*>(matrix->scales)};
    args.tile[1] = args.tile[0];
    args.activations = static_cast<const uint16_t*>(input);
    args.output = output;
    args.residual = residual;
    args.rows = matrix->rows;
    args.padded_columns = matrix->padded_columns;
    args.output_kind = output_kind;
    args.tile_rows = matrix_tile_rows(matrix);
    return launch_mfma(args, static_cast<int>(matrix->scale_scheme),
                       matrix->layout == QLLM_LAYOUT_TILED, batch, false,
                       as_stream(stream));
  }
  const uint32_t grid = (matrix->rows + 3u) / 4u;
  if (matrix->layout != QLLM_LAYOUT_ROW_MAJOR)
    return fail(QLLM_INVALID_ARGUMENT, "tiled FP4 matrix needs K % 64 == 0");
  if (matrix->scale_scheme == QLLM_SCALE_F16_BLOCK16)
    fp4_gemv_generic_kernel<kSchemeF16, false>
        <<<grid, 256, 0, as_stream(stream)>>>(
            matrix->weights, static_cast<const uint8_t*>(matrix->scales),
            input, nullptr, output, residual, matrix->rows,
            matrix->padded_columns, batch, output_kind);
  else
    fp4_gemv_generic_kernel<kSchemeUe8m0, false>
        <<<grid, 256, 0, as_stream(stream)>>>(
            matrix->weights, static_cast<const uint8_t*>(matrix->scales),
            input, nullptr, output, residual, matrix->rows,
            matrix->padded_columns, batch, output_kind);
  return launched("FP4 BF16 GEMV");
}

extern "C" size_t qllm_fp4_head_workspace_bytes(const qllm_fp4_matrix* matrix,
                                                uint32_t batch) {
  if (!matrix_ok(matrix) || !batch) return 0;
  const size_t tiles =
      (matrix->rows + matrix_tile_rows(matrix) - 1u) / matrix_tile_rows(matrix);
  return tiles * batch * (sizeof(float) + sizeof(uint32_t));
}

extern "C" int32_t qllm_fp4_head_argmax(const qllm_fp4_matrix* matrix,
                                        const void* input, size_t input_bytes,
                                        float* logits, uint32_t batch,
                                        uint32_t* tokens, void* workspace,
                                        size_t workspace_bytes,
                                        const qllm_rollout_step* advance,
                                        void* stream) {
  if (!matrix_ok(matrix) || !input || !logits || !batch || batch > 8u || !tokens ||
      !workspace || matrix->padded_columns % kChunk != 0u ||
      workspace_bytes < qllm_fp4_head_workspace_bytes(matrix, batch) ||
      input_bytes < static_cast<size_t>(batch) * matrix->padded_columns * 2u ||
      (advance && (batch != 1u || !advance->next_token || !advance->draft_tokens ||
                   !advance->rows || !advance->device_positions)))
    return fail(QLLM_INVALID_ARGUMENT, "invalid FP4 head with arg-max");
  GemmArgs args{};
  args.tile[0] = {matrix->weights, static_cast<const uint8_t*>(matrix->scales)};
  args.tile[1] = args.tile[0];
  args.activations = static_cast<const uint16_t*>(input);
  args.output = logits;
  args.rows = matrix->rows;
  args.padded_columns = matrix->padded_columns;
  args.output_kind = QLLM_OUT_F32;
  args.tile_rows = matrix_tile_rows(matrix);
  const uint32_t tiles = (matrix->rows + args.tile_rows - 1u) / args.tile_rows;
  args.argmax_values = static_cast<float*>(workspace);
  args.argmax_indices =
      reinterpret_cast<uint32_t*>(args.argmax_values + static_cast<size_t>(tiles) * batch);
  if (const int32_t status =
          launch_mfma(args, static_cast<int>(matrix->scale_scheme),
                      matrix->layout == QLLM_LAYOUT_TILED, batch, false,
                      as_stream(stream)))
    return status;
  RolloutAdvance step{};
  if (advance)
    step = {advance->next_token, advance->draft_tokens, advance->capacity,
            advance->rows, advance->device_positions};
  return launch_argmax_final(args.argmax_values, args.argmax_indices, tiles, batch,
                             tokens, advance ? &step : nullptr, as_stream(stream));
}

extern "C" int32_t qllm_fp4_gemm_bf16_partial(const qllm_fp4_matrix* matrix,
                                              const void* input,
                                              size_t input_bytes,
                                              float* partials,
                                              uint32_t k_splits, uint32_t batch,
                                              void* stream) {
  if (!matrix_ok(matrix) || matrix->layout != QLLM_LAYOUT_TILED || !input ||
      !partials || !batch || batch > 8u || !k_splits ||
      k_splits > matrix->padded_columns / kChunk || k_splits > 16u ||
      input_bytes < static_cast<size_t>(batch) * matrix->padded_columns * 2u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid FP4 BF16 partial GEMM");
  GemmArgs args{};
  args.tile[0] = {matrix->weights, static_cast<const uint8_t*>(matrix->scales)};
  args.tile[1] = args.tile[0];
  args.activations = static_cast<const uint16_t*>(input);
  args.output = partials;
  args.rows = matrix->rows;
  args.padded_columns = matrix->padded_columns;
  args.output_kind = QLLM_OUT_F32;
  args.tile_rows = matrix_tile_rows(matrix);
  args.k_splits = k_splits;
  return launch_mfma(args, static_cast<int>(matrix->scale_scheme), true, batch,
                     false, as_stream(stream));
}

namespace {

int32_t gemm_bf16_split(const qllm_fp4_matrix* matrix, const void* input,
                        size_t input_bytes, const qllm_gemm_segment* segments,
                        uint32_t segment_count, uint32_t batch,
                        void* balance_workspace, void* stream);
int32_t swiglu_bf16(const qllm_fp4_matrix* gate, const qllm_fp4_matrix* up,
                    const void* input, size_t input_bytes, void* output,
                    uint32_t batch, void* balance_workspace, void* stream);
}  // namespace

extern "C" size_t qllm_fp4_gemm_balance_workspace_bytes(void) {
  return kBalanceWorkspaceBytes;
}

extern "C" int32_t qllm_fp4_gemm_bf16_split(
    const qllm_fp4_matrix* matrix, const void* input, size_t input_bytes,
    const qllm_gemm_segment* segments, uint32_t segment_count, uint32_t batch,
    void* stream) {
  return gemm_bf16_split(matrix, input, input_bytes, segments, segment_count,
                         batch, nullptr, stream);
}

extern "C" int32_t qllm_fp4_gemm_bf16_split_balanced(
    const qllm_fp4_matrix* matrix, const void* input, size_t input_bytes,
    const qllm_gemm_segment* segments, uint32_t segment_count, uint32_t batch,
    void* workspace, size_t workspace_bytes, void* stream) {
  if (!balance_workspace_ok(workspace, workspace_bytes))
    return fail(QLLM_INVALID_ARGUMENT, "invalid balanced GEMM workspace");
  return gemm_bf16_split(matrix, input, input_bytes, segments, segment_count,
                         batch, workspace, stream);
}

extern "C" int32_t qllm_fp4_swiglu_bf16(const qllm_fp4_matrix* gate,
                                        const qllm_fp4_matrix* up,
                                        const void* input, size_t input_bytes,
                                        void* output, uint32_t batch,
                                        void* stream) {
  return swiglu_bf16(gate, up, input, input_bytes, output, batch, nullptr, stream);
}

extern "C" int32_t qllm_fp4_swiglu_bf16_balanced(
    const qllm_fp4_matrix* gate, const qllm_fp4_matrix* up, const void* input,
    size_t input_bytes, void* output, uint32_t batch, void* workspace,
    size_t workspace_bytes, void* stream) {
  if (!balance_workspace_ok(workspace, workspace_bytes))
    return fail(QLLM_INVALID_ARGUMENT, "invalid balanced GEMM workspace");
  return swiglu_bf16(gate, up, input, input_bytes, output, batch, workspace, stream);
}

namespace {
int32_t gemm_bf16_split(const qllm_fp4_matrix* matrix, const void* input,
                        size_t input_bytes, const qllm_gemm_segment* segments,
                        uint32_t segment_count, uint32_t batch,
                        void* balance_workspace, void* stream) {
  if (!matrix_ok(matrix) || !input || !segments || !segment_count ||
      segment_count > 3u || !batch || batch > 8u ||
      input_bytes < static_cast<size_t>(batch) * matrix->padded_columns * 2u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid split FP4 BF16 GEMM");
  if (matrix->padded_columns % kChunk != 0u) {
    // shapes the MFMA kernel does not take (row-major only): one plain call
    // per segment on that segment's rows
    const size_t row_bytes = matrix->padded_columns / 2u;
    const size_t scale_row_bytes =
        matrix->scale_scheme == QLLM_SCALE_F16_BLOCK16
            ? matrix->padded_columns / 8u
            : matrix->padded_columns / 32u;
    uint64_t first_row = 0;
    for (uint32_t s = 0; s < segment_count; ++s) {
      if (!segments[s].rows || first_row + segments[s].rows > matrix->rows)
        return fail(QLLM_INVALID_ARGUMENT, "invalid split FP4 BF16 GEMM segment");
      qllm_fp4_matrix part = *matrix;
      part.weights = matrix->weights + first_row * row_bytes;
      part.scales =
          static_cast<const uint8_t*>(matrix->scales) + first_row * scale_row_bytes;
      part.rows = segments[s].rows;
      const int32_t status =
          qllm_fp4_gemm_bf16(&part, input, input_bytes, segments[s].output,
                             segments[s].output_kind, nullptr, batch, stream);
      if (status != QLLM_OK) return status;
      first_row += segments[s].rows;
    }
    if (first_row != matrix->rows)
      return fail(QLLM_INVALID_ARGUMENT,
                  "split FP4 BF16 GEMM: segment rows do not add up to the matrix");
    return QLLM_OK;
  }
  GemmArgs args{};
  uint64_t total_rows = 0;
  for (uint32_t s = 0; s < segment_count; ++s) {
    if (!segments[s].output || !segments[s].rows ||
        segments[s].output_kind > QLLM_OUT_BF16)
      return fail(QLLM_INVALID_ARGUMENT, "invalid split FP4 BF16 GEMM segment");
    args.segment_rows[s] = segments[s].rows;
    args.segment_kind[s] = segments[s].output_kind;
    args.segment_output[s] = segments[s].output;
    total_rows += segments[s].rows;
  }
  if (total_rows != matrix->rows)
    return fail(QLLM_INVALID_ARGUMENT,
                "split FP4 BF16 GEMM: segment rows do not add up to the matrix");
  args.segments = segment_count;
  args.tile[0] = {matrix->weights, static_cast<const uint8_t*>(matrix->scales)};
  args.tile[1] = args.tile[0];
  args.activations = static_cast<const uint16_t*>(input);
  args.output = segments[0].output;
  args.rows = matrix->rows;
  args.padded_columns = matrix->padded_columns;
  args.output_kind = segments[0].output_kind;
  args.tile_rows = matrix_tile_rows(matrix);
  return launch_mfma(args, static_cast<int>(matrix->scale_scheme),
                     matrix->layout == QLLM_LAYOUT_TILED, batch, false,
                     as_stream(stream), balance_workspace);
}

int32_t swiglu_bf16(const qllm_fp4_matrix* gate, const qllm_fp4_matrix* up,
                    const void* input, size_t input_bytes, void* output,
                    uint32_t batch, void* balance_workspace, void* stream) {
  if (!matrix_ok(gate) || !matrix_ok(up) || gate->rows != up->rows ||
      gate->padded_columns != up->padded_columns ||
      gate->scale_scheme != up->scale_scheme || gate->layout != up->layout ||
      matrix_tile_rows(gate) != matrix_tile_rows(up) ||
      !input || !output || !batch ||
      batch > 8u || gate->padded_columns % kChunk != 0u ||
      input_bytes < static_cast<size_t>(batch) * gate->padded_columns * 2u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid fused FP4 SwiGLU GEMM");
  GemmArgs args{};
  args.tile[0] = {gate->weights, static_cast<const uint8_t*>(gate->scales)};
  args.tile[1] = {up->weights, static_cast<const uint8_t*>(up->scales)};
  args.activations = static_cast<const uint16_t*>(input);
  args.output = output;
  args.rows = gate->rows;
  args.padded_columns = gate->padded_columns;
  args.output_kind = QLLM_OUT_BF16;
  args.tile_rows = matrix_tile_rows(gate);
  return launch_mfma(args, static_cast<int>(gate->scale_scheme),
                     gate->layout == QLLM_LAYOUT_TILED, batch, true,
                     as_stream(stream), balance_workspace);
}
}  // namespace

namespace {
// the checks every Q8 matrix-core launch shares
bool q8_gemm_ok(const qllm_fp4_matrix* matrix, const int8_t* input,
                const float* input_scales, uint32_t batch) {
  return matrix_ok(matrix) && matrix->scale_scheme == QLLM_SCALE_UE8M0_BLOCK32 &&
         matrix->layout == QLLM_LAYOUT_TILED && input && input_scales && batch &&
         batch <= 8u && reinterpret_cast<uintptr_t>(input) % 16u == 0u;
}

GemmArgs q8_gemm_args(const qllm_fp4_matrix* matrix, const int8_t* input,
                      const float* input_scales) {
  GemmArgs args{};
  args.tile[0] = {matrix->weights, static_cast<const uint8_t*>(matrix->scales)};
  args.tile[1] = args.tile[0];
  args.activations = reinterpret_cast<const uint16_t*>(input);
  args.activation_scales = input_scales;
  args.rows = matrix->rows;
  args.padded_columns = matrix->padded_columns;
  args.tile_rows = matrix_tile_rows(matrix);
  return args;
}
}  // namespace

extern "C" int32_t qllm_fp4_gemm_q8(const qllm_fp4_matrix* matrix,
                                    const int8_t* input, const float* input_scales,
                                    void* output, uint32_t output_kind,
                                    const float* residual, uint32_t batch,
                                    void* stream) {
  if (!q8_gemm_ok(matrix, input, input_scales, batch) || !output ||
      output_kind > QLLM_OUT_BF16 ||
      (residual && output_kind == QLLM_OUT_BF16 &&
       static_cast<const void*>(residual) == output))
    return fail(QLLM_INVALID_ARGUMENT, "invalid FP4 x Q8 GEMM");
  GemmArgs args = q8_gemm_args(matrix, input, input_scales);
  args.output = output;
  args.output_kind = output_kind;
  args.residual = residual;
  return launch_mfma(args, kSchemeUe8m0, true, batch, false, as_stream(stream));
}

extern "C" int32_t qllm_fp4_gemm_q8_partial(const qllm_fp4_matrix* matrix,
                                            const int8_t* input,
                                            const float* input_scales,
                                            float* partials, uint32_t k_splits,
                                            uint32_t batch, void* stream) {
  if (!q8_gemm_ok(matrix, input, input_scales, batch) || !partials || !k_splits ||
      k_splits > matrix->padded_columns / kChunk || k_splits > 16u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid partial FP4 x Q8 GEMM");
  GemmArgs args = q8_gemm_args(matrix, input, input_scales);
  args.output = partials;
  args.output_kind = QLLM_OUT_F32;
  args.k_splits = k_splits;
  return launch_mfma(args, kSchemeUe8m0, true, batch, false, as_stream(stream));
}

extern "C" int32_t qllm_fp4_gemm_q8_split(const qllm_fp4_matrix* matrix,
                                          const int8_t* input,
                                          const float* input_scales,
                                          const qllm_gemm_segment* segments,
                                          uint32_t segment_count, uint32_t batch,
                                          void* workspace, size_t workspace_bytes,
                                          void* stream) {
  if (!q8_gemm_ok(matrix, input, input_scales, batch) || !segments ||
      !segment_count || segment_count > 3u ||
      (workspace && !balance_workspace_ok(workspace, workspace_bytes)))
    return fail(QLLM_INVALID_ARGUMENT, "invalid split FP4 x Q8 GEMM");
  GemmArgs args = q8_gemm_args(matrix, input, input_scales);
  uint64_t total_rows = 0;
  for (uint32_t s = 0; s < segment_count; ++s) {
    if (!segments[s].output || !segments[s].rows ||
        segments[s].output_kind > QLLM_OUT_BF16)
      return fail(QLLM_INVALID_ARGUMENT, "invalid split FP4 x Q8 GEMM segment");
    args.segment_rows[s] = segments[s].rows;
    args.segment_kind[s] = segments[s].output_kind;
    args.segment_output[s] = segments[s].output;
    total_rows += segments[s].rows;
  }
  if (total_rows != matrix->rows)
    return fail(QLLM_INVALID_ARGUMENT,
                "split FP4 x Q8 GEMM: segment rows do not add up to the matrix");
  args.segments = segment_count;
  args.output = segments[0].output;
  args.output_kind = segments[0].output_kind;
  return launch_mfma(args, kSchemeUe8m0, true, batch, false, as_stream(stream),
                     workspace);
}

extern "C" int32_t qllm_fp4_swiglu_q8(const qllm_fp4_matrix* gate,
                                      const qllm_fp4_matrix* up,
                                      const int8_t* input,
                                      const float* input_scales, float* output,
                                      uint32_t batch, void* workspace,
                                      size_t workspace_bytes, void* stream) {
  if ((workspace && !balance_workspace_ok(workspace, workspace_bytes)) ||
      !q8_gemm_ok(gate, input, input_scales, batch) || !matrix_ok(up) ||
      gate->rows != up->rows || gate->padded_columns != up->padded_columns ||
      up->scale_scheme != gate->scale_scheme || up->layout != gate->layout ||
      matrix_tile_rows(gate) != matrix_tile_rows(up) || !output)
    return fail(QLLM_INVALID_ARGUMENT, "invalid fused FP4 x Q8 SwiGLU GEMM");
  GemmArgs args = q8_gemm_args(gate, input, input_scales);
  args.tile[1] = {up->weights, static_cast<const uint8_t*>(up->scales)};
  args.output = output;
  args.output_kind = QLLM_OUT_F32;
  return launch_mfma(args, kSchemeUe8m0, true, batch, true, as_stream(stream),
                     workspace);
}

extern "C" int32_t qllm_fp4_gemv_q8_batch(const qllm_fp4_matrix* matrix,
                                          const int8_t* input,
                                          const float* input_scales,
                                          float* output, uint32_t batch,
                                          int32_t bf16_output, void* stream) {
  // the streaming layout goes to the matrix cores
  if (matrix_ok(matrix) && matrix->layout == QLLM_LAYOUT_TILED)
    return qllm_fp4_gemm_q8(matrix, input, input_scales, output,
                            bf16_output ? QLLM_OUT_F32_BF16_ROUNDED : QLLM_OUT_F32,
                            nullptr, batch, stream);
  if (!matrix_ok(matrix) || matrix->scale_scheme != QLLM_SCALE_UE8M0_BLOCK32 ||
      matrix->layout != QLLM_LAYOUT_ROW_MAJOR || !input || !input_scales ||
      !output || !batch || batch > 8u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid FP4 Q8 weight-reuse GEMV");
  const uint32_t grid = (matrix->rows + 3u) / 4u;
  fp4_gemv_generic_kernel<kSchemeUe8m0, true>
      <<<grid, 256, 0, as_stream(stream)>>>(
          matrix->weights, static_cast<const uint8_t*>(matrix->scales), input,
          input_scales, output, nullptr, matrix->rows, matrix->padded_columns,
          batch, bf16_output ? QLLM_OUT_F32_BF16_ROUNDED : QLLM_OUT_F32);
  return launched("FP4 Q8 weight-reuse GEMV");
}

extern "C" size_t qllm_fp4_packed_weight_bytes(uint32_t rows,
                                               uint32_t padded_columns,
                                               uint32_t tile_rows) {
  if (!rows || !tile_rows_ok(tile_rows)) return 0;
  const uint32_t h = tile_rows ? tile_rows : 32u;
  return static_cast<size_t>((rows + h - 1u) / h) * h * (padded_columns / 2u);
}

extern "C" size_t qllm_fp4_packed_scale_bytes(uint32_t rows,
                                              uint32_t padded_columns,
                                              uint32_t scale_scheme,
                                              uint32_t tile_rows) {
  if (!rows || !tile_rows_ok(tile_rows)) return 0;
  const uint32_t h = tile_rows ? tile_rows : 32u;
  const size_t padded_rows = static_cast<size_t>((rows + h - 1u) / h) * h;
  return scale_scheme == QLLM_SCALE_F16_BLOCK16
             ? padded_rows * (padded_columns / 16u) * 2u
             : padded_rows * (padded_columns / 32u);
}

extern "C" int32_t qllm_fp4_prepack(const qllm_fp4_matrix* source,
                                    uint32_t tile_rows, void* packed_weights,
                                    void* packed_scales,
                                    qllm_fp4_matrix* packed, void* stream) {
  if (!matrix_ok(source) || source->layout != QLLM_LAYOUT_ROW_MAJOR ||
      source->padded_columns % kChunk != 0u || !packed_weights ||
      !packed_scales || !packed || !tile_rows_ok(tile_rows))
    return fail(QLLM_INVALID_ARGUMENT, "invalid FP4 prepack");
  const uint32_t h = tile_rows ? tile_rows : 32u;
  const size_t pieces =
      qllm_fp4_packed_weight_bytes(source->rows, source->padded_columns, h) / 16u;
  const uint32_t grid =
      static_cast<uint32_t>(pieces / 256u < 16384u ? pieces / 256u + 1u : 16384u);
  fp4_prepack_kernel<<<grid, 256, 0, as_stream(stream)>>>(
      source->weights, static_cast<const uint8_t*>(source->scales),
      static_cast<uint8_t*>(packed_weights),
      static_cast<uint8_t*>(packed_scales), source->rows,
      source->padded_columns,
      source->scale_scheme == QLLM_SCALE_F16_BLOCK16 ? 1u : 0u, h);
  *packed = *source;
  packed->weights = static_cast<const uint8_t*>(packed_weights);
  packed->scales = packed_scales;
  packed->layout = QLLM_LAYOUT_TILED;
  packed->tile_rows = h;
  return launched("FP4 prepack");
}
