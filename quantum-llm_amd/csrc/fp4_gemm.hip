// FP4 (E2M1, block-scaled) weight GEMM for small batches (M <= 8 rows).
//
// Replaces fp4_gemv_q8_batch_weight_reuse / fp4_gemv_q8_batch5_tensor_core_kernel
// and fp4_gemm_bf16_block32 of the reference
// (runtime/src/cuda/transformer_kernels.cu:1025-1275, 1436-1541, 7400-7593).
//
// Two kernels:
//  * fp4_gemm_mfma_kernel  - the hot path.  At M=5 a verify step needs
//    16 flop per weight byte; at HBM speed that is ~130 TFLOP/s, above what
//    the vector ALUs deliver, so the contraction runs on the matrix cores
//    (v_mfma_f32_32x32x16_bf16) with the batch as the 32-wide M side (rows
//    >= batch are don't-care) and 32 weight rows as the N side.  Packed
//    nibbles stream from HBM with one 16-byte load per lane, are expanded in
//    registers by v_cvt_scalef32_pk_bf16_fp4 (exact), and activations are
//    staged once per workgroup in LDS in MFMA fragment order.
//  * fp4_gemv_generic_kernel - any shape/scheme/activation type, one wave per
//    output row; used for shapes the MFMA kernel does not take.
#include "common.hpp"

#include <cstdlib>

namespace qllm {
namespace {

constexpr int kSchemeUe8m0 = QLLM_SCALE_UE8M0_BLOCK32;
constexpr int kSchemeF16 = QLLM_SCALE_F16_BLOCK16;

constexpr uint32_t kChunk = 64;            // K elements per wave step

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
  const uint16_t* activations;  // bf16 [batch, padded_columns]
  void* output;
  const float* residual;
  uint32_t rows;
  uint32_t padded_columns;
  uint32_t output_kind;
  uint32_t swiglu;              // tile 1 is the up projection of tile 0
  uint32_t tile_rows;           // weight rows per tile, 8..32
  // Optional split of the output rows over up to three buffers (the q, k and
  // v projections stored as one matrix): segment s takes the next
  // segment_rows[s] rows.  segments == 0: everything goes to `output`.
  uint32_t segments;
  uint32_t segment_rows[3];
  uint32_t segment_kind[3];
  void* segment_output[3];
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

// Workgroup = WAVES waves.  The workgroup owns TILES tiles of h = tile_rows
// (at most 32) weight rows - lanes n >= h repeat row h-1 and are ignored;
// its waves interleave over 64-column chunks of K (wave w takes chunks
// w, w+WAVES, ...).  Lane (n = lane%32, g = lane/32) supplies, for each of the
// chunk's four 16-blocks b, the half g (8 weights = 4 bytes) of row n - the
// B-operand layout of the 32x32x16 MFMA.
//
// TILED selects the provider's streaming layout (see qllm_fp4_prepack): the
// 64 sixteen-byte pieces a wave loads for one (tile, chunk) are contiguous
// (one 1 KiB burst) and already hold the lane's four half-blocks.  With the
// row-major layout lane (n, g) loads the 16 bytes at row n, byte offset
// chunk*32 + g*16 (64 separate requests) and one v_permlane32_swap per dword
// pair regroups them.
//
// Activations travel with the weights: together with the weight pieces of a
// chunk a wave prefetches the batch x 64 activation values of that chunk
// (8*batch sixteen-byte pieces, one per lane), drops them into a small
// wave-private LDS ring in MFMA A-fragment order and reads the four 16-block
// fragments back.  Nothing is staged per workgroup, so there is no barrier in
// the K loop and any K that is a multiple of 64 is handled alike.
//
// Every block's MFMA starts from zero and its result is scaled in F32 by the
// block's binary16 scale, so only the accumulator registers that hold batch
// rows cost an FMA.  Batches of up to 6 rows sit in MFMA rows {0,1,2,4,5,6}:
// those are registers 0..2 of both lane halves, one FMA fewer than rows 0..5.
template <int SCHEME, int BATCH, int TILES, int WAVES, bool TILED>
__global__ __launch_bounds__(WAVES * 64) void fp4_gemm_mfma_kernel(
    const GemmArgs args) {
  // chunks in flight per lane; three with two tiles per group, which keeps
  // the kernel at three workgroups per CU so that the 544 groups of the fused
  // gate/up launch are all resident at once
  constexpr int PF = TILES == 2 ? 3 : 4;
  constexpr int PIECES = 8 * BATCH; // activation pieces per chunk
  constexpr bool COMPACT = BATCH <= 6;
  constexpr int REGS = COMPACT ? 3 : 4;  // accumulator registers in use
  // ring slot: PIECES pieces of 16 bytes, padded to 64 pieces
  __shared__ __attribute__((aligned(16))) uint4 ring[WAVES][2][64];
  __shared__ float reduce[WAVES][TILES][REGS][64];

  const uint32_t lane = threadIdx.x & 63u;
  // wave index as a scalar, so everything derived from it (chunk counts,
  // loop bounds, addresses) is uniform
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t n = lane & 31u;
  const uint32_t g = lane >> 5;
  const uint32_t K = args.padded_columns;
  const uint32_t row_bytes = K / 2u;
  const uint32_t scale_row_bytes =
      SCHEME == kSchemeF16 ? K / 8u : K / 32u;
  // batch row carried by MFMA row n on the A side (rows past the batch are
  // don't-care and repeat the last one)
  uint32_t batch_row = COMPACT ? (n >> 2) * 3u + (n & 3u) : n;
  if (batch_row >= BATCH) batch_row = BATCH - 1u;

  // Weight and scale streams: wave-uniform start of the tile's stream plus a
  // 32-bit lane offset; consecutive chunks are weight_step / scale_step apart.
  constexpr uint32_t kScaleChunk = SCHEME == kSchemeF16 ? 8u : 2u;
  const uint32_t h = args.tile_rows;
  const uint32_t tile_lane = n < h ? n : h - 1u;
  const uint32_t weight_step = TILED ? 32u * h : 32u;
  const uint32_t scale_step = TILED ? h * kScaleChunk : kScaleChunk;
  const uint8_t* weight_base[TILES];
  const uint8_t* scale_base[TILES];
  uint32_t weight_lane[TILES];
  uint32_t scale_lane[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    const uint32_t tile = args.swiglu ? blockIdx.x : blockIdx.x * TILES + t;
    const uint32_t tiles = (args.rows + h - 1u) / h;
    const uint32_t safe_tile = tile < tiles ? tile : tiles - 1u;
    if (TILED) {
      const size_t first_chunk = static_cast<size_t>(safe_tile) * (K / kChunk);
      weight_base[t] = args.tile[t].weights + first_chunk * weight_step;
      scale_base[t] = args.tile[t].scales + first_chunk * scale_step;
      weight_lane[t] = (g * h + tile_lane) * 16u;
      scale_lane[t] = tile_lane * kScaleChunk;
    } else {
      const uint32_t first_row = safe_tile * h;
      const uint32_t row = min(first_row + tile_lane, args.rows - 1u) - first_row;
      weight_base[t] =
          args.tile[t].weights + static_cast<size_t>(first_row) * row_bytes;
      scale_base[t] =
          args.tile[t].scales + static_cast<size_t>(first_row) * scale_row_bytes;
      weight_lane[t] = row * row_bytes + g * 16u;
      scale_lane[t] = row * scale_row_bytes;
    }
  }
  // activation piece this lane fetches per chunk: piece p = (block*2+half)*
  // BATCH + m  ->  act[m][chunk*64 + (block*2+half)*8 .. +8]
  const uint32_t piece = lane < PIECES ? lane : PIECES - 1u;
  const uint32_t activation_lane =
      ((piece % BATCH) * K + (piece / BATCH) * 8u) * 2u;
  const uint8_t* activation_base =
      reinterpret_cast<const uint8_t*>(args.activations);

  // The residual of this thread's output item (see the epilogue) is fetched
  // now, so that the value is there when the K loop ends.
  float residual_value = 0.0f;
  if constexpr (TILES == 1) {
    if (args.residual && !args.segments) {
      const uint32_t reg = (threadIdx.x / 64u) % REGS;
      const uint32_t batch = (COMPACT ? 3u : 4u) * (lane >> 5) + reg;
      const uint32_t row = blockIdx.x * h + n;
      if (threadIdx.x < REGS * 64u && batch < BATCH && n < h && row < args.rows)
        residual_value = args.residual[static_cast<size_t>(batch) * args.rows + row];
    }
  }

  float acc[TILES][REGS];
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int i = 0; i < REGS; ++i) acc[t][i] = 0.0f;

  const uint32_t chunks = K / kChunk;
  const uint32_t my_chunks =
      chunks > wave ? (chunks - wave + WAVES - 1u) / WAVES : 0u;
  // Prefetch is unconditional: indices past the wave's last chunk are clamped
  // to it (loaded again and ignored), which keeps the load/wait pattern of the
  // unrolled ring static.
  const uint32_t last_index = my_chunks ? my_chunks - 1u : 0u;

  uint4 codes[PF][TILES];
  uint2 scales[PF][TILES];
  uint4 activation[PF];
  auto issue = [&](int slot, uint32_t index) {
    const uint32_t chunk = wave + index * WAVES;   // uniform
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      codes[slot][t] = load_stream16(
          weight_base[t] + static_cast<size_t>(chunk) * weight_step +
          weight_lane[t]);
      const uint8_t* scale_address =
          scale_base[t] + static_cast<size_t>(chunk) * scale_step + scale_lane[t];
      if (SCHEME == kSchemeF16) {
        scales[slot][t] = load_stream8(scale_address);
      } else {
        const uint32_t pair = *reinterpret_cast<const uint16_t*>(scale_address);
        scales[slot][t] = make_uint2(pair & 0xffu, pair >> 8);
      }
    }
    activation[slot] = *reinterpret_cast<const uint4*>(
        activation_base + chunk * (kChunk * 2u) + activation_lane);
  };

  if (my_chunks) {
#pragma unroll
    for (int slot = 0; slot < PF; ++slot)
      issue(slot, min(static_cast<uint32_t>(slot), last_index));

    for (uint32_t base = 0; base < my_chunks; base += PF) {
#pragma unroll
      for (int slot = 0; slot < PF; ++slot) {
        const uint32_t index = base + slot;
        uint4 q[TILES];
        uint2 s[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
          q[t] = codes[slot][t];
          s[t] = scales[slot][t];
        }
        const uint4 x = activation[slot];
        issue(slot, min(index + PF, last_index));
        if (index >= my_chunks) continue;

        // activation pieces -> wave-private ring -> A fragments
        uint4* stage = ring[wave][slot & 1];
        stage[lane] = x;
        __builtin_amdgcn_wave_barrier();
        bf16x8 a[4];
#pragma unroll
        for (int b = 0; b < 4; ++b)
          a[b] = __builtin_bit_cast(bf16x8,
                                    stage[(b * 2u + g) * BATCH + batch_row]);
        __builtin_amdgcn_wave_barrier();

#pragma unroll
        for (int t = 0; t < TILES; ++t) {
          uint32_t packed[4];  // half g of blocks 0..3 of row n
          if (TILED) {
            packed[0] = q[t].x; packed[1] = q[t].y;
            packed[2] = q[t].z; packed[3] = q[t].w;
          } else {
            const auto s01 = __builtin_amdgcn_permlane32_swap(q[t].x, q[t].y,
                                                              false, false);
            const auto s23 = __builtin_amdgcn_permlane32_swap(q[t].z, q[t].w,
                                                              false, false);
            packed[0] = s01[0]; packed[1] = s23[0];
            packed[2] = s01[1]; packed[3] = s23[1];
          }
          float scale[4];
          float fold[4];
          if (SCHEME == kSchemeF16) {
            // binary16 scale applied in F32 after the block's MFMA
            scale[0] = f16_bits_to_f32(s[t].x & 0xffffu);
            scale[1] = f16_bits_to_f32(s[t].x >> 16);
            scale[2] = f16_bits_to_f32(s[t].y & 0xffffu);
            scale[3] = f16_bits_to_f32(s[t].y >> 16);
            fold[0] = fold[1] = fold[2] = fold[3] = 1.0f;
          } else {
            // power-of-two scale folded into the nibble->bf16 conversion
            fold[0] = fold[1] = ue8m0_to_f32(s[t].x);
            fold[2] = fold[3] = ue8m0_to_f32(s[t].y);
            scale[0] = scale[1] = scale[2] = scale[3] = 1.0f;
          }
          f32x16 d[4];
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            const bf16x8 w = expand_fp4x8(packed[b], fold[b]);
            f32x16 zero;
#pragma unroll
            for (int i = 0; i < 16; ++i) zero[i] = 0.0f;
            d[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[b], w, zero, 0, 0, 0);
          }
#pragma unroll
          for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int i = 0; i < REGS; ++i)
              acc[t][i] = fmaf(d[b][i], scale[b], acc[t][i]);
        }
      }
    }
  }

  // Cross-wave reduction through LDS.
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int i = 0; i < REGS; ++i) reduce[wave][t][i][lane] = acc[t][i];
  __syncthreads();

  // Output item of this thread: item = (tile, register i, lane); lane (n, g)
  // register i holds MFMA row 4*g + i, i.e. batch row (COMPACT ? 3 : 4)*g + i.
  // (two tiles per workgroup are the gate/up pair: one output per row pair)
  static_assert(TILES <= 2 && REGS * 64 <= WAVES * 64,
                "one output item per thread");
  const uint32_t items = (args.swiglu ? 1u : TILES) * REGS * 64u;
  const uint32_t item_tile = threadIdx.x / (REGS * 64u);
  const uint32_t item_reg = (threadIdx.x / 64u) % REGS;
  const uint32_t item_lane = threadIdx.x & 63u;
  const uint32_t item_batch = (COMPACT ? 3u : 4u) * (item_lane >> 5) + item_reg;
  const uint32_t item_tile_row = item_lane & 31u;
  const uint32_t item_row =
      (args.swiglu ? blockIdx.x : blockIdx.x * TILES + item_tile) * h + item_tile_row;
  const bool item_valid = threadIdx.x < items && item_batch < BATCH &&
                          item_tile_row < h && item_row < args.rows;
  const size_t item_index = static_cast<size_t>(item_batch) * args.rows + item_row;
  if (!item_valid) return;
  float total = 0.0f;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) total += reduce[w][item_tile][item_reg][item_lane];
  if (args.swiglu) {
    float up = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w)
      up += reduce[w][TILES - 1][item_reg][item_lane];
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

bool matrix_ok(const qllm_fp4_matrix* m) {
  return m && m->weights && m->scales && m->rows && m->columns &&
         m->padded_columns >= m->columns && m->padded_columns % 32u == 0u &&
         (m->scale_scheme == QLLM_SCALE_UE8M0_BLOCK32 ||
          m->scale_scheme == QLLM_SCALE_F16_BLOCK16) &&
         (m->layout == QLLM_LAYOUT_ROW_MAJOR ||
          (m->layout == QLLM_LAYOUT_TILED && m->padded_columns % kChunk == 0u &&
           (m->tile_rows == 0u || (m->tile_rows >= 8u && m->tile_rows <= 32u))));
}

template <int SCHEME, int BATCH, int TILES, bool TILED>
int32_t launch_mfma_waves(const GemmArgs& args, uint32_t grid, uint32_t waves,
                          hipStream_t stream) {
  if (waves == 4u)
    fp4_gemm_mfma_kernel<SCHEME, BATCH, TILES, 4, TILED>
        <<<grid, 256, 0, stream>>>(args);
  else
    fp4_gemm_mfma_kernel<SCHEME, BATCH, TILES, 8, TILED>
        <<<grid, 512, 0, stream>>>(args);
  return launched("FP4 MFMA GEMM");
}

template <int SCHEME, int TILES, bool TILED>
int32_t launch_mfma_batch(const GemmArgs& args, uint32_t batch, uint32_t grid,
                          uint32_t waves, hipStream_t stream) {
  switch (batch) {
    case 1: return launch_mfma_waves<SCHEME, 1, TILES, TILED>(args, grid, waves, stream);
    case 2: return launch_mfma_waves<SCHEME, 2, TILES, TILED>(args, grid, waves, stream);
    case 3: return launch_mfma_waves<SCHEME, 3, TILES, TILED>(args, grid, waves, stream);
    case 4: return launch_mfma_waves<SCHEME, 4, TILES, TILED>(args, grid, waves, stream);
    case 5: return launch_mfma_waves<SCHEME, 5, TILES, TILED>(args, grid, waves, stream);
    case 6: return launch_mfma_waves<SCHEME, 6, TILES, TILED>(args, grid, waves, stream);
    case 7: return launch_mfma_waves<SCHEME, 7, TILES, TILED>(args, grid, waves, stream);
    default: return launch_mfma_waves<SCHEME, 8, TILES, TILED>(args, grid, waves, stream);
  }
}

// One tile per workgroup (a gate tile and its up tile for the fused SwiGLU
// pair); four waves split K, eight when the matrix has few tiles.
int32_t launch_mfma(GemmArgs args, int scheme, bool tiled, uint32_t batch,
                    bool swiglu, hipStream_t stream) {
  const uint32_t tiles = (args.rows + args.tile_rows - 1u) / args.tile_rows;
  const uint32_t waves = tiles <= 384u && !swiglu ? 8u : 4u;
  args.swiglu = swiglu ? 1u : 0u;
#define QLLM_LAUNCH(SCHEME_, TILES_, TILED_)                                  \
  return launch_mfma_batch<SCHEME_, TILES_, TILED_>(args, batch, tiles, waves, \
                                                    stream)
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

uint32_t matrix_tile_rows(const qllm_fp4_matrix* matrix) {
  if (matrix->layout == QLLM_LAYOUT_TILED)
    return matrix->tile_rows ? matrix->tile_rows : 32u;
  return 32u;  // row-major: any height works; full MFMA tiles are cheapest
}

// Row-major -> streaming layout with tiles of h rows.  The block of (tile,
// chunk) holds 2*h pieces of 16 bytes, piece half*h + n = the four 4-byte
// half-blocks of row h*tile + n at byte offsets chunk*32 + b*8 + half*4
// (b = 0..3): exactly what lane (n, half) feeds to the four block MFMAs, and
// one contiguous burst per wave-level load.  Rows past the matrix are zero.
// Scales follow per (tile, chunk) as h consecutive row entries of 4 binary16 /
// 2 UE8M0.
__global__ void fp4_prepack_kernel(const uint8_t* weights,
                                   const uint8_t* scales, uint8_t* out_weights,
                                   uint8_t* out_scales, uint32_t rows,
                                   uint32_t padded_columns,
                                   uint32_t scale_chunk_bytes, uint32_t h) {
  const uint32_t chunks = padded_columns / kChunk;
  const uint32_t tiles = (rows + h - 1u) / h;
  const size_t pieces = static_cast<size_t>(tiles) * chunks * 2u * h;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t piece = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
       piece < pieces; piece += stride) {
    const uint32_t within = static_cast<uint32_t>(piece % (2u * h));
    const size_t block = piece / (2u * h);
    const uint32_t half = within / h;
    const uint32_t n = within % h;
    const uint32_t chunk = static_cast<uint32_t>(block % chunks);
    const uint32_t tile = static_cast<uint32_t>(block / chunks);
    const uint32_t row = tile * h + n;
    uint4 value = make_uint4(0u, 0u, 0u, 0u);
    if (row < rows) {
      const uint32_t* source = reinterpret_cast<const uint32_t*>(
          weights + static_cast<size_t>(row) * (padded_columns / 2u) +
          chunk * 32u + half * 4u);
      value = make_uint4(source[0], source[2], source[4], source[6]);
    }
    *reinterpret_cast<uint4*>(out_weights + piece * 16u) = value;
    if (half == 0u) {
      uint8_t* target = out_scales + (block * h + n) * scale_chunk_bytes;
      const uint8_t* source =
          scales + static_cast<size_t>(row) * (chunks * scale_chunk_bytes) +
          chunk * scale_chunk_bytes;
      for (uint32_t byte = 0; byte < scale_chunk_bytes; ++byte)
        target[byte] = row < rows ? source[byte] : 0u;
    }
  }
}

}  // namespace
}  // namespace qllm

using namespace qllm;

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

extern "C" int32_t qllm_fp4_gemm_bf16_split(
    const qllm_fp4_matrix* matrix, const void* input, size_t input_bytes,
    const qllm_gemm_segment* segments, uint32_t segment_count, uint32_t batch,
    void* stream) {
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
                     as_stream(stream));
}

extern "C" int32_t qllm_fp4_swiglu_bf16(const qllm_fp4_matrix* gate,
                                        const qllm_fp4_matrix* up,
                                        const void* input, size_t input_bytes,
                                        void* output, uint32_t batch,
                                        void* stream) {
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
                     as_stream(stream));
}

extern "C" int32_t qllm_fp4_gemv_q8_batch(const qllm_fp4_matrix* matrix,
                                          const int8_t* input,
                                          const float* input_scales,
                                          float* output, uint32_t batch,
                                          int32_t bf16_output, void* stream) {
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

// A tile costs the same matrix-core and conversion time whatever its height,
// so full 32-row tiles are the default; shorter ones only pay off when a
// matrix has too few rows to give every CU a tile.
static uint32_t resolve_tile_rows(uint32_t, uint32_t tile_rows) {
  return tile_rows ? tile_rows : 32u;
}

extern "C" size_t qllm_fp4_packed_weight_bytes(uint32_t rows,
                                               uint32_t padded_columns,
                                               uint32_t tile_rows) {
  if (!rows || tile_rows > 32u || (tile_rows && tile_rows < 8u)) return 0;
  const uint32_t h = resolve_tile_rows(rows, tile_rows);
  return static_cast<size_t>((rows + h - 1u) / h) * h * (padded_columns / 2u);
}

extern "C" size_t qllm_fp4_packed_scale_bytes(uint32_t rows,
                                              uint32_t padded_columns,
                                              uint32_t scale_scheme,
                                              uint32_t tile_rows) {
  if (!rows || tile_rows > 32u || (tile_rows && tile_rows < 8u)) return 0;
  const uint32_t h = resolve_tile_rows(rows, tile_rows);
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
      !packed_scales || !packed || tile_rows > 32u ||
      (tile_rows && tile_rows < 8u))
    return fail(QLLM_INVALID_ARGUMENT, "invalid FP4 prepack");
  const uint32_t h = resolve_tile_rows(source->rows, tile_rows);
  const uint32_t scale_chunk =
      source->scale_scheme == QLLM_SCALE_F16_BLOCK16 ? 8u : 2u;
  const size_t pieces =
      qllm_fp4_packed_weight_bytes(source->rows, source->padded_columns, h) / 16u;
  const uint32_t grid =
      static_cast<uint32_t>(pieces / 256u < 16384u ? pieces / 256u + 1u : 16384u);
  fp4_prepack_kernel<<<grid, 256, 0, as_stream(stream)>>>(
      source->weights, static_cast<const uint8_t*>(source->scales),
      static_cast<uint8_t*>(packed_weights),
      static_cast<uint8_t*>(packed_scales), source->rows,
      source->padded_columns, scale_chunk, h);
  *packed = *source;
  packed->weights = static_cast<const uint8_t*>(packed_weights);
  packed->scales = packed_scales;
  packed->layout = QLLM_LAYOUT_TILED;
  packed->tile_rows = h;
  return launched("FP4 prepack");
}
