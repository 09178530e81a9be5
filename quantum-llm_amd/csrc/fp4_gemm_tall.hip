// FP4 (E2M1, block-scaled) weight GEMM for tall batches (prompt prefill,
// M >> 8 rows).
//
// Replaces fp4_gemm_block32_kernel of the reference
// (runtime/src/cuda/transformer_kernels.cu:1284-1430: weights expanded to
// bf16 with their block scale, bf16 activations, 16x16x16 tensor-core tiles,
// F32 accumulation).  Here the contraction is compute-bound, so it is laid out
// for the matrix cores: a workgroup of four waves owns 128 activation rows x
// 256 weight rows; every wave keeps the 128 x 64 accumulator of its two
// 32-row weight tiles in registers (8 x 4 tiles of v_mfma_f32_16x16x32), takes
// its weights straight from the provider's streaming layout - the 16-byte
// piece a lane loads per (tile, chunk) is its B operand for the chunk's four
// instructions, no LDS and no shuffle - and shares the activation tile of the
// chunk through LDS (double-buffered, one barrier per 64 columns of K).
//
// Scale schemes:
//  * UE8M0 per 32: the power-of-two scale is folded into the nibble -> bf16
//    conversion, which stays exact; bf16 matrix instructions.
//  * binary16 per 16: weight x scale has up to 13 significant bits (a 3-bit
//    weight times an 11-bit scale).  It is split into two binary16 values,
//    hi = the product rounded to binary16 and lo = its rounding error, which
//    a fused multiply-add returns exactly; they go through the matrix cores
//    one after the other into the same F32 accumulator; the bf16 activations
//    are converted to binary16 (exact between 6.1e-5 and 65504 in magnitude -
//    the range of a decoder's normalised activations; beyond it they saturate
//    or lose low bits).  The products are the exact ones, as in the small-batch
//    kernel, at twice the matrix instructions - for block scales between 2^-13
//    (1.22e-4) and 10917 in magnitude: both halves are formed in binary16, so
//    a weight of 6 under a larger scale overflows it (the small-batch kernel
//    multiplies in F32 and stays finite), and under a smaller scale the low
//    half has bits below 2^-24 and is cut short (a relative error of up to
//    2^-11 in that weight).  Checkpoint scales lie well inside.
#include "common.hpp"

#include <type_traits>

namespace qllm {
namespace {

constexpr int kSchemeUe8m0 = QLLM_SCALE_UE8M0_BLOCK32;
constexpr int kSchemeF16 = QLLM_SCALE_F16_BLOCK16;

constexpr uint32_t kChunk = 64;          // K columns per step
constexpr uint32_t kRowsM = 128;         // activation rows per workgroup
constexpr uint32_t kTilesM = kRowsM / 16;
constexpr uint32_t kWaves = 4;
constexpr uint32_t kTilesPerWave = 2;    // 32-row weight tiles per wave
constexpr uint32_t kTilesN = kWaves * kTilesPerWave;   // per workgroup
constexpr uint32_t kTileRows = 32;
constexpr uint32_t kBand = 8;            // activation tiles per band of the grid
// LDS row of the activation tile: 64 values of 16 bits plus 16 bytes, so that
// the sixteen rows a fragment load touches fall on different banks
constexpr uint32_t kLdsRow = kChunk * 2u + 16u;

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

struct TallArgs {
  const uint8_t* weights;        // streaming layout, 32-row tiles
  const uint8_t* scales;
  // SWIGLU form: `weights` / `scales` are the gate matrix, these the up matrix
  // of the same shape; output = bf16(bf16(silu(gate . x)) * (up . x))
  const uint8_t* up_weights;
  const uint8_t* up_scales;
  const uint16_t* activations;   // bf16 [batch, padded_columns]
  uint32_t rows;                 // weight rows = output columns
  uint32_t padded_columns;
  uint32_t batch;
  uint32_t m_tiles;
  uint32_t n_tiles;
  void* output;                  // [batch, rows]
  uint32_t output_kind;
  const float* residual;
  // optional split of the output columns over up to three buffers
  uint32_t segments;
  uint32_t segment_rows[3];
  uint32_t segment_kind[3];
  void* segment_output[3];
};

__device__ __forceinline__ void store_value(void* output, uint32_t kind,
                                            size_t index, float value) {
  if (kind == QLLM_OUT_BF16)
    static_cast<uint16_t*>(output)[index] =
        static_cast<uint16_t>(f32_to_bf16_bits(value));
  else if (kind == QLLM_OUT_F32_BF16_ROUNDED)
    static_cast<float*>(output)[index] = bf16_round(value);
  else
    static_cast<float*>(output)[index] = value;
}

// Two bf16 values (one dword) -> two binary16 values.  Round toward zero only
// matters outside binary16's normal range, where it saturates instead of
// producing infinities.
__device__ __forceinline__ uint32_t bf16x2_to_f16x2(uint32_t pair) {
  const float low = __uint_as_float(pair << 16);
  const float high = __uint_as_float(pair & 0xffff0000u);
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(low, high));
}

template <int SCHEME>
struct Operand;

template <>
struct Operand<kSchemeUe8m0> {
  using Vector = bf16x8;
  static constexpr int kParts = 1;
  // `scale` = the block's power of two
  static __device__ __forceinline__ void weights(uint32_t packed, float scale,
                                                 uint32_t, Vector (&out)[1]) {
    const bf16x2 p0 = fp4x2_to_bf16<0>(packed, scale);
    const bf16x2 p1 = fp4x2_to_bf16<1>(packed, scale);
    const bf16x2 p2 = fp4x2_to_bf16<2>(packed, scale);
    const bf16x2 p3 = fp4x2_to_bf16<3>(packed, scale);
    Vector w;
    w[0] = p0[0]; w[1] = p0[1]; w[2] = p1[0]; w[3] = p1[1];
    w[4] = p2[0]; w[5] = p2[1]; w[6] = p3[0]; w[7] = p3[1];
    out[0] = w;
  }
  static __device__ __forceinline__ f32x4 mfma(Vector a, Vector b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t stage(uint32_t pair) { return pair; }
};

typedef __attribute__((ext_vector_type(2))) float f32x2;

template <>
struct Operand<kSchemeF16> {
  using Vector = f16x8;
  static constexpr int kParts = 2;
  // `scale_bits` = the block's binary16 scale; out[0] = hi, out[1] = lo with
  // hi + lo = weight x scale exactly
  // hi = the product rounded to binary16, lo = the rounding error, which a
  // fused multiply-add returns exactly (it has at most two significant bits):
  // three packed instructions per pair of weights.
  static __device__ __forceinline__ void weights(uint32_t packed, float,
                                                 uint32_t scale_bits,
                                                 Vector (&out)[2]) {
    const f16x2 scale =
        __builtin_bit_cast(f16x2, scale_bits | (scale_bits << 16));
    Vector hi, lo;
#pragma unroll
    for (int pair = 0; pair < 4; ++pair) {
      f16x2 w;
      switch (pair) {
        case 0: w = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(packed, 1.0f, 0); break;
        case 1: w = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(packed, 1.0f, 1); break;
        case 2: w = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(packed, 1.0f, 2); break;
        default: w = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(packed, 1.0f, 3); break;
      }
      const f16x2 top = w * scale;
      const f16x2 rest = __builtin_elementwise_fma(w, scale, -top);
      hi[2 * pair] = top[0]; hi[2 * pair + 1] = top[1];
      lo[2 * pair] = rest[0]; lo[2 * pair + 1] = rest[1];
    }
    out[0] = hi;
    out[1] = lo;
  }
  static __device__ __forceinline__ f32x4 mfma(Vector a, Vector b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t stage(uint32_t pair) {
    return bf16x2_to_f16x2(pair);
  }
};

// Workgroup (m_tile, n_tile): activation rows [128 m_tile, +128), weight rows
// [256 n_tile, +256).
//
// SWIGLU: a wave's two tiles are the same 32 rows of the gate and of the up
// matrix (a workgroup covers 128 rows of each), and the epilogue writes
// silu(gate) * up in bf16 with the rounding points of the separate
// SiLU-product launch - no F32 round trip of the two projections.
template <int SCHEME, bool SWIGLU = false>
__global__ __launch_bounds__(kWaves * 64, 2) void fp4_gemm_tall_kernel(
    const TallArgs args) {
  using Op = Operand<SCHEME>;
  using Vector = typename Op::Vector;
  constexpr bool F16 = SCHEME == kSchemeF16;
  __shared__ __attribute__((aligned(16))) uint8_t tile[2][kRowsM * kLdsRow];

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t n = lane & 15u;
  const uint32_t g = lane >> 4;
  const uint32_t K = args.padded_columns;
  const uint32_t chunks = K / kChunk;

  // Workgroups are dealt to the eight XCDs in turn, so XCD x runs the ids
  // x, x + 8, ...: give it a contiguous range of tiles instead.  Within the
  // range the tiles go band by band (kBand activation tiles high), column by
  // column: the 64 workgroups an XCD runs at a time then cover about 8 x 8
  // tiles and fetch 8 + 8 operand tiles per K step into its L2 rather than
  // 64 + 1.
  const uint32_t total = args.m_tiles * args.n_tiles;
  const uint32_t xcd = blockIdx.x % 8u;
  const uint32_t id = xcd * (total / 8u) + min(xcd, total % 8u) + blockIdx.x / 8u;
  const uint32_t band_tiles = kBand * args.n_tiles;
  const uint32_t band = id / band_tiles;
  const uint32_t in_band = id - band * band_tiles;
  const uint32_t height = min(kBand, args.m_tiles - band * kBand);
  const uint32_t m_tile = band * kBand + in_band % height;
  const uint32_t n_tile = in_band / height;
  const uint32_t first_m = m_tile * kRowsM;

  // weight streams of this wave's tiles (tiles past the matrix repeat the last
  // one and are not stored)
  const uint32_t tile_count = (args.rows + kTileRows - 1u) / kTileRows;
  const uint8_t* weight_stream[kTilesPerWave];
  const uint8_t* scale_stream[kTilesPerWave];
  uint32_t tile_index[kTilesPerWave];
#pragma unroll
  for (uint32_t t = 0; t < kTilesPerWave; ++t) {
    tile_index[t] = SWIGLU ? n_tile * kWaves + wave
                           : n_tile * kTilesN + wave * kTilesPerWave + t;
    const size_t stream = min(tile_index[t], tile_count - 1u);
    weight_stream[t] = (SWIGLU && t ? args.up_weights : args.weights) +
                       stream * chunks * (kTileRows * 32u) + (g * 16u + n) * 16u;
    scale_stream[t] =
        (SWIGLU && t ? args.up_scales : args.scales) +
        stream * chunks * (kTileRows * (F16 ? 8u : 2u)) +
        (F16 ? ((g >> 1) * 16u + n) * 8u : n * 4u);
  }

  // activation tile: thread -> (row, half of the 64 columns), 64 bytes.  Rows
  // past the batch stage row 0 again: their results are never stored, and a
  // load under a branch would make every wait for the weights conservative.
  const uint32_t stage_row = threadIdx.x >> 1;
  const uint32_t stage_half = threadIdx.x & 1u;
  const bool stage_live = first_m + stage_row < args.batch;
  const uint8_t* stage_source =
      reinterpret_cast<const uint8_t*>(args.activations) +
      (static_cast<size_t>(stage_live ? first_m + stage_row : 0u) * K +
       stage_half * 32u) * 2u;
  const uint32_t stage_target = stage_row * kLdsRow + stage_half * 64u;
  // fragment of m-tile mt, span s: row 16 mt + n, columns 32 s + 8 g .. + 8
  const uint32_t fragment_offset = n * kLdsRow + g * 16u;

  f32x4 acc[kTilesM][kTilesPerWave][2];
#pragma unroll
  for (uint32_t mt = 0; mt < kTilesM; ++mt)
#pragma unroll
    for (uint32_t t = 0; t < kTilesPerWave; ++t)
#pragma unroll
      for (uint32_t j = 0; j < 2u; ++j) acc[mt][t][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  uint4 staged[4];
  const auto fetch_activations = [&](uint32_t chunk) {
#pragma unroll
    for (uint32_t piece = 0; piece < 4u; ++piece)
      staged[piece] = *reinterpret_cast<const uint4*>(
          stage_source + static_cast<size_t>(chunk) * 128u + piece * 16u);
  };
  const auto store_activations = [&](uint32_t buffer) {
#pragma unroll
    for (uint32_t piece = 0; piece < 4u; ++piece) {
      uint4 v = staged[piece];
      v.x = Op::stage(v.x); v.y = Op::stage(v.y);
      v.z = Op::stage(v.z); v.w = Op::stage(v.w);
      *reinterpret_cast<uint4*>(&tile[buffer][stage_target + piece * 16u]) = v;
    }
  };
  // (slot indices are compile-time constants throughout: an array indexed by a
  // run-time slot would live in scratch memory, and every reload from there
  // would wait for the prefetch that was just issued)
  uint4 codes[2][kTilesPerWave];
  uint2 scales[2][kTilesPerWave];
  const auto fetch_weights = [&]<int slot>(std::integral_constant<int, slot>,
                                           uint32_t chunk) {
#pragma unroll
    for (uint32_t t = 0; t < kTilesPerWave; ++t) {
      codes[slot][t] = *reinterpret_cast<const uint4*>(
          weight_stream[t] + static_cast<size_t>(chunk) * (kTileRows * 32u));
      if constexpr (F16) {
        scales[slot][t] = *reinterpret_cast<const uint2*>(
            scale_stream[t] + static_cast<size_t>(chunk) * (kTileRows * 8u));
      } else {
        scales[slot][t].x = *reinterpret_cast<const uint32_t*>(
            scale_stream[t] + static_cast<size_t>(chunk) * (kTileRows * 2u));
        scales[slot][t].y = 0u;
      }
    }
  };

  fetch_activations(0u);
  fetch_weights(std::integral_constant<int, 0>{}, 0u);
  store_activations(0u);

  const auto step = [&]<int slot>(std::integral_constant<int, slot>,
                                  uint32_t chunk) {
    __syncthreads();   // tile[slot] is complete; tile[slot ^ 1] is free
    const uint32_t next = chunk + 1u < chunks ? chunk + 1u : chunk;
    fetch_activations(next);
    fetch_weights(std::integral_constant<int, slot ^ 1>{}, next);
    // the loads stay here, a whole step ahead of their use (left alone, the
    // scheduler sinks them to the end of the step to shorten live ranges)
    __builtin_amdgcn_sched_barrier(0);

    const uint8_t* current = tile[slot];
#pragma unroll
    for (uint32_t s = 0; s < 2u; ++s) {
      Vector a[kTilesM];
#pragma unroll
      for (uint32_t mt = 0; mt < kTilesM; ++mt)
        a[mt] = __builtin_bit_cast(
            Vector, *reinterpret_cast<const uint4*>(
                        current + mt * 16u * kLdsRow + fragment_offset + s * 64u));
#pragma unroll
      for (uint32_t t = 0; t < kTilesPerWave; ++t) {
        const uint4 q = codes[slot][t];
        const uint32_t packed[4] = {q.x, q.y, q.z, q.w};   // index 2j + s
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j) {
          // scale of (j, s): binary16 halves of the two words, or UE8M0 bytes
          const uint32_t word = j ? scales[slot][t].y : scales[slot][t].x;
          const uint32_t f16_bits = s ? word >> 16 : word & 0xffffu;
          const float fold =
              F16 ? 1.0f
                  : ue8m0_to_f32((scales[slot][t].x >> (8u * (2u * j + s))) & 0xffu);
          Vector w[Op::kParts];
          Op::weights(packed[2u * j + s], fold, f16_bits, w);
#pragma unroll
          for (int part = 0; part < Op::kParts; ++part)
#pragma unroll
            for (uint32_t mt = 0; mt < kTilesM; ++mt)
              acc[mt][t][j] = Op::mfma(a[mt], w[part], acc[mt][t][j]);
        }
      }
    }
    if (chunk + 1u < chunks) store_activations(slot ^ 1u);
  };
  for (uint32_t chunk = 0; chunk < chunks; chunk += 2u) {
    step(std::integral_constant<int, 0>{}, chunk);
    if (chunk + 1u < chunks) step(std::integral_constant<int, 1>{}, chunk + 1u);
  }

  // D register i of lane (n, g): activation row 16 mt + 4 g + i, weight row
  // 32 tile + 16 j + n
  if constexpr (SWIGLU) {
    if (tile_index[0] >= tile_count) return;
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
      const uint32_t column = tile_index[0] * kTileRows + 16u * j + n;
      if (column >= args.rows) continue;
#pragma unroll
      for (uint32_t mt = 0; mt < kTilesM; ++mt)
#pragma unroll
        for (uint32_t i = 0; i < 4u; ++i) {
          const uint32_t row = first_m + 16u * mt + 4u * g + i;
          if (row >= args.batch) continue;
          const float gate = acc[mt][0][j][i];
          const float activated = bf16_round(gate / (1.0f + expf(-gate)));
          static_cast<uint16_t*>(args.output)[static_cast<size_t>(row) * args.rows +
                                              column] =
              static_cast<uint16_t>(f32_to_bf16_bits(activated * acc[mt][1][j][i]));
        }
    }
    return;
  }
#pragma unroll
  for (uint32_t t = 0; t < kTilesPerWave; ++t) {
    if (tile_index[t] >= tile_count) continue;
    const uint32_t tile_first = tile_index[t] * kTileRows;
    // destination of the tile's columns (segments are multiples of 32 rows)
    void* destination = args.output;
    uint32_t kind = args.output_kind;
    uint32_t width = args.rows;
    uint32_t local_first = tile_first;
    if (args.segments) {
      uint32_t segment = 0;
      while (segment + 1u < args.segments &&
             local_first >= args.segment_rows[segment]) {
        local_first -= args.segment_rows[segment];
        ++segment;
      }
      destination = args.segment_output[segment];
      kind = args.segment_kind[segment];
      width = args.segment_rows[segment];
    }
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
      const uint32_t column = tile_first + 16u * j + n;
      if (column >= args.rows) continue;
      const uint32_t local_column = local_first + 16u * j + n;
#pragma unroll
      for (uint32_t mt = 0; mt < kTilesM; ++mt)
#pragma unroll
        for (uint32_t i = 0; i < 4u; ++i) {
          const uint32_t row = first_m + 16u * mt + 4u * g + i;
          if (row >= args.batch) continue;
          float value = acc[mt][t][j][i];
          if (args.residual && !args.segments)
            value += args.residual[static_cast<size_t>(row) * args.rows + column];
          store_value(destination, kind,
                      static_cast<size_t>(row) * width + local_column, value);
        }
    }
  }
}

bool tall_matrix_ok(const qllm_fp4_matrix* m) {
  return m && m->weights && m->scales && m->rows && m->columns &&
         m->padded_columns >= m->columns && m->padded_columns % kChunk == 0u &&
         (m->scale_scheme == QLLM_SCALE_UE8M0_BLOCK32 ||
          m->scale_scheme == QLLM_SCALE_F16_BLOCK16) &&
         m->layout == QLLM_LAYOUT_TILED &&
         (m->tile_rows == 0u || m->tile_rows == kTileRows);
}

int32_t launch_tall(TallArgs args, uint32_t scheme, hipStream_t stream) {
  args.m_tiles = (args.batch + kRowsM - 1u) / kRowsM;
  const bool swiglu = args.up_weights != nullptr;
  const uint32_t rows_per_workgroup = (swiglu ? kWaves : kTilesN) * kTileRows;
  args.n_tiles = (args.rows + rows_per_workgroup - 1u) / rows_per_workgroup;
  const uint32_t grid = args.m_tiles * args.n_tiles;
  if (swiglu && scheme == QLLM_SCALE_F16_BLOCK16)
    fp4_gemm_tall_kernel<kSchemeF16, true><<<grid, kWaves * 64, 0, stream>>>(args);
  else if (swiglu)
    fp4_gemm_tall_kernel<kSchemeUe8m0, true><<<grid, kWaves * 64, 0, stream>>>(args);
  else if (scheme == QLLM_SCALE_F16_BLOCK16)
    fp4_gemm_tall_kernel<kSchemeF16><<<grid, kWaves * 64, 0, stream>>>(args);
  else
    fp4_gemm_tall_kernel<kSchemeUe8m0><<<grid, kWaves * 64, 0, stream>>>(args);
  return launched("tall FP4 GEMM");
}

}  // namespace
}  // namespace qllm

using namespace qllm;

extern "C" int32_t qllm_fp4_gemm_bf16_tall(const qllm_fp4_matrix* matrix,
                                           const void* input, size_t input_bytes,
                                           void* output, uint32_t output_kind,
                                           const float* residual, uint32_t batch,
                                           void* stream) {
  if (!tall_matrix_ok(matrix) || !input || !output || !batch ||
      batch > (1u << 20) || output_kind > QLLM_OUT_BF16 ||
      (reinterpret_cast<uintptr_t>(input) & 15u) ||
      input_bytes < static_cast<size_t>(batch) * matrix->padded_columns * 2u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid tall FP4 GEMM");
  if (residual && output_kind == QLLM_OUT_BF16 &&
      static_cast<const void*>(residual) == output)
    return fail(QLLM_INVALID_ARGUMENT,
                "tall FP4 GEMM: bf16 output cannot alias the f32 residual");
  TallArgs args{};
  args.weights = matrix->weights;
  args.scales = static_cast<const uint8_t*>(matrix->scales);
  args.activations = static_cast<const uint16_t*>(input);
  args.rows = matrix->rows;
  args.padded_columns = matrix->padded_columns;
  args.batch = batch;
  args.output = output;
  args.output_kind = output_kind;
  args.residual = residual;
  return launch_tall(args, matrix->scale_scheme, as_stream(stream));
}

extern "C" int32_t qllm_fp4_swiglu_bf16_tall(const qllm_fp4_matrix* gate,
                                             const qllm_fp4_matrix* up,
                                             const void* input, size_t input_bytes,
                                             void* output_bf16, uint32_t batch,
                                             void* stream) {
  if (!tall_matrix_ok(gate) || !tall_matrix_ok(up) || gate->rows != up->rows ||
      gate->padded_columns != up->padded_columns ||
      gate->scale_scheme != up->scale_scheme || !input || !output_bf16 ||
      !batch || batch > (1u << 20) ||
      (reinterpret_cast<uintptr_t>(input) & 15u) ||
      input_bytes < static_cast<size_t>(batch) * gate->padded_columns * 2u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid tall FP4 SwiGLU");
  TallArgs args{};
  args.weights = gate->weights;
  args.scales = static_cast<const uint8_t*>(gate->scales);
  args.up_weights = up->weights;
  args.up_scales = static_cast<const uint8_t*>(up->scales);
  args.activations = static_cast<const uint16_t*>(input);
  args.rows = gate->rows;
  args.padded_columns = gate->padded_columns;
  args.batch = batch;
  args.output = output_bf16;
  args.output_kind = QLLM_OUT_BF16;
  return launch_tall(args, gate->scale_scheme, as_stream(stream));
}

extern "C" int32_t qllm_fp4_gemm_bf16_tall_split(
    const qllm_fp4_matrix* matrix, const void* input, size_t input_bytes,
    const qllm_gemm_segment* segments, uint32_t segment_count, uint32_t batch,
    void* stream) {
  if (!tall_matrix_ok(matrix) || !input || !segments || !segment_count ||
      segment_count > 3u || !batch || batch > (1u << 20) ||
      (reinterpret_cast<uintptr_t>(input) & 15u) ||
      input_bytes < static_cast<size_t>(batch) * matrix->padded_columns * 2u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid split tall FP4 GEMM");
  TallArgs args{};
  uint64_t total = 0;
  for (uint32_t index = 0; index < segment_count; ++index) {
    if (!segments[index].output || !segments[index].rows ||
        segments[index].rows % kTileRows || segments[index].output_kind > QLLM_OUT_BF16)
      return fail(QLLM_INVALID_ARGUMENT,
                  "split tall FP4 GEMM: segments must be multiples of 32 rows");
    args.segment_rows[index] = segments[index].rows;
    args.segment_kind[index] = segments[index].output_kind;
    args.segment_output[index] = segments[index].output;
    total += segments[index].rows;
  }
  if (total != matrix->rows)
    return fail(QLLM_INVALID_ARGUMENT,
                "split tall FP4 GEMM: segments do not cover the matrix");
  args.segments = segment_count;
  args.weights = matrix->weights;
  args.scales = static_cast<const uint8_t*>(matrix->scales);
  args.activations = static_cast<const uint16_t*>(input);
  args.rows = matrix->rows;
  args.padded_columns = matrix->padded_columns;
  args.batch = batch;
  return launch_tall(args, matrix->scale_scheme, as_stream(stream));
}
