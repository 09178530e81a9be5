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

namespace qllm {
namespace {

constexpr int kSchemeUe8m0 = QLLM_SCALE_UE8M0_BLOCK32;
constexpr int kSchemeF16 = QLLM_SCALE_F16_BLOCK16;

constexpr uint32_t kChunk = 64;            // K elements per wave step
constexpr uint32_t kLdsActivationBytes = 64 * 1024;

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
  uint32_t phase_columns;       // K handled per LDS staging phase
  uint32_t output_kind;
  uint32_t swiglu;              // tile 1 is the up projection of tile 0
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

// Workgroup = WAVES waves.  The workgroup owns TILES tiles of 32 weight rows;
// its waves interleave over 64-column chunks of K (wave w takes chunks
// w, w+WAVES, ...), so together they stream whole 128-byte lines of each row.
// Lane (n = lane%32, g = lane/32) loads the 16 bytes at
//   row n, byte offset chunk*32 + g*16
// i.e. 16-blocks {2g, 2g+1} of the chunk.  One v_permlane32_swap per dword
// pair regroups that into "half g of block b" - the B-operand layout of the
// 32x32x16 MFMA - without touching LDS.
template <int SCHEME, int BATCH, int TILES, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void fp4_gemm_mfma_kernel(
    const GemmArgs args) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  uint4* fragments = reinterpret_cast<uint4*>(lds_raw);

  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t n = lane & 31u;
  const uint32_t g = lane >> 5;
  const uint32_t K = args.padded_columns;
  const uint32_t row_bytes = K / 2u;
  const uint32_t scale_row_bytes =
      SCHEME == kSchemeF16 ? K / 8u : K / 32u;
  const uint32_t m_lane = n < BATCH ? n : BATCH - 1u;

  const uint8_t* weight_row[TILES];
  const uint8_t* scale_row[TILES];
  uint32_t out_row[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    uint32_t row;
    if (args.swiglu)
      row = blockIdx.x * 32u + n;
    else
      row = (blockIdx.x * TILES + t) * 32u + n;
    out_row[t] = row;
    const uint32_t safe = row < args.rows ? row : args.rows - 1u;
    weight_row[t] = args.tile[t].weights + static_cast<size_t>(safe) * row_bytes +
                    g * 16u;
    scale_row[t] = args.tile[t].scales + static_cast<size_t>(safe) * scale_row_bytes;
  }

  // F16 scheme: per-block results are scaled in F32 after the MFMA.
  // UE8M0 scheme: the power-of-two scale is folded into the nibble->bf16
  // conversion (exact), so the MFMA accumulates across the whole K range.
  float acc[TILES][4];
  f32x16 macc[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[t][i] = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) macc[t][i] = 0.0f;
  }

  constexpr int PF = 4;  // chunks in flight per lane
  for (uint32_t phase_begin = 0; phase_begin < K;
       phase_begin += args.phase_columns) {
    const uint32_t phase_columns =
        min(args.phase_columns, K - phase_begin);
    const uint32_t phase_chunks = phase_columns / kChunk;
    const uint32_t my_chunks =
        phase_chunks > wave ? (phase_chunks - wave + WAVES - 1u) / WAVES : 0u;

    uint4 codes[PF][TILES];
    uint2 scales[PF][TILES];
    auto issue = [&](int slot, uint32_t index) {
      const uint32_t chunk = phase_begin / kChunk + wave + index * WAVES;
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
        codes[slot][t] = load_stream16(weight_row[t] + chunk * 32u);
        if (SCHEME == kSchemeF16) {
          scales[slot][t] = load_stream8(scale_row[t] + chunk * 8u);
        } else {
          const uint32_t pair = *reinterpret_cast<const uint16_t*>(
              scale_row[t] + chunk * 2u);
          scales[slot][t] = make_uint2(pair & 0xffu, pair >> 8);
        }
      }
    };
#pragma unroll
    for (int slot = 0; slot < PF; ++slot)
      if (static_cast<uint32_t>(slot) < my_chunks) issue(slot, slot);

    // Stage this phase's activations into LDS in fragment order:
    // fragments[(block*2 + half)*BATCH + m] = act[m][block*16 + half*8 .. +8].
    __syncthreads();  // previous phase's readers are done
    {
      const uint32_t pieces_per_row = phase_columns / 8u;
      const uint32_t pieces = pieces_per_row * BATCH;
      for (uint32_t piece = threadIdx.x; piece < pieces;
           piece += WAVES * 64u) {
        const uint32_t m = piece / pieces_per_row;
        const uint32_t position = piece - m * pieces_per_row;
        const uint4 value = *reinterpret_cast<const uint4*>(
            args.activations + static_cast<size_t>(m) * K + phase_begin +
            position * 8u);
        fragments[position * BATCH + m] = value;
      }
    }
    __syncthreads();

    for (uint32_t base = 0; base < my_chunks; base += PF) {
#pragma unroll
      for (int slot = 0; slot < PF; ++slot) {
        const uint32_t index = base + slot;
        if (index >= my_chunks) break;
        uint4 q[TILES];
        uint2 s[TILES];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
          q[t] = codes[slot][t];
          s[t] = scales[slot][t];
        }
        if (index + PF < my_chunks) issue(slot, index + PF);

        const uint32_t local_chunk = wave + index * WAVES;
        // activation fragments of the four 16-blocks of this chunk
        bf16x8 a[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const uint4 raw =
              fragments[((local_chunk * 4u + b) * 2u + g) * BATCH + m_lane];
          a[b] = __builtin_bit_cast(bf16x8, raw);
        }
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
          const auto s01 = __builtin_amdgcn_permlane32_swap(q[t].x, q[t].y,
                                                            false, false);
          const auto s23 = __builtin_amdgcn_permlane32_swap(q[t].z, q[t].w,
                                                            false, false);
          // block order inside the chunk: s01[0]=b0, s23[0]=b1, s01[1]=b2,
          // s23[1]=b3
          const uint32_t packed[4] = {s01[0], s23[0], s01[1], s23[1]};
          if (SCHEME == kSchemeF16) {
            const float scale[4] = {
                f16_bits_to_f32(s[t].x & 0xffffu), f16_bits_to_f32(s[t].x >> 16),
                f16_bits_to_f32(s[t].y & 0xffffu), f16_bits_to_f32(s[t].y >> 16)};
#pragma unroll
            for (int b = 0; b < 4; ++b) {
              const bf16x8 w = expand_fp4x8(packed[b], 1.0f);
              f32x16 zero;
#pragma unroll
              for (int i = 0; i < 16; ++i) zero[i] = 0.0f;
              const f32x16 d = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  a[b], w, zero, 0, 0, 0);
#pragma unroll
              for (int i = 0; i < 4; ++i)
                acc[t][i] = fmaf(d[i], scale[b], acc[t][i]);
            }
          } else {
            const float scale_low = ue8m0_to_f32(s[t].x);
            const float scale_high = ue8m0_to_f32(s[t].y);
#pragma unroll
            for (int b = 0; b < 4; ++b) {
              const bf16x8 w =
                  expand_fp4x8(packed[b], b < 2 ? scale_low : scale_high);
              macc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                  a[b], w, macc[t], 0, 0, 0);
            }
          }
        }
      }
    }
  }

  if (SCHEME != kSchemeF16) {
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[t][i] = macc[t][i];
  }

  // Cross-wave reduction through LDS (reuses the activation staging area).
  __syncthreads();
  float* reduce = reinterpret_cast<float*>(lds_raw);
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      reduce[((wave * TILES + t) * 4 + i) * 64 + lane] = acc[t][i];
  __syncthreads();

  const uint32_t items = (args.swiglu ? 1u : TILES) * 256u;
  for (uint32_t item = threadIdx.x; item < items; item += WAVES * 64u) {
    const uint32_t t = item >> 8;
    const uint32_t i = (item >> 6) & 3u;
    const uint32_t source_lane = item & 63u;
    const uint32_t m = 4u * (source_lane >> 5) + i;
    const uint32_t row =
        args.swiglu ? blockIdx.x * 32u + (source_lane & 31u)
                    : (blockIdx.x * TILES + t) * 32u + (source_lane & 31u);
    if (m >= BATCH || row >= args.rows) continue;
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w)
      total += reduce[((w * TILES + t) * 4 + i) * 64 + source_lane];
    const size_t index = static_cast<size_t>(m) * args.rows + row;
    if (args.swiglu) {
      float up = 0.0f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w)
        up += reduce[((w * TILES + (TILES - 1)) * 4 + i) * 64 + source_lane];
      const float activated = bf16_round(total / (1.0f + __expf(-total)));
      static_cast<uint16_t*>(args.output)[index] =
          static_cast<uint16_t>(f32_to_bf16_bits(activated * up));
    } else {
      if (args.residual) total += args.residual[index];
      store_output(args.output, args.output_kind, index, total);
    }
  }
  (void)out_row;
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
          m->scale_scheme == QLLM_SCALE_F16_BLOCK16);
}

uint32_t phase_columns_for(uint32_t K, uint32_t batch, uint32_t waves) {
  const uint32_t granule = kChunk * waves;
  const uint32_t limit = kLdsActivationBytes / (2u * batch) / granule * granule;
  if (K <= limit) return K;
  const uint32_t phases = (K + limit - 1u) / limit;
  return ((K + phases - 1u) / phases + granule - 1u) / granule * granule;
}

template <int SCHEME, int BATCH, int TILES>
int32_t launch_mfma_waves(const GemmArgs& args, uint32_t grid, uint32_t waves,
                          size_t lds_bytes, hipStream_t stream) {
  switch (waves) {
    case 4:
      fp4_gemm_mfma_kernel<SCHEME, BATCH, TILES, 4>
          <<<grid, 256, lds_bytes, stream>>>(args);
      break;
    case 8:
      fp4_gemm_mfma_kernel<SCHEME, BATCH, TILES, 8>
          <<<grid, 512, lds_bytes, stream>>>(args);
      break;
    default:
      fp4_gemm_mfma_kernel<SCHEME, BATCH, TILES, 16>
          <<<grid, 1024, lds_bytes, stream>>>(args);
      break;
  }
  return launched("FP4 MFMA GEMM");
}

template <int SCHEME, int TILES>
int32_t launch_mfma_batch(const GemmArgs& args, uint32_t batch, uint32_t grid,
                          uint32_t waves, size_t lds_bytes,
                          hipStream_t stream) {
  switch (batch) {
    case 1: return launch_mfma_waves<SCHEME, 1, TILES>(args, grid, waves, lds_bytes, stream);
    case 2: return launch_mfma_waves<SCHEME, 2, TILES>(args, grid, waves, lds_bytes, stream);
    case 3: return launch_mfma_waves<SCHEME, 3, TILES>(args, grid, waves, lds_bytes, stream);
    case 4: return launch_mfma_waves<SCHEME, 4, TILES>(args, grid, waves, lds_bytes, stream);
    case 5: return launch_mfma_waves<SCHEME, 5, TILES>(args, grid, waves, lds_bytes, stream);
    case 6: return launch_mfma_waves<SCHEME, 6, TILES>(args, grid, waves, lds_bytes, stream);
    case 7: return launch_mfma_waves<SCHEME, 7, TILES>(args, grid, waves, lds_bytes, stream);
    default: return launch_mfma_waves<SCHEME, 8, TILES>(args, grid, waves, lds_bytes, stream);
  }
}

// Chooses tiles per workgroup and waves per workgroup so that the launch
// keeps roughly 3-5 thousand waves in flight on 256 CUs (4 SIMDs each).
int32_t launch_mfma(GemmArgs args, int scheme, uint32_t batch, bool swiglu,
                    hipStream_t stream) {
  const uint32_t tiles = (args.rows + 31u) / 32u;
  uint32_t tiles_per_group = 1u;
  uint32_t waves = 4u;
  if (swiglu) {
    tiles_per_group = 2u;
    waves = tiles >= 768u ? 4u : (tiles >= 384u ? 8u : 16u);
  } else if (tiles >= 1024u) {
    tiles_per_group = 2u;
  } else if (tiles < 384u) {
    waves = tiles >= 192u ? 8u : 16u;
  }
  const uint32_t grid =
      swiglu ? tiles : (tiles + tiles_per_group - 1u) / tiles_per_group;
  args.phase_columns = phase_columns_for(args.padded_columns, batch, waves);
  args.swiglu = swiglu ? 1u : 0u;
  const size_t stage_bytes =
      static_cast<size_t>(args.phase_columns) * 2u * batch;
  const size_t reduce_bytes =
      static_cast<size_t>(waves) * tiles_per_group * 4u * 64u * sizeof(float);
  const size_t lds_bytes = stage_bytes > reduce_bytes ? stage_bytes : reduce_bytes;
  if (scheme == kSchemeF16) {
    if (tiles_per_group == 2u)
      return launch_mfma_batch<kSchemeF16, 2>(args, batch, grid, waves, lds_bytes, stream);
    return launch_mfma_batch<kSchemeF16, 1>(args, batch, grid, waves, lds_bytes, stream);
  }
  if (tiles_per_group == 2u)
    return launch_mfma_batch<kSchemeUe8m0, 2>(args, batch, grid, waves, lds_bytes, stream);
  return launch_mfma_batch<kSchemeUe8m0, 1>(args, batch, grid, waves, lds_bytes, stream);
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
    return launch_mfma(args, static_cast<int>(matrix->scale_scheme), batch,
                       false, as_stream(stream));
  }
  const uint32_t grid = (matrix->rows + 3u) / 4u;
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

extern "C" int32_t qllm_fp4_swiglu_bf16(const qllm_fp4_matrix* gate,
                                        const qllm_fp4_matrix* up,
                                        const void* input, size_t input_bytes,
                                        void* output, uint32_t batch,
                                        void* stream) {
  if (!matrix_ok(gate) || !matrix_ok(up) || gate->rows != up->rows ||
      gate->padded_columns != up->padded_columns ||
      gate->scale_scheme != up->scale_scheme || !input || !output || !batch ||
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
  return launch_mfma(args, static_cast<int>(gate->scale_scheme), batch, true,
                     as_stream(stream));
}

extern "C" int32_t qllm_fp4_gemv_q8_batch(const qllm_fp4_matrix* matrix,
                                          const int8_t* input,
                                          const float* input_scales,
                                          float* output, uint32_t batch,
                                          int32_t bf16_output, void* stream) {
  if (!matrix_ok(matrix) || matrix->scale_scheme != QLLM_SCALE_UE8M0_BLOCK32 ||
      !input || !input_scales || !output || !batch || batch > 8u)
    return fail(QLLM_INVALID_ARGUMENT, "invalid FP4 Q8 weight-reuse GEMV");
  const uint32_t grid = (matrix->rows + 3u) / 4u;
  fp4_gemv_generic_kernel<kSchemeUe8m0, true>
      <<<grid, 256, 0, as_stream(stream)>>>(
          matrix->weights, static_cast<const uint8_t*>(matrix->scales), input,
          input_scales, output, nullptr, matrix->rows, matrix->padded_columns,
          batch, bf16_output ? QLLM_OUT_F32_BF16_ROUNDED : QLLM_OUT_F32);
  return launched("FP4 Q8 weight-reuse GEMV");
}
