// Token selection over the lm_head logits: batched argmax, exact descending
// top-k and the presence penalty.  Replaces argmax_batch_kernel,
// topk_logits_partials_kernel / topk_logits_reduce_kernel and
// presence_penalty_kernel (runtime/src/cuda/transformer_kernels.cu:7059-7186).
// Ordering rule everywhere: larger value first, equal values by lower index,
// NaN never selected.
#include "common.hpp"

#include <mutex>

namespace qllm {
namespace {

constexpr uint32_t kNoIndex = 0xffffffffu;
constexpr uint32_t kArgmaxChunk = 2048;   // items per stage-1 block
constexpr uint32_t kTopkChunk = 4096;     // items per stage-1 block
constexpr uint32_t kTopkThreads = 256;
constexpr uint32_t kTopkPerThread = kTopkChunk / kTopkThreads;

__device__ __forceinline__ bool better(float value, uint32_t index, float best,
                                       uint32_t best_index) {
  return value > best || (value == best && index < best_index);
}

__device__ __forceinline__ void wave_best(float& value, uint32_t& index) {
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) {
    const float other = __shfl_xor(value, offset, 64);
    const uint32_t other_index = __shfl_xor(index, offset, 64);
    if (better(other, other_index, value, index)) {
      value = other;
      index = other_index;
    }
  }
}

// Block-wide best; result valid in every thread.
__device__ __forceinline__ void block_best(float& value, uint32_t& index,
                                           float* values, uint32_t* indices) {
  wave_best(value, index);
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t waves = (blockDim.x + 63u) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63u) == 0u) {
    values[wave] = value;
    indices[wave] = index;
  }
  __syncthreads();
  value = values[0];
  index = indices[0];
  for (uint32_t other = 1; other < waves; ++other)
    if (better(values[other], indices[other], value, index)) {
      value = values[other];
      index = indices[other];
    }
}

__global__ __launch_bounds__(256) void argmax_partial_kernel(
    const float* values, uint32_t count, float* partial_values,
    uint32_t* partial_indices, uint32_t blocks_per_row) {
  __shared__ float shared_values[4];
  __shared__ uint32_t shared_indices[4];
  const uint32_t request = blockIdx.y;
  const float* row = values + static_cast<size_t>(request) * count;
  const uint32_t first = blockIdx.x * kArgmaxChunk;
  const uint32_t last = min(count, first + kArgmaxChunk);
  float best = -INFINITY;
  uint32_t index = kNoIndex;
  if (last - first == kArgmaxChunk &&
      (reinterpret_cast<uintptr_t>(row + first) & 15u) == 0u) {
    // a whole, aligned chunk: both 16-byte loads of a thread are in flight
    // before the first comparison
    float4 loaded[kArgmaxChunk / 1024u];
#pragma unroll
    for (uint32_t part = 0; part < kArgmaxChunk / 1024u; ++part)
      loaded[part] = *reinterpret_cast<const float4*>(
          row + first + part * 1024u + threadIdx.x * 4u);
#pragma unroll
    for (uint32_t part = 0; part < kArgmaxChunk / 1024u; ++part) {
      const uint32_t item = first + part * 1024u + threadIdx.x * 4u;
      const float four[4] = {loaded[part].x, loaded[part].y, loaded[part].z,
                             loaded[part].w};
#pragma unroll
      for (uint32_t lane = 0; lane < 4u; ++lane)
        if (better(four[lane], item + lane, best, index)) {
          best = four[lane];
          index = item + lane;
        }
    }
  } else {
    for (uint32_t item = first + threadIdx.x; item < last; item += blockDim.x) {
      const float value = row[item];
      if (better(value, item, best, index)) {
        best = value;
        index = item;
      }
    }
  }
  block_best(best, index, shared_values, shared_indices);
  if (threadIdx.x == 0u) {
    partial_values[request * blocks_per_row + blockIdx.x] = best;
    partial_indices[request * blocks_per_row + blockIdx.x] = index;
  }
}

// `advance.positions` non-null (one row): thread 0 also does what
// rollout_advance_kernel does with the winner.
__global__ __launch_bounds__(256) void argmax_final_kernel(
    const float* partial_values, const uint32_t* partial_indices,
    uint32_t blocks_per_row, uint32_t* output, RolloutAdvance advance) {
  __shared__ float shared_values[4];
  __shared__ uint32_t shared_indices[4];
  const uint32_t request = blockIdx.x;
  float best = -INFINITY;
  uint32_t index = kNoIndex;
  for (uint32_t item = threadIdx.x; item < blocks_per_row; item += blockDim.x) {
    const float value = partial_values[request * blocks_per_row + item];
    const uint32_t candidate = partial_indices[request * blocks_per_row + item];
    if (better(value, candidate, best, index)) {
      best = value;
      index = candidate;
    }
  }
  block_best(best, index, shared_values, shared_indices);
  if (threadIdx.x != 0u) return;
  output[request] = index;
  if (advance.positions && request == 0u) {
    const uint32_t slot = advance.positions[3];
    advance.next_token[0] = index;
    if (slot < advance.capacity) advance.draft_tokens[slot] = index;
    advance.positions[0] += advance.rows;
    advance.positions[1] += advance.rows;
    advance.positions[2] += advance.rows;
    advance.positions[3] = slot + 1u;
  }
}

__global__ __launch_bounds__(64) void rollout_advance_kernel(
    const uint32_t* selected, uint32_t* next_token, uint32_t* draft_tokens,
    uint32_t capacity, uint32_t rows, uint32_t* positions) {
  if (threadIdx.x != 0u) return;
  const uint32_t token = selected[0];
  const uint32_t slot = positions[3];
  next_token[0] = token;
  if (slot < capacity) draft_tokens[slot] = token;
  positions[0] += rows;
  positions[1] += rows;
  positions[2] += rows;
  positions[3] = slot + 1u;
}

// Stage 1: every block extracts the top_k of its chunk, in order, by top_k
// rounds of "block argmax, winner retires".  Stage 2 (one block) does the
// same over the stage-1 survivors.  Items live in registers.
template <uint32_t PER_THREAD>
__device__ __forceinline__ void select_rounds(float (&value)[PER_THREAD],
                                              uint32_t (&index)[PER_THREAD],
                                              uint32_t top_k, float* out_values,
                                              uint32_t* out_indices,
                                              float* shared_values,
                                              uint32_t* shared_indices) {
  for (uint32_t rank = 0; rank < top_k; ++rank) {
    float best = -INFINITY;
    uint32_t best_index = kNoIndex;
#pragma unroll
    for (uint32_t slot = 0; slot < PER_THREAD; ++slot)
      if (index[slot] != kNoIndex &&
          better(value[slot], index[slot], best, best_index)) {
        best = value[slot];
        best_index = index[slot];
      }
    block_best(best, best_index, shared_values, shared_indices);
    if (threadIdx.x == 0u) {
      out_values[rank] = best;
      out_indices[rank] = best_index;
    }
    if (best_index == kNoIndex) {
      // fewer than top_k candidates: pad the remaining ranks
      for (uint32_t rest = rank + 1u + threadIdx.x; rest < top_k;
           rest += blockDim.x) {
        out_values[rest] = -INFINITY;
        out_indices[rest] = kNoIndex;
      }
      return;
    }
#pragma unroll
    for (uint32_t slot = 0; slot < PER_THREAD; ++slot)
      if (index[slot] == best_index) index[slot] = kNoIndex;
  }
}

__global__ __launch_bounds__(kTopkThreads) void topk_partial_kernel(
    const float* values, uint32_t count, uint32_t top_k, float* partial_values,
    uint32_t* partial_indices) {
  __shared__ float shared_values[4];
  __shared__ uint32_t shared_indices[4];
  const uint32_t first = blockIdx.x * kTopkChunk;
  float value[kTopkPerThread];
  uint32_t index[kTopkPerThread];
#pragma unroll
  for (uint32_t slot = 0; slot < kTopkPerThread; ++slot) {
    const uint32_t item = first + slot * kTopkThreads + threadIdx.x;
    float loaded = item < count ? values[item] : NAN;
    const bool usable = item < count && !isnan(loaded);
    value[slot] = usable ? loaded : -INFINITY;
    index[slot] = usable ? item : kNoIndex;
  }
  select_rounds<kTopkPerThread>(value, index, top_k,
                                partial_values + blockIdx.x * top_k,
                                partial_indices + blockIdx.x * top_k,
                                shared_values, shared_indices);
}

constexpr uint32_t kMergeThreads = 1024;
constexpr uint32_t kMergePerThread = 40;  // up to 40960 survivors

__global__ __launch_bounds__(kMergeThreads) void topk_merge_kernel(
    const float* partial_values, const uint32_t* partial_indices,
    uint32_t survivors, uint32_t top_k, float* output_values,
    uint32_t* output_indices) {
  __shared__ float shared_values[16];
  __shared__ uint32_t shared_indices[16];
  float value[kMergePerThread];
  uint32_t index[kMergePerThread];
#pragma unroll
  for (uint32_t slot = 0; slot < kMergePerThread; ++slot) {
    const uint32_t item = slot * kMergeThreads + threadIdx.x;
    const bool usable = item < survivors && partial_indices[item] != kNoIndex;
    value[slot] = usable ? partial_values[item] : -INFINITY;
    index[slot] = usable ? partial_indices[item] : kNoIndex;
  }
  select_rounds<kMergePerThread>(value, index, top_k, output_values,
                                 output_indices, shared_values, shared_indices);
}

// ---- batched top-k by threshold ------------------------------------------------
//
// The k rounds above cost a block reduction each.  For k <= 64 the rows of a
// batch are served by two launches instead:
//   1. the maximum of every chunk of `chunk` items (one wave per chunk);
//   2. per row, one workgroup: the k-th largest chunk maximum is a threshold
//      that at least k items reach (the chunk maxima themselves), so the top k
//      lie among the items >= threshold; those - a few hundred for logits
//      whose large values are spread over the vocabulary - are gathered into
//      LDS and ranked against each other, rank r going to output slot r.
// With fewer chunks than k the threshold is -inf (every item is a candidate).
// If more candidates turn up than LDS holds (large values packed into a few
// chunks), the workgroup falls back to k rounds over the whole row.  Results
// are those of the rounds: same order, same ties, NaN excluded, missing ranks
// padded with (-inf, no index).
constexpr uint32_t kSelectThreads = 1024;
constexpr uint32_t kSelectCandidates = 4096;
constexpr uint32_t kSelectMaxChunks = 4096;
constexpr uint32_t kSelectMaxK = 64;

__global__ __launch_bounds__(256) void chunk_max_kernel(
    const float* values, uint32_t count, size_t row_stride, uint32_t chunk,
    uint32_t chunks_per_row, float* maxima) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t index = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (index >= chunks_per_row) return;
  const float* row = values + blockIdx.y * row_stride;
  const uint32_t first = index * chunk;
  const uint32_t last = min(count, first + chunk);
  float best = -INFINITY;
  for (uint32_t item = first + lane; item < last; item += 64u) {
    const float value = row[item];
    if (value > best) best = value;   // NaN never wins
  }
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1)
    best = fmaxf(best, __shfl_xor(best, offset, 64));
  if (lane == 0u) maxima[blockIdx.y * chunks_per_row + index] = best;
}

__global__ __launch_bounds__(kSelectThreads) void topk_threshold_kernel(
    const float* values, uint32_t count, size_t row_stride, uint32_t top_k,
    const float* maxima, uint32_t chunks_per_row, float* output_values,
    uint32_t* output_indices) {
  __shared__ float candidate_values[kSelectCandidates];
  __shared__ uint32_t candidate_indices[kSelectCandidates];
  __shared__ float threshold;
  __shared__ uint32_t candidates;
  __shared__ float shared_values[16];
  __shared__ uint32_t shared_indices[16];
  const float* row = values + blockIdx.x * row_stride;
  float* out_values = output_values + static_cast<size_t>(blockIdx.x) * top_k;
  uint32_t* out_indices = output_indices + static_cast<size_t>(blockIdx.x) * top_k;

  // the k-th largest chunk maximum (staged in candidate_values)
  if (threadIdx.x == 0u) {
    threshold = -INFINITY;
    candidates = 0u;
  }
  for (uint32_t item = threadIdx.x; item < chunks_per_row; item += kSelectThreads)
    candidate_values[item] = maxima[blockIdx.x * chunks_per_row + item];
  __syncthreads();
  if (chunks_per_row >= top_k)
    for (uint32_t item = threadIdx.x; item < chunks_per_row; item += kSelectThreads) {
      const float mine = candidate_values[item];
      uint32_t rank = 0;
      for (uint32_t other = 0; other < chunks_per_row; ++other) {
        const float value = candidate_values[other];
        rank += value > mine || (value == mine && other < item) ? 1u : 0u;
      }
      if (rank == top_k - 1u) threshold = mine;
    }
  __syncthreads();
  const float limit = threshold;
  __syncthreads();   // the staged maxima are overwritten from here on

  for (uint32_t item = threadIdx.x; item < count; item += kSelectThreads) {
    const float value = row[item];
    if (value >= limit) {   // false for NaN
      const uint32_t slot = atomicAdd(&candidates, 1u);
      if (slot < kSelectCandidates) {
        candidate_values[slot] = value;
        candidate_indices[slot] = item;
      }
    }
  }
  __syncthreads();
  const uint32_t found = candidates;

  if (found <= kSelectCandidates) {
    for (uint32_t item = threadIdx.x; item < found; item += kSelectThreads) {
      const float mine = candidate_values[item];
      const uint32_t mine_index = candidate_indices[item];
      uint32_t rank = 0;
      for (uint32_t other = 0; other < found; ++other)
        rank += better(candidate_values[other], candidate_indices[other], mine,
                       mine_index) ? 1u : 0u;
      if (rank < top_k) {
        out_values[rank] = mine;
        out_indices[rank] = mine_index;
      }
    }
    for (uint32_t rank = found + threadIdx.x; rank < top_k; rank += kSelectThreads) {
      out_values[rank] = -INFINITY;
      out_indices[rank] = kNoIndex;
    }
    return;
  }

  // More candidates than LDS holds: k rounds over the row, each taking the
  // best item that comes after the previous winner in the order.
  float previous = INFINITY;
  uint32_t previous_index = 0u;
  bool first_round = true;
  for (uint32_t rank = 0; rank < top_k; ++rank) {
    float best = -INFINITY;
    uint32_t best_index = kNoIndex;
    for (uint32_t item = threadIdx.x; item < count; item += kSelectThreads) {
      const float value = row[item];
      if (isnan(value)) continue;
      if (!first_round && !better(previous, previous_index, value, item)) continue;
      if (best_index == kNoIndex || better(value, item, best, best_index)) {
        best = value;
        best_index = item;
      }
    }
    block_best(best, best_index, shared_values, shared_indices);
    if (threadIdx.x == 0u) {
      out_values[rank] = best_index == kNoIndex ? -INFINITY : best;
      out_indices[rank] = best_index;
    }
    if (best_index == kNoIndex) {
      for (uint32_t rest = rank + 1u + threadIdx.x; rest < top_k;
           rest += kSelectThreads) {
        out_values[rest] = -INFINITY;
        out_indices[rest] = kNoIndex;
      }
      return;
    }
    previous = best;
    previous_index = best_index;
    first_round = false;
  }
}

// chunk size: a power of two >= 64 aiming at 4 k chunks per row, at most
// kSelectMaxChunks chunks
uint32_t select_chunk(uint32_t count, uint32_t top_k) {
  uint32_t chunk = 64u;
  while (chunk * 2u <= count / (4u * top_k)) chunk *= 2u;
  while ((count + chunk - 1u) / chunk > kSelectMaxChunks) chunk *= 2u;
  return chunk;
}

// transformer_kernels.cu:7180-7186
__global__ void presence_penalty_kernel(float* logits, const uint8_t* emitted,
                                        uint32_t count, float penalty) {
  const uint32_t index = blockIdx.x * blockDim.x + threadIdx.x;
  if (index < count && emitted[index] != 0u) logits[index] -= penalty;
}

// The verify step's rows in one launch: row r is penalised where a token was
// emitted before the step or is one of the drafts the rows before r carry
// (the reference penalises row by row and marks draft r in a scratch copy of
// the presence bytes in between, dense_fp4_provider.cpp:11182-11202).
__global__ __launch_bounds__(256) void presence_penalty_rows_kernel(
    float* logits, size_t row_stride, const uint8_t* emitted,
    const uint32_t* drafts, uint32_t rows, uint32_t count, float penalty) {
  const uint32_t index = blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= count) return;
  bool present = emitted[index] != 0u;
  for (uint32_t row = 0; row < rows; ++row) {
    if (present) logits[row * row_stride + index] -= penalty;
    if (row + 1u < rows && drafts[row] == index) present = true;
  }
}

__global__ __launch_bounds__(64) void mark_presence_kernel(
    uint8_t* emitted, const uint32_t* tokens, uint32_t token_count,
    uint32_t count) {
  if (threadIdx.x < token_count && tokens[threadIdx.x] < count)
    emitted[tokens[threadIdx.x]] = 1u;
}

}  // namespace

int32_t launch_argmax_final(const float* partial_values,
                            const uint32_t* partial_indices, uint32_t blocks,
                            uint32_t batch, uint32_t* output,
                            const RolloutAdvance* advance, hipStream_t stream) {
  argmax_final_kernel<<<batch, 256, 0, stream>>>(
      partial_values, partial_indices, blocks, output,
      advance ? *advance : RolloutAdvance{});
  return launched("argmax of the head's tile maxima");
}

}  // namespace qllm

using namespace qllm;

extern "C" size_t qllm_argmax_workspace_bytes(uint32_t count, uint32_t batch) {
  const size_t blocks = (static_cast<size_t>(count) + kArgmaxChunk - 1u) / kArgmaxChunk;
  return blocks * batch * (sizeof(float) + sizeof(uint32_t));
}

extern "C" int32_t qllm_argmax_batch(const float* values, uint32_t count,
                                     uint32_t batch, uint32_t* output,
                                     void* workspace, size_t workspace_bytes,
                                     void* stream) {
  if (!values || !count || !batch || !output || !workspace ||
      workspace_bytes < qllm_argmax_workspace_bytes(count, batch))
    return fail(QLLM_INVALID_ARGUMENT, "invalid argmax batch");
  const uint32_t blocks = (count + kArgmaxChunk - 1u) / kArgmaxChunk;
  float* partial_values = static_cast<float*>(workspace);
  uint32_t* partial_indices = reinterpret_cast<uint32_t*>(
      partial_values + static_cast<size_t>(blocks) * batch);
  argmax_partial_kernel<<<dim3(blocks, batch), 256, 0, as_stream(stream)>>>(
      values, count, partial_values, partial_indices, blocks);
  argmax_final_kernel<<<batch, 256, 0, as_stream(stream)>>>(
      partial_values, partial_indices, blocks, output, RolloutAdvance{});
  return launched("argmax batch");
}

// ---- argmax without an allocation -------------------------------------------
// The stage-1 partials of qllm_argmax_batch in a fixed array inside the code
// object instead of a caller's workspace.  Each device that loads the library
// holds its own copy; host code reaches it through the address
// hipGetSymbolAddress reports for the current device, never through the
// array's name.
namespace qllm {
namespace {

constexpr size_t kStaticArgmaxBytes = 64u * 1024u;
constexpr int kStaticArgmaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticArgmaxBytes];

std::mutex static_argmax_mutex;
void* static_argmax_address[kStaticArgmaxDevices] = {};

// Address of `scratch` on the current device, looked up once per device.
int32_t static_argmax_scratch(void** address) {
  int device = -1;
  if (const int32_t status = checked(hipGetDevice(&device), "hipGetDevice"))
    return status;
  if (device < 0 || device >= kStaticArgmaxDevices)
    return fail(QLLM_INVALID_ARGUMENT, "argmax static: device index above 63");
  std::lock_guard<std::mutex> guard(static_argmax_mutex);
  if (!static_argmax_address[device]) {
    void* found = nullptr;
    if (const int32_t status =
            checked(hipGetSymbolAddress(&found, HIP_SYMBOL(scratch)),
                    "hipGetSymbolAddress(argmax scratch)"))
      return status;
    if (!found) return fail(QLLM_INTERNAL, "argmax static: no scratch address");
    static_argmax_address[device] = found;
  }
  *address = static_argmax_address[device];
  return QLLM_OK;
}

}  // namespace
}  // namespace qllm

extern "C" size_t qllm_argmax_static_capacity_bytes(void) {
  return kStaticArgmaxBytes;
}

extern "C" int32_t qllm_argmax_batch_static(const float* values, uint32_t count,
                                            uint32_t batch, uint32_t* output,
                                            void* stream) {
  if (!values || !count || !batch || !output)
    return fail(QLLM_INVALID_ARGUMENT, "invalid argmax batch");
  if (qllm_argmax_workspace_bytes(count, batch) > kStaticArgmaxBytes)
    return fail(QLLM_INVALID_ARGUMENT,
                "argmax static: ceil(count / 2048) * batch exceeds 8192 "
                "(the 64 KiB scratch array); use qllm_argmax_batch with a "
                "workspace");
  void* workspace = nullptr;
  if (const int32_t status = static_argmax_scratch(&workspace)) return status;
  const uint32_t blocks = (count + kArgmaxChunk - 1u) / kArgmaxChunk;
  float* partial_values = static_cast<float*>(workspace);
  uint32_t* partial_indices = reinterpret_cast<uint32_t*>(
      partial_values + static_cast<size_t>(blocks) * batch);
  // every partial the final kernel reads is written by this call's first
  // kernel, so nothing left by an earlier call needs clearing
  argmax_partial_kernel<<<dim3(blocks, batch), 256, 0, as_stream(stream)>>>(
      values, count, partial_values, partial_indices, blocks);
  argmax_final_kernel<<<batch, 256, 0, as_stream(stream)>>>(
      partial_values, partial_indices, blocks, output, RolloutAdvance{});
  return launched("argmax batch static");
}

extern "C" int32_t qllm_rollout_advance(const uint32_t* selected,
                                        uint32_t* next_token,
                                        uint32_t* draft_tokens,
                                        uint32_t capacity, uint32_t rows,
                                        uint32_t* device_positions,
                                        void* stream) {
  if (!selected || !next_token || !draft_tokens || !rows || !device_positions)
    return fail(QLLM_INVALID_ARGUMENT, "invalid rollout advance");
  rollout_advance_kernel<<<1, 64, 0, as_stream(stream)>>>(
      selected, next_token, draft_tokens, capacity, rows, device_positions);
  return launched("rollout advance");
}

extern "C" size_t qllm_topk_workspace_bytes(uint32_t count, uint32_t top_k) {
  const size_t blocks = (static_cast<size_t>(count) + kTopkChunk - 1u) / kTopkChunk;
  return blocks * top_k * (sizeof(float) + sizeof(uint32_t));
}

extern "C" int32_t qllm_topk_logits(const float* values, uint32_t count,
                                    uint32_t top_k, float* output_values,
                                    uint32_t* output_indices, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  if (!values || !count || !top_k || top_k > 1024u || top_k > count ||
      !output_values || !output_indices || !workspace ||
      workspace_bytes < qllm_topk_workspace_bytes(count, top_k))
    return fail(QLLM_INVALID_ARGUMENT, "invalid top-k logits");
  const uint32_t blocks = (count + kTopkChunk - 1u) / kTopkChunk;
  const uint64_t survivors = static_cast<uint64_t>(blocks) * top_k;
  if (survivors > static_cast<uint64_t>(kMergeThreads) * kMergePerThread)
    return fail(QLLM_INVALID_ARGUMENT,
                "top-k logits: count * top_k exceeds the merge capacity");
  float* partial_values = static_cast<float*>(workspace);
  uint32_t* partial_indices = reinterpret_cast<uint32_t*>(
      partial_values + static_cast<size_t>(blocks) * top_k);
  topk_partial_kernel<<<blocks, kTopkThreads, 0, as_stream(stream)>>>(
      values, count, top_k, partial_values, partial_indices);
  topk_merge_kernel<<<1, kMergeThreads, 0, as_stream(stream)>>>(
      partial_values, partial_indices, static_cast<uint32_t>(survivors), top_k,
      output_values, output_indices);
  return launched("top-k logits");
}

extern "C" size_t qllm_topk_batch_workspace_bytes(uint32_t count,
                                                  uint32_t top_k,
                                                  uint32_t rows) {
  if (!count || !top_k || top_k > kSelectMaxK || !rows) return 0;
  const uint32_t chunk = select_chunk(count, top_k);
  return static_cast<size_t>((count + chunk - 1u) / chunk) * rows * sizeof(float);
}

extern "C" int32_t qllm_topk_logits_batch(const float* values, uint32_t count,
                                          size_t row_stride, uint32_t top_k,
                                          uint32_t rows, float* output_values,
                                          uint32_t* output_indices,
                                          void* workspace,
                                          size_t workspace_bytes,
                                          void* stream) {
  if (!values || !count || !top_k || top_k > kSelectMaxK || top_k > count ||
      !rows || rows > 65535u || row_stride < count || !output_values ||
      !output_indices || !workspace ||
      workspace_bytes < qllm_topk_batch_workspace_bytes(count, top_k, rows))
    return fail(QLLM_INVALID_ARGUMENT, "invalid batched top-k logits");
  const uint32_t chunk = select_chunk(count, top_k);
  const uint32_t chunks = (count + chunk - 1u) / chunk;
  float* maxima = static_cast<float*>(workspace);
  chunk_max_kernel<<<dim3((chunks + 3u) / 4u, rows), 256, 0, as_stream(stream)>>>(
      values, count, row_stride, chunk, chunks, maxima);
  topk_threshold_kernel<<<rows, kSelectThreads, 0, as_stream(stream)>>>(
      values, count, row_stride, top_k, maxima, chunks, output_values,
      output_indices);
  return launched("batched top-k logits");
}

extern "C" int32_t qllm_apply_presence_penalty(float* logits,
                                               const uint8_t* emitted,
                                               uint32_t count, float penalty,
                                               void* stream) {
  if (!logits || !emitted || !count)
    return fail(QLLM_INVALID_ARGUMENT, "invalid presence penalty");
  presence_penalty_kernel<<<(count + 255u) / 256u, 256, 0, as_stream(stream)>>>(
      logits, emitted, count, penalty);
  return launched("presence penalty");
}

extern "C" int32_t qllm_apply_presence_penalty_rows(
    float* logits, size_t row_stride, const uint8_t* emitted,
    const uint32_t* drafts, uint32_t rows, uint32_t count, float penalty,
    void* stream) {
  if (!logits || !emitted || !count || !rows || row_stride < count ||
      (rows > 1u && !drafts))
    return fail(QLLM_INVALID_ARGUMENT, "invalid presence penalty rows");
  presence_penalty_rows_kernel<<<(count + 255u) / 256u, 256, 0,
                                 as_stream(stream)>>>(
      logits, row_stride, emitted, drafts, rows, count, penalty);
  return launched("presence penalty rows");
}

extern "C" int32_t qllm_mark_presence(uint8_t* emitted, const uint32_t* tokens,
                                      uint32_t token_count, uint32_t count,
                                      void* stream) {
  if (!emitted || !tokens || !token_count || token_count > 64u || !count)
    return fail(QLLM_INVALID_ARGUMENT, "invalid presence marks");
  mark_presence_kernel<<<1, 64, 0, as_stream(stream)>>>(emitted, tokens,
                                                        token_count, count);
  return launched("presence marks");
}
