// Greedy sampling on the device, inside the captured decode step: the token of every row is
// the first index of its largest logit; it is written where the next step reads its input
// token, the row's position moves on by one and the token is appended to a per-row history
// the host reads once after many steps.
#include "nq_e8.hip.h"
#include "nq_host.h"

namespace nq {

struct Best {
    float value;
    int64_t index;
};

// The larger value wins, NaN counts as larger than every number (torch.argmax does the same),
// equal values keep the lower index.
__device__ __forceinline__ bool beats(float value, int64_t index, const Best &best) {
    const bool value_nan = value != value, best_nan = best.value != best.value;
    if (value_nan || best_nan) return value_nan && (!best_nan || index < best.index);
    return value > best.value || (value == best.value && index < best.index);
}

template <typename T>
__device__ __forceinline__ float logit_as_float(T raw);
template <>
__device__ __forceinline__ float logit_as_float<float>(float raw) { return raw; }
template <>
__device__ __forceinline__ float logit_as_float<uint16_t>(uint16_t raw) { return bf16_to_f32(raw); }
template <>
__device__ __forceinline__ float logit_as_float<_Float16>(_Float16 raw) { return (float)raw; }

// Scratch of one call: per row a ticket counter and up to kSamplerSplits partial results.
constexpr int kSamplerSplits = 32;

struct SamplerScratch {
    int32_t *tickets;        // [rows], zero between calls
    int64_t *part_index;     // [rows][kSamplerSplits]
    float *part_value;       // [rows][kSamplerSplits]
};

__host__ __device__ inline size_t sampler_ticket_bytes(int rows) { return ((size_t)rows * 4 + 15) / 16 * 16; }

// grid (stretches <= kSamplerSplits, rows) x 256 lanes: every workgroup scans one stretch of a row (one
// compute unit alone reads a 256 KB row far too slowly), publishes its best and takes a ticket;
// the workgroup that draws the last ticket of a row folds the row's partial results and writes
// the outputs.  Nothing waits for anything: the ticket counter returns to zero for the next call.
template <typename T>
__global__ void __launch_bounds__(256)
greedy_sample_kernel(const T *__restrict__ logits, int64_t vocab, int64_t row_stride,
                     const uint8_t *__restrict__ active, int64_t *__restrict__ tokens,
                     int64_t *__restrict__ positions, int64_t *__restrict__ history, int history_steps,
                     int rows, int32_t *__restrict__ cursors, int vector_loads, SamplerScratch scratch) {
    constexpr int kPer = 16 / sizeof(T);
    __shared__ Best wave_best[4];
    const int split = blockIdx.x, splits = gridDim.x, row = blockIdx.y, tid = threadIdx.x;
    const T *line = logits + (int64_t)row * row_stride;
    Best best{-__builtin_inff(), vocab};
    if (vector_loads) {
        // a stretch of whole 16-byte vectors, up to four loads in flight per lane
        constexpr int kDepth = 4;
        const int64_t vectors = vocab / kPer;
        const int64_t stretch = (vectors + splits - 1) / splits;
        const int64_t begin = split * stretch, end = begin + stretch < vectors ? begin + stretch : vectors;
        for (int64_t v0 = begin + tid; v0 < end; v0 += (int64_t)kDepth * blockDim.x) {
            uint4 raw[kDepth];
#pragma unroll
            for (int d = 0; d < kDepth; d++) {
                const int64_t v = v0 + (int64_t)d * blockDim.x;
                raw[d] = reinterpret_cast<const uint4 *>(line)[v < end ? v : v0];
            }
#pragma unroll
            for (int d = 0; d < kDepth; d++) {
                const int64_t v = v0 + (int64_t)d * blockDim.x;
                if (v >= end) break;
                T item[kPer];
                __builtin_memcpy(item, &raw[d], 16);
                // within a vector only a larger value replaces the best: indices rise
                float top = logit_as_float<T>(item[0]);
                int at = 0;
#pragma unroll
                for (int j = 1; j < kPer; j++) {
                    const float value = logit_as_float<T>(item[j]);
                    const bool wins = (value > top) || (value != value && top == top);
                    top = wins ? value : top;
                    at = wins ? j : at;
                }
                if (beats(top, v * kPer + at, best)) best = Best{top, v * kPer + at};
            }
        }
        if (split == splits - 1) {
            for (int64_t i = vectors * kPer + tid; i < vocab; i += blockDim.x) {
                const float value = logit_as_float<T>(line[i]);
                if (beats(value, i, best)) best = Best{value, i};
            }
        }
    } else {
        const int64_t stretch = (vocab + splits - 1) / splits;
        const int64_t begin = split * stretch, end = begin + stretch < vocab ? begin + stretch : vocab;
        for (int64_t i = begin + tid; i < end; i += blockDim.x) {
            const float value = logit_as_float<T>(line[i]);
            if (beats(value, i, best)) best = Best{value, i};
        }
    }
#pragma unroll
    for (int offset = 32; offset >= 1; offset >>= 1) {
        const float other_value = __shfl_xor(best.value, offset, 64);
        const int64_t other_index = __shfl_xor((long long)best.index, offset, 64);
        if (beats(other_value, other_index, best)) best = Best{other_value, other_index};
    }
    if ((tid & 63) == 0) wave_best[tid >> 6] = best;
    __syncthreads();
    if (tid >= 64) return;
    // first wavefront: publish, take a ticket, and fold the row if it was the last one
    int last = 0;
    if (tid == 0) {
        for (int w = 1; w < 4; w++)
            if (beats(wave_best[w].value, wave_best[w].index, best)) best = wave_best[w];
        const int64_t slot = (int64_t)row * kSamplerSplits + split;
        __hip_atomic_store(scratch.part_value + slot, best.value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(scratch.part_index + slot, best.index, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // the release half of the ticket orders the two stores before it
        const int32_t ticket = __hip_atomic_fetch_add(scratch.tickets + row, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        last = ticket == splits - 1;
    }
    last = __shfl(last, 0, 64);
    if (!last) return;
    __threadfence();
    const int from = tid & (kSamplerSplits - 1);
    const int64_t slot = (int64_t)row * kSamplerSplits + (from < splits ? from : 0);
    best.value = __hip_atomic_load(scratch.part_value + slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    best.index = __hip_atomic_load(scratch.part_index + slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int offset = kSamplerSplits / 2; offset >= 1; offset >>= 1) {
        const float other_value = __shfl_xor(best.value, offset, 64);
        const int64_t other_index = __shfl_xor((long long)best.index, offset, 64);
        if (beats(other_value, other_index, best)) best = Best{other_value, other_index};
    }
    if (tid == 0) {
        __hip_atomic_store(scratch.tickets + row, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool live = active == nullptr || active[row] != 0;
        if (live) {
            tokens[row] = best.index;
            if (positions) positions[row] = positions[row] + 1;
            if (history) {
                const int32_t at = cursors[row];
                history[(int64_t)(at % history_steps) * rows + row] = best.index;
                cursors[row] = at + 1;
            }
        }
    }
}

}  // namespace nq

extern "C" size_t nq_greedy_sample_workspace_bytes(int rows) {
    if (rows < 1) return 0;
    return nq::sampler_ticket_bytes(rows) + (size_t)rows * nq::kSamplerSplits * (sizeof(int64_t) + sizeof(float));
}

extern "C" int nq_greedy_sample(const void *logits_dev, int logits_dtype, int rows, int64_t vocab, int64_t row_stride,
                                const uint8_t *active_mask_dev, int64_t *tokens_dev, int64_t *positions_dev,
                                int64_t *history_dev, int history_steps, int32_t *cursors_dev, void *workspace_dev,
                                size_t workspace_bytes, void *stream) {
    NQ_REQUIRE(rows >= 1 && rows <= 65535 && vocab >= 1 && row_stride >= vocab, NQ_ERR_SHAPE,
               "nq_greedy_sample: rows (at most 65535) and vocab must be positive and row_stride at least vocab");
    NQ_REQUIRE(logits_dev && tokens_dev, NQ_ERR_ARGUMENT, "nq_greedy_sample: null pointer");
    NQ_REQUIRE(!history_dev || (cursors_dev && history_steps >= 1), NQ_ERR_ARGUMENT,
               "nq_greedy_sample: a history needs its row cursors and a positive number of steps");
    const size_t need = nq_greedy_sample_workspace_bytes(rows);
    NQ_REQUIRE(workspace_dev && workspace_bytes >= need && nq::aligned(workspace_dev, 16), NQ_ERR_WORKSPACE,
               "nq_greedy_sample: needs a 16-byte aligned %zu-byte workspace, got %zu", need, workspace_bytes);
    nq::SamplerScratch scratch;
    scratch.tickets = reinterpret_cast<int32_t *>(workspace_dev);
    scratch.part_index = reinterpret_cast<int64_t *>(reinterpret_cast<char *>(workspace_dev) + nq::sampler_ticket_bytes(rows));
    scratch.part_value = reinterpret_cast<float *>(scratch.part_index + (size_t)rows * nq::kSamplerSplits);
    // about 128 workgroups in all: every one pays a release of its cache at the ticket, which is
    // what a launch of many rows spends its time on (16 rows: 12.8 us with 8 stretches, 16.7 with 32)
    int splits = 128 / rows;
    splits = splits < 8 ? 8 : (splits > nq::kSamplerSplits ? nq::kSamplerSplits : splits);
    const hipStream_t s = (hipStream_t)stream;
#define NQ_LAUNCH_SAMPLER(T)                                                                                   \
    do {                                                                                                       \
        const int vector_loads = nq::aligned(logits_dev, 16) && (row_stride * sizeof(T)) % 16 == 0;            \
        hipLaunchKernelGGL(nq::greedy_sample_kernel<T>, dim3((unsigned)splits, (unsigned)rows), dim3(256), 0, s,   \
                           reinterpret_cast<const T *>(logits_dev), vocab, row_stride, active_mask_dev,        \
                           tokens_dev, positions_dev, history_dev, history_steps, rows, cursors_dev,           \
                           vector_loads, scratch);                                                             \
    } while (0)
    if (logits_dtype == NQ_BF16) NQ_LAUNCH_SAMPLER(uint16_t);
    else if (logits_dtype == NQ_F16) NQ_LAUNCH_SAMPLER(_Float16);
    else if (logits_dtype == NQ_F32) NQ_LAUNCH_SAMPLER(float);
    else return nq::fail(NQ_ERR_ARGUMENT, "nq_greedy_sample: unknown dtype tag %d", logits_dtype);
#undef NQ_LAUNCH_SAMPLER
    return nq::check_launch("nq_greedy_sample");
}
