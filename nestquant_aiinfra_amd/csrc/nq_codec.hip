// E8 codec kernels: nearest point, row quantiser with multi-beta selection (NQA4 / NQKV4
// encoder) and its inverse.  Reference: nestquant/core/quantizer.py:214-301, 39-51;
// nestquant/runtime/nqkv_page.py:97-185, 332-372, 446-456, 22-95; nestquant/runtime/cuda_e8.cu:8-59.
#define NQ_PHASE_STAMP_ARRAY g_phase_stamps
#include "nq_rowlanes.hip.h"
#include "nq_host.h"

#include <math.h>
#include <type_traits>

#ifdef NQ_PHASE_STAMPS
// Measuring builds only: the stamps the last encoder launch left (wall clock, 10 ns units).
extern "C" int nq_debug_phase_stamps(unsigned long long *out16) {
    if (hipDeviceSynchronize() != hipSuccess) return NQ_ERR_LAUNCH;
    return hipMemcpyFromSymbol(out16, HIP_SYMBOL(nq::g_phase_stamps), 16 * sizeof(unsigned long long)) == hipSuccess
               ? NQ_OK : NQ_ERR_LAUNCH;
}
#endif

namespace nq {

// ---------------------------------------------------------------------------------------
// e8_nearest: one lane per vector, two 128-bit loads and stores per lane.
// ---------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) e8_nearest_kernel(const float4 *x, float4 *out, int64_t count) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const float4 lo = x[2 * i], hi = x[2 * i + 1];
    const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    float r[8];
    e8_nearest(v, r);
    out[2 * i] = make_float4(r[0], r[1], r[2], r[3]);
    out[2 * i + 1] = make_float4(r[4], r[5], r[6], r[7]);
}

// ---------------------------------------------------------------------------------------
// Row quantiser.
//
// A workgroup owns `rows_per_wg` consecutive rows, staged once in LDS as float32.
//   phase 1  coalesced load (+ promotion) of the rows into LDS;
//   phase 2  row norms in the reference's order: eight interleaved fused-multiply-add
//            chains (element i feeds chain i % 8), chains added 0..7, sqrt; eight lanes
//            per row run the chains, the rest of the workgroup waits;
//   phase 3  one lane per (block, beta) pair: a quad of lanes evaluates the four betas of
//            one block, the per-block argmin (first minimum) is a two-step quad exchange,
//            the winning lane stores the 32-bit code word, and the 2-bit ids of four
//            neighbouring blocks are merged into one byte with two more exchanges.
// ---------------------------------------------------------------------------------------
// 16-byte global load of consecutive elements, promoted to float32 and stored to LDS
struct half_bits { uint16_t v; };
template <typename T> struct RowLoader;
template <> struct RowLoader<float> {
    static constexpr int kPerVector = 4;
    static __device__ __forceinline__ void load(const float *x, int64_t v, float *dst) {
        *reinterpret_cast<float4 *>(dst) = reinterpret_cast<const float4 *>(x)[v];
    }
    static __device__ __forceinline__ float scalar(const float *x, int64_t i) { return x[i]; }
};
template <> struct RowLoader<uint16_t> {
    static constexpr int kPerVector = 8;
    static __device__ __forceinline__ void load(const uint16_t *x, int64_t v, float *dst) {
        const uint4 raw = reinterpret_cast<const uint4 *>(x)[v];
        reinterpret_cast<float4 *>(dst)[0] = make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                                                         __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u));
        reinterpret_cast<float4 *>(dst)[1] = make_float4(__uint_as_float(raw.z << 16), __uint_as_float(raw.z & 0xffff0000u),
                                                         __uint_as_float(raw.w << 16), __uint_as_float(raw.w & 0xffff0000u));
    }
    static __device__ __forceinline__ float scalar(const uint16_t *x, int64_t i) { return bf16_to_f32(x[i]); }
};
template <> struct RowLoader<half_bits> {
    static constexpr int kPerVector = 8;
    static __device__ __forceinline__ void load(const half_bits *x, int64_t v, float *dst) {
        const uint4 raw = reinterpret_cast<const uint4 *>(x)[v];
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            dst[2 * j] = f16_to_f32((uint16_t)(w[j] & 0xffffu));
            dst[2 * j + 1] = f16_to_f32((uint16_t)(w[j] >> 16));
        }
    }
    static __device__ __forceinline__ float scalar(const half_bits *x, int64_t i) { return f16_to_f32(x[i].v); }
};


// Stages rows [first, first + rows_per_wg * n) into `staged` through the element-wise stage
// of `pro` (see InputPrologue).  Every global operand of a 16-byte vector is requested before
// any is used, so the kernel pays one memory round trip, not one per operand.  `weights`
// (n floats of LDS) holds the norm weight in mode 1.  Ends with a barrier.
template <int kPrologue>
__device__ __forceinline__ void stage_with_prologue(const uint16_t *__restrict__ x, const InputPrologue &pro,
                                                    float *staged, float *row_scale, float *weights,
                                                    int64_t first, int64_t limit, int rows_per_wg, int n,
                                                    bool writes_outputs) {
    __shared__ float row_sums[64];
    const int tid = threadIdx.x;
    const int row_vectors = n >> 3, vectors = rows_per_wg * row_vectors;
    const uint4 zero = make_uint4(0, 0, 0, 0);
    if (kPrologue == 3) {
        // one lane per eight output dimensions of one head: out = sum_c acc_c w_c / sum_c sum_c w_c with
        // w_c = exp(max_c - max).  Online over batches of four chunks (the batch of lane_prologue, so
        // that both encoders round alike) whose maxima, sums and numerators are all requested before
        // the first is used (one memory latency per batch, not per chunk); chunks without tokens carry
        // no numerator (their entry is read, never used) and weigh nothing.
        constexpr int kBatch = 4;
        const float kNone = -__builtin_inff();
        for (int v = tid; v < vectors; v += blockDim.x) {
            const int64_t g = first + (int64_t)v * 8;
            float y[8];
#pragma unroll
            for (int j = 0; j < 8; j++) y[j] = 0.0f;
            if (g < limit) {
                const int64_t head = (g / n) * pro.heads + (g % n) / 64;
                const float *m = pro.part_max + head * pro.parts, *sum = pro.part_sum + head * pro.parts;
                const float *acc = pro.part_acc + head * pro.parts * 64 + (g % 64);
                float top = kNone, denom = 0.0f;
                for (int c0 = 0; c0 < pro.parts; c0 += kBatch) {
                    float mc[kBatch], sc[kBatch];
                    float4 lo[kBatch], hi[kBatch];
#pragma unroll
                    for (int j = 0; j < kBatch; j++) {
                        const int c = min(c0 + j, pro.parts - 1);
                        mc[j] = m[c];
                        sc[j] = sum[c];
                        lo[j] = *reinterpret_cast<const float4 *>(acc + (int64_t)c * 64);
                        hi[j] = *reinterpret_cast<const float4 *>(acc + (int64_t)c * 64 + 4);
                    }
                    float batch_top = kNone;
#pragma unroll
                    for (int j = 0; j < kBatch; j++) {
                        if (c0 + j >= pro.parts) sc[j] = 0.0f;
                        batch_top = fmaxf(batch_top, mc[j]);
                    }
                    const float next_top = fmaxf(top, batch_top);
                    if (next_top > kNone) {
                        const float keep = top > kNone ? __expf(top - next_top) : 0.0f;
                        denom = denom * keep;
#pragma unroll
                        for (int i = 0; i < 8; i++) y[i] = y[i] * keep;
#pragma unroll
                        for (int j = 0; j < kBatch; j++) {
                            const float w = sc[j] > 0.0f ? __expf(mc[j] - next_top) : 0.0f;
                            denom = denom + sc[j] * w;
                            const bool used = w > 0.0f;
                            y[0] += used ? lo[j].x * w : 0.0f; y[1] += used ? lo[j].y * w : 0.0f;
                            y[2] += used ? lo[j].z * w : 0.0f; y[3] += used ? lo[j].w * w : 0.0f;
                            y[4] += used ? hi[j].x * w : 0.0f; y[5] += used ? hi[j].y * w : 0.0f;
                            y[6] += used ? hi[j].z * w : 0.0f; y[7] += used ? hi[j].w * w : 0.0f;
                        }
                        top = next_top;
                    }
                }
#pragma unroll
                for (int j = 0; j < 8; j += 2) {
                    y[j] = denom > 0.0f ? y[j] / denom : 0.0f;               // inactive or empty rows give zeros
                    y[j + 1] = denom > 0.0f ? y[j + 1] / denom : 0.0f;
                    round_pair<1>(y[j], y[j + 1]);
                }
                if (writes_outputs && pro.normed_out)
                    reinterpret_cast<uint4 *>(pro.normed_out)[g >> 3] = pack_bf16x8_exact(y);
            }
            *reinterpret_cast<float4 *>(staged + v * 8) = make_float4(y[0], y[1], y[2], y[3]);
            *reinterpret_cast<float4 *>(staged + v * 8 + 4) = make_float4(y[4], y[5], y[6], y[7]);
        }
        __syncthreads();
        return;
    }
    for (int v = tid; v < vectors; v += blockDim.x) {
        const int64_t g = first + (int64_t)v * 8;
        const bool live = g < limit;
        const uint4 raw_x = live ? reinterpret_cast<const uint4 *>(x)[g >> 3] : zero;
        uint4 raw_a = zero, raw_w = zero;
        if (kPrologue == 1) {
            if (live && pro.residual) raw_a = reinterpret_cast<const uint4 *>(pro.residual)[g >> 3];
            if (v < row_vectors) raw_w = reinterpret_cast<const uint4 *>(pro.weight)[v];
        } else {
            if (live) raw_a = reinterpret_cast<const uint4 *>(pro.gate)[g >> 3];
        }
        float h[8], a[8];
        unpack_bf16x8(raw_x, h);
        unpack_bf16x8(raw_a, a);
        if (kPrologue == 1) {
            if (pro.residual) {
#pragma unroll
                for (int j = 0; j < 8; j += 2) {
                    h[j] = h[j] + a[j];
                    h[j + 1] = h[j + 1] + a[j + 1];
                    round_pair<1>(h[j], h[j + 1]);
                }
            }
            if (live && writes_outputs && pro.residual_out)
                reinterpret_cast<uint4 *>(pro.residual_out)[g >> 3] = pack_bf16x8_exact(h);
            if (v < row_vectors) {
                float w[8];
                unpack_bf16x8(raw_w, w);
#pragma unroll
                for (int j = 0; j < 8; j++) weights[v * 8 + j] = w[j];
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
                float s0 = a[j] / (1.0f + __expf(-a[j])), s1 = a[j + 1] / (1.0f + __expf(-a[j + 1]));
                round_pair<1>(s0, s1);
                h[j] = s0 * h[j];
                h[j + 1] = s1 * h[j + 1];
                round_pair<1>(h[j], h[j + 1]);
            }
            if (live && writes_outputs && pro.normed_out)
                reinterpret_cast<uint4 *>(pro.normed_out)[g >> 3] = pack_bf16x8_exact(h);
        }
        *reinterpret_cast<float4 *>(staged + v * 8) = make_float4(h[0], h[1], h[2], h[3]);
        *reinterpret_cast<float4 *>(staged + v * 8 + 4) = make_float4(h[4], h[5], h[6], h[7]);
    }
    __syncthreads();
    if (kPrologue != 1) return;

    // LlamaRMSNorm: bf16(weight * bf16(h * rsqrt(mean(h^2) + eps))), one row at a time
    const int rows16 = (int)(blockDim.x >> 4);
    for (int r = 0; r < rows_per_wg; r++) {
        float sum = 0.0f;
        for (int i = tid; i < n; i += blockDim.x) sum = __builtin_fmaf(staged[r * n + i], staged[r * n + i], sum);
        sum = sum + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, sum), 0xB1, 0xF, 0xF, true));
        sum = sum + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, sum), 0x4E, 0xF, 0xF, true));
        sum = sum + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, sum), 0x141, 0xF, 0xF, true));
        sum = sum + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, sum), 0x140, 0xF, 0xF, true));
        if ((tid & 15) == 0) row_sums[tid >> 4] = sum;
        __syncthreads();
        float total = 0.0f;
        for (int w = 0; w < rows16; w++) total = total + row_sums[w];
        if (tid == 0) row_scale[r] = 1.0f / __builtin_sqrtf(total / (float)n + pro.eps);
        __syncthreads();
    }
    for (int v = tid; v < vectors; v += blockDim.x) {
        const int64_t g = first + (int64_t)v * 8;
        const int r = rows_per_wg == 1 ? 0 : v / row_vectors;
        const int column = (v - r * row_vectors) * 8;
        const float scale = row_scale[r];
        float y[8];
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            y[j] = staged[v * 8 + j] * scale;
            y[j + 1] = staged[v * 8 + j + 1] * scale;
            round_pair<1>(y[j], y[j + 1]);
            y[j] = weights[column + j] * y[j];
            y[j + 1] = weights[column + j + 1] * y[j + 1];
            round_pair<1>(y[j], y[j + 1]);
        }
        *reinterpret_cast<float4 *>(staged + v * 8) = make_float4(y[0], y[1], y[2], y[3]);
        *reinterpret_cast<float4 *>(staged + v * 8 + 4) = make_float4(y[4], y[5], y[6], y[7]);
        if (g < limit && writes_outputs && pro.normed_out)
            reinterpret_cast<uint4 *>(pro.normed_out)[g >> 3] = pack_bf16x8_exact(y);
    }
    __syncthreads();
}

// Where the encoder kernels put a block's results: the packed streams, and optionally the
// BF16 decode of the stored code as the linear kernels consume it.
struct RowSink {
    uint32_t *codes; uint8_t *beta_ids; uint4 *decoded; const float *row_norm;
    int64_t row0, rows; int blocks_per_row; float sqrt_n;
    __device__ __forceinline__ bool wants(int r) const { return row0 + r < rows; }
    __device__ __forceinline__ void code(int r, int b, uint32_t word, const float (&recon)[8], float beta) const {
        const int64_t gblock = (row0 + r) * blocks_per_row + b;
        codes[gblock] = word;
        if (decoded) {
            // the BF16 decode of the stored code, as the linear kernels consume it
            const float back = row_norm[r] / sqrt_n;
            uint32_t h[8];
#pragma unroll
            for (int j = 0; j < 8; j++) h[j] = f32_to_bf16((recon[j] * beta) * back);
            decoded[gblock] = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16),
                                         h[4] | (h[5] << 16), h[6] | (h[7] << 16));
        }
    }
    __device__ __forceinline__ void beta_byte(int r, int b, uint32_t byte) const {
        beta_ids[((row0 + r) * blocks_per_row + b) >> 2] = (uint8_t)byte;
    }
    __device__ __forceinline__ uint32_t counter(int r, int b) const {
        return (uint32_t)((row0 + r) * blocks_per_row + b) * 8u;
    }
};

struct SharedBetas {
    const float *table;
    __device__ __forceinline__ const float *operator()(int) const { return table; }
};

template <typename T, bool kDithered, int kPrologue>
__global__ void __launch_bounds__(1024)
quantize_rows_kernel(const T *__restrict__ x, int64_t rows, int n, float q, float inv_q,
                     const float *__restrict__ betas, int beta_count, float sqrt_n,
                     uint32_t seed_plus_offset, uint32_t *__restrict__ codes,
                     uint8_t *__restrict__ beta_ids, float *__restrict__ norms,
                     uint4 *__restrict__ decoded, int rows_per_wg, int slices, int vector_loads,
                     int hadamard_stage_dtype, InputPrologue pro) {
    extern __shared__ float lds[];
    float *row_scale = lds + (size_t)rows_per_wg * n;
    float *row_norm = row_scale + rows_per_wg;
    const int tid = threadIdx.x;
    // With few rows a single row is spread over `slices` workgroups (rows_per_wg == 1): each
    // stages the whole row and repeats the norm, then encodes its own range of blocks.
    const int slice = blockIdx.x % slices;
    const int64_t row0 = (int64_t)(blockIdx.x / slices) * rows_per_wg;
    const int blocks_per_row = n >> 3;

    // phase 1
    NQ_STAMP(0);
    const int64_t first = row0 * n, limit = rows * (int64_t)n;
    if (kPrologue != 0) {
        stage_with_prologue<kPrologue>(reinterpret_cast<const uint16_t *>(x), pro, lds, row_scale, row_norm + rows_per_wg,
                                       first, limit, rows_per_wg, n, slice == 0);
        if (codes == nullptr) return;                      // element-wise stage only
    } else if (vector_loads) {
        // n is a multiple of 32, so every row is a whole number of 16-byte vectors
        constexpr int kPer = RowLoader<T>::kPerVector;
        const int vectors = rows_per_wg * n / kPer;
#pragma unroll 4
        for (int v = tid; v < vectors; v += blockDim.x) {
            const int64_t g = first + (int64_t)v * kPer;
            if (g < limit) {
                RowLoader<T>::load(x, g / kPer, lds + v * kPer);
            } else {
#pragma unroll
                for (int j = 0; j < kPer; j++) lds[v * kPer + j] = 0.0f;
            }
        }
    } else {
        for (int idx = tid; idx < rows_per_wg * n; idx += blockDim.x) {
            const int64_t g = first + idx;
            lds[idx] = g < limit ? RowLoader<T>::scalar(x, g) : 0.0f;
        }
    }
    __syncthreads();
    NQ_STAMP(1);

    // optional input rotation, in the arithmetic of the caller's tensor dtype
    if (hadamard_stage_dtype >= 0) staged_hadamard(lds, rows_per_wg, n, hadamard_stage_dtype);
    NQ_STAMP(2);

    // phase 2
    staged_row_norms(lds, rows_per_wg, n, sqrt_n, row_scale, row_norm);
    if (slice == 0 && tid < rows_per_wg && row0 + tid < rows) norms[row0 + tid] = row_norm[tid];
    NQ_STAMP(3);

    // phase 3
    const int slice_pairs = rows_per_wg * blocks_per_row * 4 / slices;     // a multiple of 16
    const RowSink sink{codes, beta_ids, decoded, row_norm, row0, rows, blocks_per_row, sqrt_n};
    const SharedBetas betas_of{betas};
    quantize_staged_pairs<kDithered>(lds, row_scale, n, q, inv_q, betas_of, beta_count, seed_plus_offset,
                                     slice_pairs * slice, slice_pairs * (slice + 1), sink);
    NQ_STAMP(4);
}


// Many rows: 256 lanes per workgroup, `rows_per_wg` rows of together at least 2048 values, one
// lane per block in the encode phase (several such workgroups share a compute unit and fill
// each other's serial stretches: the norm chain, the barriers of the rotation).
template <typename T, int kPrologue>
__global__ void __launch_bounds__(256)
quantize_rows_bulk_kernel(const T *__restrict__ x, int64_t rows, int n, float q, float inv_q,
                          const float *__restrict__ betas, int beta_count, float sqrt_n,
                          uint32_t *__restrict__ codes, uint8_t *__restrict__ beta_ids,
                          float *__restrict__ norms, uint4 *__restrict__ decoded, int rows_per_wg,
                          int vector_loads, int hadamard_stage_dtype, InputPrologue pro) {
    extern __shared__ float lds[];
    float *row_scale = lds + (size_t)rows_per_wg * n;
    float *row_norm = row_scale + rows_per_wg;
    const int tid = threadIdx.x;
    const int64_t row0 = (int64_t)blockIdx.x * rows_per_wg;
    const int64_t first = row0 * n, limit = rows * (int64_t)n;
    if (kPrologue != 0) {
        stage_with_prologue<kPrologue>(reinterpret_cast<const uint16_t *>(x), pro, lds, row_scale, row_norm + rows_per_wg,
                                       first, limit, rows_per_wg, n, true);
        if (codes == nullptr) return;                      // element-wise stage only
    } else if (vector_loads) {
        constexpr int kPer = RowLoader<T>::kPerVector;
        const int vectors = rows_per_wg * n / kPer;
#pragma unroll 4
        for (int v = tid; v < vectors; v += blockDim.x) {
            const int64_t g = first + (int64_t)v * kPer;
            if (g < limit) {
                RowLoader<T>::load(x, g / kPer, lds + v * kPer);
            } else {
#pragma unroll
                for (int j = 0; j < kPer; j++) lds[v * kPer + j] = 0.0f;
            }
        }
    } else {
        for (int idx = tid; idx < rows_per_wg * n; idx += blockDim.x) {
            const int64_t g = first + idx;
            lds[idx] = g < limit ? RowLoader<T>::scalar(x, g) : 0.0f;
        }
    }
    if (kPrologue == 0) __syncthreads();
    if (hadamard_stage_dtype >= 0) staged_hadamard(lds, rows_per_wg, n, hadamard_stage_dtype);
    staged_row_norms(lds, rows_per_wg, n, sqrt_n, row_scale, row_norm);
    if (tid < rows_per_wg && row0 + tid < rows) norms[row0 + tid] = row_norm[tid];
    const RowSink sink{codes, beta_ids, decoded, row_norm, row0, rows, n >> 3, sqrt_n};
    quantize_staged_blocks(lds, row_scale, n, q, inv_q, SharedBetas{betas}, beta_count, 0,
                           rows_per_wg * (n >> 3), sink);
}

// ---------------------------------------------------------------------------------------
// Dequantise rows: one lane per block.
// ---------------------------------------------------------------------------------------
template <bool kDithered>
__global__ void __launch_bounds__(256)
dequantize_rows_kernel(const uint32_t *__restrict__ codes, const uint8_t *__restrict__ beta_ids,
                       const float *__restrict__ norms, const float *__restrict__ betas,
                       int64_t blocks, int blocks_per_row, float q, float sqrt_n,
                       uint32_t seed_plus_offset, void *__restrict__ out, int out_dtype) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= blocks) return;
    const int64_t row = g / blocks_per_row;
    float v[8];
    decode_codeword<kDithered>(codes[g], q, seed_plus_offset + (uint32_t)g * 8u, v);
    const float beta = betas[(beta_ids[g >> 2] >> (2 * (g & 3))) & 3];
    const float scale = norms[row] / sqrt_n;            // IEEE division (tensor / python float)
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = (v[j] * beta) * scale;
    if (out_dtype == NQ_F32) {
        float4 *o = reinterpret_cast<float4 *>(out) + 2 * g;
        o[0] = make_float4(v[0], v[1], v[2], v[3]);
        o[1] = make_float4(v[4], v[5], v[6], v[7]);
    } else if (out_dtype == NQ_BF16) {
        uint4 w;
        w.x = f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
        w.y = f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
        w.z = f32_to_bf16(v[4]) | ((uint32_t)f32_to_bf16(v[5]) << 16);
        w.w = f32_to_bf16(v[6]) | ((uint32_t)f32_to_bf16(v[7]) << 16);
        reinterpret_cast<uint4 *>(out)[g] = w;
    } else {
        _Float16 *o = reinterpret_cast<_Float16 *>(out) + 8 * g;
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] = (_Float16)v[j];
    }
}

// ---------------------------------------------------------------------------------------
// Stand-alone Hadamard rotation of rows (post-RoPE queries and keys, prefill inputs).
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(1024)
hadamard_rows_kernel(const T *__restrict__ x, int64_t rows, int n, int rows_per_wg, int stage_dtype,
                     void *__restrict__ out, int out_dtype, int vector_io) {
    extern __shared__ float lds[];
    const int64_t row0 = (int64_t)blockIdx.x * rows_per_wg;
    const int64_t first = row0 * n, limit = rows * (int64_t)n;
    const int staged = rows_per_wg * n;
    if (vector_io) {
        // rows are whole numbers of 16-byte vectors, input and output 16-byte aligned
        constexpr int kPer = RowLoader<T>::kPerVector;
        for (int v = threadIdx.x; v < staged / kPer; v += blockDim.x) {
            const int64_t g = first + (int64_t)v * kPer;
            if (g < limit) {
                RowLoader<T>::load(x, g / kPer, lds + v * kPer);
            } else {
#pragma unroll
                for (int j = 0; j < kPer; j++) lds[v * kPer + j] = 0.0f;
            }
        }
    } else {
        for (int idx = threadIdx.x; idx < staged; idx += blockDim.x)
            lds[idx] = first + idx < limit ? RowLoader<T>::scalar(x, first + idx) : 0.0f;
    }
    __syncthreads();
    staged_hadamard(lds, rows_per_wg, n, stage_dtype);
    if (vector_io && out_dtype != NQ_F16) {
        for (int v = threadIdx.x; v < staged / 8; v += blockDim.x) {
            const int64_t g = first + (int64_t)v * 8;
            if (g >= limit) continue;
            const float4 lo = *reinterpret_cast<const float4 *>(lds + v * 8), hi = *reinterpret_cast<const float4 *>(lds + v * 8 + 4);
            if (out_dtype == NQ_BF16) {
                const float y[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                reinterpret_cast<uint4 *>(out)[g >> 3] = pack_bf16x8(y);
            } else {
                reinterpret_cast<float4 *>(out)[g >> 2] = lo;
                reinterpret_cast<float4 *>(out)[(g >> 2) + 1] = hi;
            }
        }
        return;
    }
    for (int idx = threadIdx.x; idx < staged; idx += blockDim.x) {
        const int64_t g = first + idx;
        if (g >= limit) continue;
        if (out_dtype == NQ_BF16) reinterpret_cast<uint16_t *>(out)[g] = f32_to_bf16(lds[idx]);
        else if (out_dtype == NQ_F16) reinterpret_cast<_Float16 *>(out)[g] = (_Float16)lds[idx];
        else reinterpret_cast<float *>(out)[g] = lds[idx];
    }
}

// Rotary position embedding and / or Hadamard rotation of BF16 head vectors [rows, heads, D]
// (prefill queries and keys): eight values per lane, D / 8 neighbouring lanes per vector, no
// LDS.  The embedding is (x * cos) + (rotate_half(x) * sin) in BF16 tensor arithmetic (every
// product and the sum rounded to BF16); the rotation runs float32 butterflies and rounds once.
// A second tensor of the same rows with a head count of its own (the keys beside the queries) may
// follow the first in the same launch: its chunks are numbered after the first tensor's.
template <int D>
__global__ void __launch_bounds__(256)
rope_hadamard_kernel(const uint16_t *__restrict__ x, int64_t vectors, int heads,
                     const uint16_t *__restrict__ x2, int64_t vectors2, int heads2,
                     const uint16_t *__restrict__ rope_cos, const uint16_t *__restrict__ rope_sin,
                     int rotate, uint16_t *__restrict__ out, uint16_t *__restrict__ out2) {
    constexpr int kLanes = D / 8;
    int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;              // one 8-value chunk each
    if (g >= (vectors + vectors2) * kLanes) return;                           // whole vectors leave together
    if (g >= vectors * kLanes) {                                              // (a vector never straddles the two)
        g -= vectors * kLanes;
        x = x2; out = out2; heads = heads2;
    }
    const int lane = threadIdx.x & 63, part = (int)(g % kLanes);
    float v[8];
    unpack_bf16x8(reinterpret_cast<const uint4 *>(x)[g], v);
    if (rope_cos) {
        const int64_t at = (g / kLanes / heads) * kLanes + part;
        float c[8], s[8];
        unpack_bf16x8(reinterpret_cast<const uint4 *>(rope_cos)[at], c);
        unpack_bf16x8(reinterpret_cast<const uint4 *>(rope_sin)[at], s);
        const bool upper = part >= kLanes / 2;
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            float o0 = lane_xor<kLanes / 2>(v[j]), o1 = lane_xor<kLanes / 2>(v[j + 1]);
            float a0 = v[j] * c[j], a1 = v[j + 1] * c[j + 1];
            round_pair<1>(a0, a1);
            float b0 = o0 * s[j], b1 = o1 * s[j + 1];
            round_pair<1>(b0, b1);
            v[j] = upper ? a0 + b0 : a0 - b0;
            v[j + 1] = upper ? a1 + b1 : a1 - b1;
            round_pair<1>(v[j], v[j + 1]);
        }
    }
    if (rotate) {
#pragma unroll
        for (int s = 0; s < 3; s++) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                if (j & (1 << s)) continue;
                const float left = v[j], right = v[j + (1 << s)];
                v[j] = left + right;
                v[j + (1 << s)] = left - right;
            }
        }
        lane_stage<1, 0>(v, lane);
        lane_stage<2, 0>(v, lane);
        lane_stage<4, 0>(v, lane);
        if (kLanes > 8) lane_stage<8, 0>(v, lane);
        const float inv = 1.0f / __builtin_sqrtf((float)D);
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = v[j] * inv;
    }
    reinterpret_cast<uint4 *>(out)[g] = pack_bf16x8(v);
}

}  // namespace nq

extern "C" int nq_hadamard(const void *x_dev, int x_dtype, int64_t rows, int64_t n, int stage_dtype,
                           void *out_dev, int out_dtype, void *stream) {
    NQ_REQUIRE(rows >= 1 && n >= 2 && (n & (n - 1)) == 0 && n <= 32768, NQ_ERR_SHAPE,
               "nq_hadamard: feature count %lld must be a power of two in [2, 32768]", (long long)n);
    NQ_REQUIRE(x_dev && out_dev, NQ_ERR_ARGUMENT, "nq_hadamard: null pointer");
    for (int tag : {x_dtype, stage_dtype, out_dtype})
        NQ_REQUIRE(tag == NQ_F32 || tag == NQ_BF16 || tag == NQ_F16, NQ_ERR_ARGUMENT,
                   "nq_hadamard: unknown dtype tag %d", tag);
    int rows_per_wg = (int)(2048 / n);
    if (rows_per_wg < 1) rows_per_wg = 1;
    if (rows_per_wg > rows) rows_per_wg = (int)rows;
    const size_t lds_bytes = (size_t)rows_per_wg * n * sizeof(float);
    const int64_t grid = (rows + rows_per_wg - 1) / rows_per_wg;
    NQ_REQUIRE(grid <= 0x7fffffff, NQ_ERR_SHAPE, "nq_hadamard: too many rows");
    // eight values per lane: long rows get up to 1024 lanes
    int threads = (int)((int64_t)rows_per_wg * n / 8);
    threads = threads < 64 ? 64 : (threads > 1024 ? 1024 : (threads + 63) / 64 * 64);
    const int vector_io = n % 8 == 0 && nq::aligned(x_dev, 16) && nq::aligned(out_dev, 16);
    hipStream_t s = (hipStream_t)stream;
#define NQ_LAUNCH_HADAMARD(T)                                                                          \
    do {                                                                                               \
        auto kernel = nq::hadamard_rows_kernel<T>;                                                     \
        if (lds_bytes > 48 * 1024)                                                                     \
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),                          \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);     \
        hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(threads), lds_bytes, s,                  \
                           reinterpret_cast<const T *>(x_dev), rows, (int)n, rows_per_wg, stage_dtype, \
                           out_dev, out_dtype, vector_io);                                             \
    } while (0)
    if (x_dtype == NQ_F32) NQ_LAUNCH_HADAMARD(float);
    else if (x_dtype == NQ_BF16) NQ_LAUNCH_HADAMARD(uint16_t);
    else NQ_LAUNCH_HADAMARD(nq::half_bits);
#undef NQ_LAUNCH_HADAMARD
    return nq::check_launch("nq_hadamard");
}

namespace {

int launch_rope_hadamard(const char *entry, const void *x, int heads, void *out, const void *x2, int heads2, void *out2,
                         int64_t rows, int head_dim, const void *rope_cos, const void *rope_sin, int hadamard,
                         hipStream_t s) {
    NQ_REQUIRE(rows >= 1 && heads >= 1 && heads2 >= 0, NQ_ERR_SHAPE, "%s: rows and heads must be positive", entry);
    NQ_REQUIRE(head_dim == 64 || head_dim == 128, NQ_ERR_SHAPE, "%s: head_dim %d is not 64 or 128", entry, head_dim);
    NQ_REQUIRE(x && out && (heads2 == 0 || (x2 && out2)), NQ_ERR_ARGUMENT, "%s: null pointer", entry);
    NQ_REQUIRE((rope_cos == nullptr) == (rope_sin == nullptr), NQ_ERR_ARGUMENT, "%s: rotary tables come as a pair", entry);
    NQ_REQUIRE(nq::aligned(x, 16) && nq::aligned(out, 16) && nq::aligned(x2, 16) && nq::aligned(out2, 16) &&
                   nq::aligned(rope_cos, 16) && nq::aligned(rope_sin, 16),
               NQ_ERR_ARGUMENT, "%s: pointers must be 16-byte aligned", entry);
    const int64_t vectors = rows * heads, vectors2 = rows * heads2, chunks = (vectors + vectors2) * (head_dim / 8);
    const int64_t grid = (chunks + 255) / 256;
    NQ_REQUIRE(grid <= 0x7fffffff, NQ_ERR_SHAPE, "%s: too many vectors", entry);
    // the second tensor's chunks start at a multiple of the 8 or 16 lanes of a vector, so the lanes that
    // exchange values still sit side by side in one wavefront
    auto kernel = head_dim == 64 ? nq::rope_hadamard_kernel<64> : nq::rope_hadamard_kernel<128>;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(256), 0, s, reinterpret_cast<const uint16_t *>(x), vectors, heads,
                       reinterpret_cast<const uint16_t *>(x2), vectors2, heads2,
                       reinterpret_cast<const uint16_t *>(rope_cos), reinterpret_cast<const uint16_t *>(rope_sin), hadamard,
                       reinterpret_cast<uint16_t *>(out), reinterpret_cast<uint16_t *>(out2));
    return nq::check_launch(entry);
}

}  // namespace

extern "C" int nq_rope_hadamard(const void *x_dev, int64_t rows, int heads, int head_dim, const void *rope_cos_dev,
                                const void *rope_sin_dev, int hadamard, void *out_dev, void *stream) {
    return launch_rope_hadamard("nq_rope_hadamard", x_dev, heads, out_dev, nullptr, 0, nullptr, rows, head_dim,
                                rope_cos_dev, rope_sin_dev, hadamard, (hipStream_t)stream);
}

extern "C" int nq_rope_hadamard_pair(const void *query_dev, int query_heads, void *query_out_dev, const void *key_dev,
                                     int key_heads, void *key_out_dev, int64_t rows, int head_dim,
                                     const void *rope_cos_dev, const void *rope_sin_dev, int hadamard, void *stream) {
    NQ_REQUIRE(key_heads >= 1, NQ_ERR_SHAPE, "nq_rope_hadamard_pair: rows and heads must be positive");
    return launch_rope_hadamard("nq_rope_hadamard_pair", query_dev, query_heads, query_out_dev, key_dev, key_heads,
                                key_out_dev, rows, head_dim, rope_cos_dev, rope_sin_dev, hadamard, (hipStream_t)stream);
}

extern "C" int nq_e8_nearest(const float *x_dev, float *out_dev, int64_t count, void *stream) {
    NQ_REQUIRE(count >= 0, NQ_ERR_SHAPE, "nq_e8_nearest: count must be non-negative");
    if (count == 0) return NQ_OK;
    NQ_REQUIRE(x_dev && out_dev, NQ_ERR_ARGUMENT, "nq_e8_nearest: null pointer");
    NQ_REQUIRE(nq::aligned(x_dev, 16) && nq::aligned(out_dev, 16), NQ_ERR_ARGUMENT,
               "nq_e8_nearest: pointers must be 16-byte aligned");
    const int threads = 256;
    const int64_t grid = (count + threads - 1) / threads;
    NQ_REQUIRE(grid <= 0x7fffffff, NQ_ERR_SHAPE, "nq_e8_nearest: too many vectors");
    hipLaunchKernelGGL(nq::e8_nearest_kernel, dim3((unsigned)grid), dim3(threads), 0,
                       (hipStream_t)stream, reinterpret_cast<const float4 *>(x_dev),
                       reinterpret_cast<float4 *>(out_dev), count);
    return nq::check_launch("nq_e8_nearest");
}

namespace {

// from this many values on, undithered rows go to the kernel built for throughput
constexpr int64_t kBulkElements = 1 << 21;
// Rows of 2048, 4096 or 8192 values on the kernel with one lane per eight values: up to
// kLanesKernelRows rows with every lane on one (block, beta) pair (us against the row-at-a-time kernel,
// 128 / 384 rows of 2048 values: 7.9 / 17.2 against 9.2 / 14.7), from there to kBlockLanesRows rows (and
// whatever is too small for the many-row kernel) with one lane per block (384 rows of 2048 / 8192 values:
// 13.5 / 42.1 against 14.6 / 47.5; 1024 rows: 21.5 / 84.0 against the many-row kernel's 21.5 / 77.5)
constexpr int64_t kLanesKernelRows = 192;
constexpr int64_t kBlockLanesRows = 512;
// (rows of 8192 values: two 1024-lane workgroups a row, one workgroup per compute unit, so 128 rows fill
// the chip and 192 rows took two rounds: 34.3 us against 19.3 for 128; with a lane per block, one workgroup
// a row, they are one round again: 24.2 us.  Rows of 4096 values, 129 to 192 of them: 15.9 against 14.5)
int64_t every_lane_rows(int n) { return n >= 4096 ? 128 : kLanesKernelRows; }

template <typename T, bool kDithered, int kPrologue = 0>
int launch_quantize(const void *x, int64_t rows, int n, int q, const float *betas, int beta_count,
                    uint32_t seed_plus_offset, uint8_t *codes, uint8_t *beta_ids, float *norms,
                    void *decoded, int hadamard_stage_dtype, hipStream_t stream,
                    nq::InputPrologue prologue = nq::InputPrologue{}) {
    // Rows of 2048, 4096 or 8192 values, q = 14, every operand 16-byte aligned, BF16 (or float32
    // without a rotation): the kernel with one lane per eight values.  Up to 16 rows (a decode step) are
    // laid out for the shortest path through one row, a prefill chunk of up to 192 rows for the fewest
    // instructions per (block, beta) pair with four workgroups a row, some hundreds of rows for the
    // fewest instructions per block with one workgroup a row; the many-row kernel takes over from there.
    constexpr bool kBf16 = std::is_same<T, uint16_t>::value, kF32 = std::is_same<T, float>::value;
    const bool lanes_input = kBf16 || (kF32 && kPrologue == 0 && hadamard_stage_dtype < 0);
    if ((kBf16 || kF32) && lanes_input && !kDithered && q == 14 && (n == 2048 || n == 4096 || n == 8192) &&
        nq::aligned(x, 16) && (kPrologue != 3 || rows <= 16) && (kBf16 || rows > every_lane_rows(n)) &&
        (rows <= kBlockLanesRows || rows * (int64_t)n < kBulkElements)) {
        // decode step: a workgroup of n / 8 lanes encodes n / 256 blocks per pass with eight lanes per
        // (block, beta) pair: 32 slices of one pass each (rows of 4096 values: while that keeps the
        // launch within one 512-lane workgroup per compute unit, 16 slices of two passes beyond: 9.3
        // against 9.9 us at 10 rows; rows of 2048 values always: 7.0 against 7.4 us); an 8192-value
        // row keeps one lane per pair, slices of 256 pairs.  Prefill chunk: every lane one pair, four slices a row (two, when four would put
        // more than two 1024-lane workgroups on a compute unit).
        const int form = rows > every_lane_rows(n) ? nq::kBlockLanes
                         : (rows > 16 ? nq::kEveryLane : (n > 4096 ? nq::kFirstLanes : nq::kEightLanes));
        int slices = n > 4096 ? n / 512 : (rows * 32 <= 256 || n <= 2048 ? 32 : 16);
        if (form == nq::kEveryLane) slices = n <= 2048 || rows * 4 * (n / 2048) <= 1024 ? 4 : 2;
        if (form == nq::kBlockLanes) slices = 1;
        if (rows * slices > 0x7fffffff) return nq::fail(NQ_ERR_SHAPE, "nq_quantize_rows: too many rows");
        const size_t lds_bytes = (size_t)(8 * ((n >> 3) + 8) + n + 4 + 8) * sizeof(float);   // + norm, beta choices
        using Kernel = void (*)(const void *, int, int64_t, int, const float *, int, float, uint32_t *, uint8_t *, float *,
                                uint4 *, int, int, nq::InputPrologue);
        Kernel kernel = form == nq::kEightLanes   ? (Kernel)nq::quantize_row_lanes_kernel<kPrologue, nq::kEightLanes>
                        : form == nq::kFirstLanes ? (Kernel)nq::quantize_row_lanes_kernel<kPrologue, nq::kFirstLanes>
                        : form == nq::kEveryLane  ? (Kernel)nq::quantize_row_lanes_kernel<kPrologue, nq::kEveryLane>
                                                  : (Kernel)nq::quantize_row_lanes_kernel<kPrologue, nq::kBlockLanes>;
        if (lds_bytes > 48 * 1024) {
            hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            if (status != hipSuccess)
                return nq::fail(NQ_ERR_LAUNCH, "nq_quantize_rows: cannot reserve %zu bytes of LDS: %s",
                                lds_bytes, hipGetErrorString(status));
        }
        hipLaunchKernelGGL(kernel, dim3((unsigned)(rows * slices)), dim3(n / 8), lds_bytes, stream, x, (int)kF32, rows, n,
                           betas, beta_count, (float)sqrt((double)n), reinterpret_cast<uint32_t *>(codes), beta_ids,
                           norms, reinterpret_cast<uint4 *>(decoded), slices, hadamard_stage_dtype >= 0 ? 1 : 0, prologue);
        return nq::check_launch("nq_quantize_rows");
    }
    if (!kDithered && kPrologue != 3 && rows * (int64_t)n >= kBulkElements) {
        int rows_per_wg = n >= 2048 ? 1 : 2048 / n;
        const size_t lds_bytes = ((size_t)rows_per_wg * n + 2 * rows_per_wg + (kPrologue == 1 ? n : 0)) * sizeof(float);
        auto kernel = nq::quantize_rows_bulk_kernel<T, kPrologue>;
        if (lds_bytes > 48 * 1024) {
            hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            if (status != hipSuccess)
                return nq::fail(NQ_ERR_LAUNCH, "nq_quantize_rows: cannot reserve %zu bytes of LDS: %s",
                                lds_bytes, hipGetErrorString(status));
        }
        const int64_t grid = (rows + rows_per_wg - 1) / rows_per_wg;
        if (grid > 0x7fffffff) return nq::fail(NQ_ERR_SHAPE, "nq_quantize_rows: too many rows");
        hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(256), lds_bytes, stream,
                           reinterpret_cast<const T *>(x), rows, n, (float)q, 1.0f / (float)q, betas, beta_count,
                           (float)sqrt((double)n), reinterpret_cast<uint32_t *>(codes), beta_ids, norms,
                           reinterpret_cast<uint4 *>(decoded), rows_per_wg, (int)nq::aligned(x, 16),
                           hadamard_stage_dtype, prologue);
        return nq::check_launch("nq_quantize_rows");
    }
    const int pairs_per_row = n / 2;
    const int target = pairs_per_row < 256 ? 256 : (pairs_per_row < 1024 ? pairs_per_row : 1024);
    int rows_per_wg = target / pairs_per_row;
    if (rows_per_wg < 1) rows_per_wg = 1;
    if (rows_per_wg > rows) rows_per_wg = (int)rows;
    int threads = rows_per_wg * pairs_per_row;
    if (threads > 1024) threads = 1024;
    // few long rows (decode activations): spread each row over several workgroups of 256
    // lanes so that the whole chip encodes it; beta bytes need 16-pair alignment
    int slices = 1;
    if (rows_per_wg == 1 && pairs_per_row > 256) {
        // long rows keep 1024 lanes for staging, rotation and the norm; about two such
        // workgroups (or four of 256 lanes) per CU in total
        const int sliced_threads = n >= 4096 ? 1024 : 256;
        const int64_t wanted = (sliced_threads == 1024 ? 512 : 1024) / rows;
        while (slices * 2 <= wanted && pairs_per_row / (slices * 2) >= 256 &&
               pairs_per_row % (slices * 2 * 16) == 0)
            slices *= 2;
        if (slices > 1) threads = sliced_threads;
    }
    if (threads < 64) threads = 64;
    const size_t lds_bytes = ((size_t)rows_per_wg * n + 2 * rows_per_wg + (kPrologue == 1 ? n : 0)) * sizeof(float);
    auto kernel = nq::quantize_rows_kernel<T, kDithered, kPrologue>;
    if (lds_bytes > 48 * 1024) {
        hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                                (int)lds_bytes);
        if (status != hipSuccess)
            return nq::fail(NQ_ERR_LAUNCH, "nq_quantize_rows: cannot reserve %zu bytes of LDS: %s",
                            lds_bytes, hipGetErrorString(status));
    }
    const int64_t grid = ((rows + rows_per_wg - 1) / rows_per_wg) * slices;
    if (grid > 0x7fffffff) return nq::fail(NQ_ERR_SHAPE, "nq_quantize_rows: too many rows");
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(threads), lds_bytes, stream,
                       reinterpret_cast<const T *>(x), rows, n, (float)q, 1.0f / (float)q, betas,
                       beta_count, (float)sqrt((double)n), seed_plus_offset,
                       reinterpret_cast<uint32_t *>(codes), beta_ids, norms,
                       reinterpret_cast<uint4 *>(decoded), rows_per_wg, slices,
                       (int)nq::aligned(x, 16), hadamard_stage_dtype, prologue);
    return nq::check_launch("nq_quantize_rows");
}

}  // namespace

extern "C" int nq_quantize_rows(const void *x_dev, int x_dtype, int64_t rows, int64_t n, int q,
                                const float *betas_dev, int beta_count, int has_dither, int64_t seed,
                                int64_t block_offset, int hadamard, uint8_t *codes_dev,
                                uint8_t *beta_ids_dev, float *norms_dev, void *decoded_bf16_dev,
                                void *stream) {
    NQ_REQUIRE(rows >= 1 && n >= 1, NQ_ERR_SHAPE, "nq_quantize_rows: rows and n must be positive");
    NQ_REQUIRE(n % 32 == 0, NQ_ERR_SHAPE,
               "nq_quantize_rows: feature count %lld must be a multiple of 32", (long long)n);
    NQ_REQUIRE(n <= 32768, NQ_ERR_SHAPE, "nq_quantize_rows: feature count %lld exceeds 32768",
               (long long)n);
    NQ_REQUIRE(q >= 2 && q <= 16, NQ_ERR_SHAPE, "nq_quantize_rows: q must be in [2, 16] for 4-bit codes");
    NQ_REQUIRE(beta_count >= 1 && beta_count <= 4, NQ_ERR_SHAPE,
               "nq_quantize_rows: beta_count must be in [1, 4] for 2-bit ids");
    NQ_REQUIRE(x_dev && betas_dev && codes_dev && beta_ids_dev && norms_dev, NQ_ERR_ARGUMENT,
               "nq_quantize_rows: null pointer");
    NQ_REQUIRE(nq::aligned(codes_dev, 4), NQ_ERR_ARGUMENT, "nq_quantize_rows: codes must be 4-byte aligned");
    NQ_REQUIRE(!decoded_bf16_dev || nq::aligned(decoded_bf16_dev, 16), NQ_ERR_ARGUMENT,
               "nq_quantize_rows: decoded output must be 16-byte aligned");
    NQ_REQUIRE(!hadamard || (n & (n - 1)) == 0, NQ_ERR_SHAPE,
               "nq_quantize_rows: the Hadamard rotation needs a power-of-two feature count, got %lld", (long long)n);
    NQ_REQUIRE(x_dtype == NQ_F32 || x_dtype == NQ_BF16 || x_dtype == NQ_F16, NQ_ERR_ARGUMENT,
               "nq_quantize_rows: unknown dtype tag %d", x_dtype);
    const int stage_dtype = hadamard ? x_dtype : -1;
    uint32_t seed_plus_offset = 0;
    if (has_dither) {
        NQ_REQUIRE(seed >= 0 && seed < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
                   "nq_quantize_rows: seed must be in [0, 2**31)");
        NQ_REQUIRE(block_offset >= 0 && block_offset + rows * (n / 8) <= ((int64_t)1 << 28), NQ_ERR_SHAPE,
                   "nq_quantize_rows: block range exceeds the stateless dither counter space");
        seed_plus_offset = (uint32_t)((uint64_t)seed + (uint64_t)block_offset * 8u);
    }
    hipStream_t s = (hipStream_t)stream;
#define NQ_DISPATCH_QUANTIZE(T)                                                                    \
    (has_dither ? launch_quantize<T, true>(x_dev, rows, (int)n, q, betas_dev, beta_count,           \
                                           seed_plus_offset, codes_dev, beta_ids_dev, norms_dev,  \
                                           decoded_bf16_dev, stage_dtype, s)                        \
                : launch_quantize<T, false>(x_dev, rows, (int)n, q, betas_dev, beta_count, 0u,      \
                                            codes_dev, beta_ids_dev, norms_dev, decoded_bf16_dev, stage_dtype, s))
    switch (x_dtype) {
        case NQ_F32: return NQ_DISPATCH_QUANTIZE(float);
        case NQ_BF16: return NQ_DISPATCH_QUANTIZE(uint16_t);
        case NQ_F16: return NQ_DISPATCH_QUANTIZE(nq::half_bits);
        default: return nq::fail(NQ_ERR_ARGUMENT, "nq_quantize_rows: unknown dtype tag %d", x_dtype);
    }
#undef NQ_DISPATCH_QUANTIZE
}

extern "C" int nq_fused_input_stage(const void *x_dev, int64_t rows, int64_t n, int mode,
                                    const void *residual_dev, void *residual_out_dev,
                                    const void *norm_weight_dev, float eps, const void *gate_dev,
                                    void *staged_out_dev, int q, const float *betas_dev, int beta_count,
                                    int hadamard, uint8_t *codes_dev, uint8_t *beta_ids_dev,
                                    float *norms_dev, void *decoded_bf16_dev, void *stream) {
    NQ_REQUIRE(rows >= 1 && n >= 32 && n % 32 == 0 && n <= 32768, NQ_ERR_SHAPE,
               "nq_fused_input_stage: rows must be positive and n a multiple of 32 up to 32768");
    NQ_REQUIRE(mode == 1 || mode == 2, NQ_ERR_ARGUMENT,
               "nq_fused_input_stage: mode must be 1 (residual + RMSNorm) or 2 (SiLU(gate) * x)");
    NQ_REQUIRE(x_dev, NQ_ERR_ARGUMENT, "nq_fused_input_stage: null input");
    NQ_REQUIRE(mode != 1 || norm_weight_dev, NQ_ERR_ARGUMENT, "nq_fused_input_stage: mode 1 needs the norm weight");
    NQ_REQUIRE(mode != 2 || gate_dev, NQ_ERR_ARGUMENT, "nq_fused_input_stage: mode 2 needs the gate rows");
    NQ_REQUIRE(mode != 1 || (eps >= 0.0f && eps < 1.0f), NQ_ERR_ARGUMENT, "nq_fused_input_stage: eps out of range");
    NQ_REQUIRE(nq::aligned(x_dev, 16) && nq::aligned(residual_dev, 16) && nq::aligned(residual_out_dev, 16) &&
                   nq::aligned(norm_weight_dev, 16) && nq::aligned(gate_dev, 16) && nq::aligned(staged_out_dev, 16),
               NQ_ERR_ARGUMENT, "nq_fused_input_stage: BF16 rows must be 16-byte aligned");
    const bool encodes = codes_dev != nullptr;
    NQ_REQUIRE(encodes || staged_out_dev || residual_out_dev, NQ_ERR_ARGUMENT,
               "nq_fused_input_stage: nothing to produce");
    if (encodes) {
        NQ_REQUIRE(betas_dev && beta_ids_dev && norms_dev, NQ_ERR_ARGUMENT, "nq_fused_input_stage: null pointer");
        NQ_REQUIRE(q >= 2 && q <= 16 && beta_count >= 1 && beta_count <= 4, NQ_ERR_SHAPE,
                   "nq_fused_input_stage: q must be in [2, 16] and beta_count in [1, 4]");
        NQ_REQUIRE(nq::aligned(codes_dev, 4) && nq::aligned(decoded_bf16_dev, 16), NQ_ERR_ARGUMENT,
                   "nq_fused_input_stage: codes need 4-byte, the decoded output 16-byte alignment");
        NQ_REQUIRE(!hadamard || (n & (n - 1)) == 0, NQ_ERR_SHAPE,
                   "nq_fused_input_stage: the Hadamard rotation needs a power-of-two feature count");
    }
    nq::InputPrologue prologue{};
    prologue.residual = reinterpret_cast<const uint16_t *>(residual_dev);
    prologue.weight = reinterpret_cast<const uint16_t *>(norm_weight_dev);
    prologue.gate = reinterpret_cast<const uint16_t *>(gate_dev);
    prologue.residual_out = reinterpret_cast<uint16_t *>(residual_out_dev);
    prologue.normed_out = reinterpret_cast<uint16_t *>(staged_out_dev);
    prologue.eps = eps;
    const int stage_dtype = (encodes && hadamard) ? NQ_BF16 : -1;
    hipStream_t s = (hipStream_t)stream;
    if (mode == 1)
        return launch_quantize<uint16_t, false, 1>(x_dev, rows, (int)n, encodes ? q : 14, betas_dev, beta_count, 0u,
                                                   codes_dev, beta_ids_dev, norms_dev, decoded_bf16_dev,
                                                   stage_dtype, s, prologue);
    return launch_quantize<uint16_t, false, 2>(x_dev, rows, (int)n, encodes ? q : 14, betas_dev, beta_count, 0u,
                                               codes_dev, beta_ids_dev, norms_dev, decoded_bf16_dev, stage_dtype,
                                               s, prologue);
}

extern "C" int nq_attention_output_stage(const void *workspace_dev, int64_t rows, int q_heads, int head_dim,
                                         int parts, void *staged_out_dev, int q, const float *betas_dev,
                                         int beta_count, int hadamard, uint8_t *codes_dev, uint8_t *beta_ids_dev,
                                         float *norms_dev, void *decoded_bf16_dev, void *stream) {
    NQ_REQUIRE(rows >= 1 && q_heads >= 1 && parts >= 1 && parts <= 512, NQ_ERR_SHAPE,
               "nq_attention_output_stage: rows, heads and parts (at most 512) must be positive");
    NQ_REQUIRE(head_dim == 64, NQ_ERR_SHAPE, "nq_attention_output_stage: head_dim %d is not 64", head_dim);
    const int64_t n = (int64_t)q_heads * head_dim;
    NQ_REQUIRE(n % 32 == 0 && n <= 32768, NQ_ERR_SHAPE, "nq_attention_output_stage: heads * head_dim exceeds 32768");
    NQ_REQUIRE(workspace_dev && nq::aligned(workspace_dev, 16), NQ_ERR_ARGUMENT,
               "nq_attention_output_stage: the attention workspace must be given, 16-byte aligned");
    const bool encodes = codes_dev != nullptr;
    NQ_REQUIRE(encodes || staged_out_dev, NQ_ERR_ARGUMENT, "nq_attention_output_stage: nothing to produce");
    if (encodes) {
        NQ_REQUIRE(betas_dev && beta_ids_dev && norms_dev, NQ_ERR_ARGUMENT, "nq_attention_output_stage: null pointer");
        NQ_REQUIRE(q >= 2 && q <= 16 && beta_count >= 1 && beta_count <= 4, NQ_ERR_SHAPE,
                   "nq_attention_output_stage: q must be in [2, 16] and beta_count in [1, 4]");
        NQ_REQUIRE(nq::aligned(codes_dev, 4) && nq::aligned(decoded_bf16_dev, 16) && nq::aligned(staged_out_dev, 16),
                   NQ_ERR_ARGUMENT, "nq_attention_output_stage: codes need 4-byte, BF16 outputs 16-byte alignment");
        NQ_REQUIRE(!hadamard || (n & (n - 1)) == 0, NQ_ERR_SHAPE,
                   "nq_attention_output_stage: the Hadamard rotation needs a power-of-two feature count");
    }
    // the layout nq_nqkv_attention_decode leaves in its workspace
    const size_t heads_total = (size_t)rows * q_heads;
    nq::InputPrologue prologue{};
    prologue.part_max = reinterpret_cast<const float *>(workspace_dev);
    prologue.part_sum = prologue.part_max + heads_total * parts;
    prologue.part_acc = prologue.part_sum + heads_total * parts;
    prologue.parts = parts;
    prologue.heads = q_heads;
    prologue.normed_out = reinterpret_cast<uint16_t *>(staged_out_dev);
    const int stage_dtype = (encodes && hadamard) ? NQ_BF16 : -1;
    return launch_quantize<uint16_t, false, 3>(workspace_dev, rows, (int)n, encodes ? q : 14, betas_dev, beta_count, 0u,
                                               codes_dev, beta_ids_dev, norms_dev, decoded_bf16_dev, stage_dtype,
                                               (hipStream_t)stream, prologue);
}

extern "C" int nq_dequantize_rows(const uint8_t *codes_dev, const uint8_t *beta_ids_dev,
                                  const float *norms_dev, const float *betas_dev, int64_t rows,
                                  int64_t n, int q, int has_dither, int64_t seed,
                                  int64_t block_offset, void *out_dev, int out_dtype, void *stream) {
    NQ_REQUIRE(rows >= 1 && n >= 1, NQ_ERR_SHAPE, "nq_dequantize_rows: rows and n must be positive");
    NQ_REQUIRE(n % 32 == 0, NQ_ERR_SHAPE,
               "nq_dequantize_rows: feature count %lld must be a multiple of 32", (long long)n);
    NQ_REQUIRE(q >= 2 && q <= 16, NQ_ERR_SHAPE, "nq_dequantize_rows: q must be in [2, 16]");
    NQ_REQUIRE(out_dtype == NQ_F32 || out_dtype == NQ_BF16 || out_dtype == NQ_F16, NQ_ERR_ARGUMENT,
               "nq_dequantize_rows: unknown dtype tag %d", out_dtype);
    NQ_REQUIRE(codes_dev && beta_ids_dev && norms_dev && betas_dev && out_dev, NQ_ERR_ARGUMENT,
               "nq_dequantize_rows: null pointer");
    NQ_REQUIRE(nq::aligned(codes_dev, 4) && nq::aligned(out_dev, 16), NQ_ERR_ARGUMENT,
               "nq_dequantize_rows: codes need 4-byte and out 16-byte alignment");
    const int64_t blocks = rows * (n / 8);
    if (has_dither) {
        NQ_REQUIRE(seed >= 0 && seed < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
                   "nq_dequantize_rows: seed must be in [0, 2**31)");
        NQ_REQUIRE(block_offset >= 0 && block_offset + blocks <= ((int64_t)1 << 28), NQ_ERR_SHAPE,
                   "nq_dequantize_rows: block range exceeds the stateless dither counter space");
    }
    const int threads = 256;
    const int64_t grid = (blocks + threads - 1) / threads;
    NQ_REQUIRE(grid <= 0x7fffffff, NQ_ERR_SHAPE, "nq_dequantize_rows: too many blocks");
    const uint32_t seed_plus_offset = (uint32_t)((uint64_t)seed + (uint64_t)block_offset * 8u);
    const float sqrt_n = (float)sqrt((double)n);
    const uint32_t *codes = reinterpret_cast<const uint32_t *>(codes_dev);
    if (has_dither)
        hipLaunchKernelGGL(nq::dequantize_rows_kernel<true>, dim3((unsigned)grid), dim3(threads), 0,
                           (hipStream_t)stream, codes, beta_ids_dev, norms_dev, betas_dev, blocks,
                           (int)(n / 8), (float)q, sqrt_n, seed_plus_offset, out_dev, out_dtype);
    else
        hipLaunchKernelGGL(nq::dequantize_rows_kernel<false>, dim3((unsigned)grid), dim3(threads), 0,
                           (hipStream_t)stream, codes, beta_ids_dev, norms_dev, betas_dev, blocks,
                           (int)(n / 8), (float)q, sqrt_n, 0u, out_dev, out_dtype);
    return nq::check_launch("nq_dequantize_rows");
}
