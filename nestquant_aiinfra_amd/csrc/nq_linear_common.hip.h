// Pieces shared by the packed W4A4 linear kernels (decode GEMV and prefill GEMM).
#pragma once

#include "nq_e8.hip.h"
#include "nq_host.h"

// the row count from which the decode linears run on the matrix cores (measuring builds set another)
#ifndef NQ_MFMA_FROM_ROWS
#define NQ_MFMA_FROM_ROWS 2
#endif

namespace nq {


// NQA4 streams -> BF16 [M, K], exactly bf16((decode * beta) * (norm / sqrt(K)))
static __global__ void __launch_bounds__(256)
decode_activation_kernel(const uint32_t *__restrict__ codes, const uint8_t *__restrict__ beta_ids,
                         const float *__restrict__ norms, const float *__restrict__ betas,
                         int64_t blocks, int blocks_per_row, float sqrt_k, uint4 *__restrict__ out) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= blocks) return;
    float v[8];
    decode_codeword<false>(codes[g], 14.0f, 0u, v);
    const float beta = betas[(beta_ids[g >> 2] >> (2 * (g & 3))) & 3];
    const float scale = norms[g / blocks_per_row] / sqrt_k;
    uint32_t h[8];
#pragma unroll
    for (int j = 0; j < 8; j++) h[j] = f32_to_bf16((v[j] * beta) * scale);
    out[g] = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
}


// Decodes the NQA4 streams of [m, k] into BF16 at `out` (16-byte aligned, m * k * 2 bytes).
inline int launch_decode_activation(const uint8_t *codes, const uint8_t *beta_ids, const float *norms,
                                    const float *betas, int m, int k, void *out, hipStream_t stream) {
    const int64_t blocks = (int64_t)m * (k / 8);
    hipLaunchKernelGGL(decode_activation_kernel, dim3((unsigned)((blocks + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const uint32_t *>(codes), beta_ids, norms, betas, blocks, k / 8,
                       (float)sqrt((double)k), reinterpret_cast<uint4 *>(out));
    return check_launch("activation decode");
}

// partial [split][M][N] float32 -> out [M][N]; slices added in ascending order
// (same rule as nestquant/runtime/nqrt4_w4a4_mma.cu:411-420).
static __global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float *__restrict__ partial, int split, int64_t count,
                     float *__restrict__ out_f32, uint16_t *__restrict__ out_bf16) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float total = 0.0f;
    for (int s = 0; s < split; s++) total = total + partial[(int64_t)s * count + i];
    if (out_f32) out_f32[i] = total;
    else out_bf16[i] = f32_to_bf16(total);
}

inline int launch_splitk_reduce(const float *partials, int split, int64_t count, void *out, int out_dtype,
                                hipStream_t stream) {
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, partials,
                       split, count, out_dtype == NQ_F32 ? (float *)out : nullptr,
                       out_dtype == NQ_F32 ? nullptr : (uint16_t *)out);
    return check_launch("split-K reduce");
}

// The same sum for partial results laid out weight by weight (the grouped launch of the fused
// kernel): elements [end[g - 1], end[g]) of a slice belong to out[g], BF16, in the same order.
constexpr int kReduceMaxOutputs = 4;
struct ReduceOutputs {
    uint16_t *out[kReduceMaxOutputs];
    int64_t end[kReduceMaxOutputs];
};

static __global__ void __launch_bounds__(256)
splitk_reduce_grouped_kernel(const float *__restrict__ partial, int split, int64_t count, ReduceOutputs outputs) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float total = 0.0f;
    for (int s = 0; s < split; s++) total = total + partial[(int64_t)s * count + i];
    // selects, not an index into the argument: the struct stays in scalar registers
    const bool first = i < outputs.end[0], second = i < outputs.end[1], third = i < outputs.end[2];
    uint16_t *out = first ? outputs.out[0] : (second ? outputs.out[1] : (third ? outputs.out[2] : outputs.out[3]));
    const int64_t begin = first ? 0 : (second ? outputs.end[0] : (third ? outputs.end[1] : outputs.end[2]));
    out[i - begin] = f32_to_bf16(total);
}

inline int launch_splitk_reduce_grouped(const float *partials, int split, int64_t count, const ReduceOutputs &outputs,
                                        hipStream_t stream) {
    hipLaunchKernelGGL(splitk_reduce_grouped_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream,
                       partials, split, count, outputs);
    return check_launch("split-K reduce");
}

inline size_t align256(size_t bytes) { return (bytes + 255) & ~(size_t)255; }

// Sum over the 16 lanes of a DPP row, left in every lane of the row: exchanges inside quads,
// then the mirrored half row, then the mirrored row.
__device__ __forceinline__ float row16_sum(float v) {
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));  // row_mirror
    return v;
}

// Several weights that share one activation (q/k/v or gate/up) in one launch: the grid is the
// concatenation of their channel groups.
constexpr int kGemvMaxGroup = 4;
struct GemvWeights {
    const uint32_t *words[kGemvMaxGroup];
    const uint16_t *tails[kGemvMaxGroup];
    const float *norms[kGemvMaxGroup], *betas[kGemvMaxGroup];
    void *out[kGemvMaxGroup];
    int n[kGemvMaxGroup], first_group[kGemvMaxGroup];
    uint32_t seed_plus_offset[kGemvMaxGroup];
    int count;
};

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

}  // namespace nq
