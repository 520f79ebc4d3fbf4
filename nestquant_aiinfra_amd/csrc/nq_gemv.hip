// Packed W4A4 linear for decode (M = 1..8 tokens): both operands are decoded in registers
// from their 4-bit streams; nothing but packed words, norms and the output touches HBM.
//
// Layout of the work.  grid = (ceil(N / rows_per_wg), split_k); a workgroup of four
// wavefronts owns `rows_per_wg` output channels and one K slice.
//   * The NQA4 activation slice is decoded once per workgroup into LDS as BF16 [M][slice]
//     (the reference re-decodes it in every warp, nestquant/runtime/nqrt4_w4a4_mma.cu:914-925).
//   * A wavefront streams one weight row at a time: each lane issues one 128-bit load
//     (four consecutive E8 blocks = 32 weights) plus the one byte holding their four
//     beta ids, so a wavefront reads 1 KiB of contiguous code words per step.
//   * Each lane regenerates the dither of its blocks, decodes them (lattice.py / codec.py
//     arithmetic, see nq_e8.hip.h), rounds to BF16 like the reference kernels
//     (nqrt4_cooperative_device.cuh:150-171) and accumulates M dot products in FP32.
//   * Lanes are combined with a fixed butterfly; K slices are combined by a second kernel in
//     ascending slice order, so results are run-to-run deterministic.
#include "nq_e8.hip.h"
#include "nq_host.h"

#include <math.h>

namespace nq {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / 64;

template <int M>
__global__ void __launch_bounds__(kGemvThreads)
w4a4_gemv_kernel(const uint32_t *__restrict__ act_codes, const uint8_t *__restrict__ act_beta_ids,
                 const float *__restrict__ act_norms, const float *__restrict__ act_betas,
                 const uint32_t *__restrict__ w_codes, const uint8_t *__restrict__ w_beta_ids,
                 const float *__restrict__ w_norms, const float *__restrict__ w_betas,
                 int m_rows, int k_size, int n_size, int k_slice, int rows_per_wg,
                 uint32_t seed_plus_offset, float sqrt_k, float *__restrict__ out_f32,
                 uint16_t *__restrict__ out_bf16) {
    extern __shared__ uint4 act_lds[];                       // [M][k_slice / 8] blocks of 8 BF16
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int blocks_per_row = k_size >> 3;
    const int slice_blocks = k_slice >> 3;
    const int slice_first_block = blockIdx.y * slice_blocks;
    const float q = 14.0f;

    // ---- activation slice -> LDS (BF16), one lane per block --------------------------------
    for (int i = tid; i < M * slice_blocks; i += kGemvThreads) {
        const int m = i / slice_blocks, b = i - m * slice_blocks;
        uint4 packed = make_uint4(0, 0, 0, 0);
        if (m < m_rows) {
            const int64_t g = (int64_t)m * blocks_per_row + slice_first_block + b;
            float v[8];
            decode_codeword<false>(act_codes[g], q, 0u, v);
            const float beta = act_betas[(act_beta_ids[g >> 2] >> (2 * (g & 3))) & 3];
            const float scale = act_norms[m] / sqrt_k;
            uint32_t h[8];
#pragma unroll
            for (int j = 0; j < 8; j++) h[j] = f32_to_bf16((v[j] * beta) * scale);
            packed = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16),
                                h[6] | (h[7] << 16));
        }
        act_lds[i] = packed;
    }
    __syncthreads();

    const float wbeta[4] = {w_betas[0], w_betas[1], w_betas[2], w_betas[3]};

    // ---- weight rows ---------------------------------------------------------------------------
    for (int r = wave; r < rows_per_wg; r += kGemvWaves) {
        const int n = blockIdx.x * rows_per_wg + r;
        if (n >= n_size) break;
        const float wscale = w_norms[n] / sqrt_k;
        const int64_t row_first_block = (int64_t)n * blocks_per_row + slice_first_block;
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; m++) acc[m] = 0.0f;

        for (int b0 = lane * 4; b0 < slice_blocks; b0 += 64 * 4) {
            const int64_t g0 = row_first_block + b0;                     // multiple of 4
            const uint4 words = *reinterpret_cast<const uint4 *>(w_codes + g0);
            const uint32_t ids = w_beta_ids[g0 >> 2];
            const uint32_t word[4] = {words.x, words.y, words.z, words.w};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                float v[8];
                decode_codeword<true>(word[t], q, seed_plus_offset + (uint32_t)(g0 + t) * 8u, v);
                const float scale = wbeta[(ids >> (2 * t)) & 3];
                float w[8];
#pragma unroll
                for (int j = 0; j < 8; j++)
                    w[j] = bf16_to_f32(f32_to_bf16((v[j] * scale) * wscale));
#pragma unroll
                for (int m = 0; m < M; m++) {
                    const uint4 a = act_lds[m * slice_blocks + b0 + t];
                    const uint32_t aw[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        acc[m] = __builtin_fmaf(__uint_as_float(aw[j] << 16), w[2 * j], acc[m]);
                        acc[m] = __builtin_fmaf(__uint_as_float(aw[j] & 0xffff0000u), w[2 * j + 1], acc[m]);
                    }
                }
            }
        }

        // fixed butterfly over the 64 lanes
#pragma unroll
        for (int m = 0; m < M; m++) {
            float v = acc[m];
#pragma unroll
            for (int offset = 32; offset >= 1; offset >>= 1) v = v + __shfl_xor(v, offset, 64);
            acc[m] = v;
        }
        if (lane == 0) {
#pragma unroll
            for (int m = 0; m < M; m++) {
                if (m >= m_rows) break;
                if (out_f32)
                    out_f32[((int64_t)blockIdx.y * m_rows + m) * n_size + n] = acc[m];
                else
                    out_bf16[(int64_t)m * n_size + n] = f32_to_bf16(acc[m]);
            }
        }
    }
}

// partial [split][M][N] float32 -> out [M][N]; slices added in ascending order
// (same rule as nestquant/runtime/nqrt4_w4a4_mma.cu:411-420).
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float *__restrict__ partial, int split, int64_t count,
                     float *__restrict__ out_f32, uint16_t *__restrict__ out_bf16) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float total = 0.0f;
    for (int s = 0; s < split; s++) total = total + partial[(int64_t)s * count + i];
    if (out_f32) out_f32[i] = total;
    else out_bf16[i] = f32_to_bf16(total);
}

}  // namespace nq

namespace {

int m_tile_of(int m) { return m == 1 ? 1 : (m == 2 ? 2 : (m <= 4 ? 4 : 8)); }

// A wavefront consumes 2048 K-elements per step, so slices shorter than that idle lanes.
// Split long-K, narrow-N shapes (down_proj) until there are enough wavefronts for 256 CUs,
// and in any case until the BF16 activation slice fits in 64 KiB of LDS.
int pick_split(int m, int k, int n, int requested) {
    if (requested > 0) return requested;
    int split = 1;
    while (split < 8 && (k / (split * 2)) % 32 == 0 &&
           ((size_t)m_tile_of(m) * (k / split) * 2 > 64 * 1024 ||
            ((int64_t)n * split < 8192 && k / (split * 2) >= 2048)))
        split *= 2;
    return split;
}

}  // namespace

extern "C" size_t nq_w4a4_gemv_workspace_bytes(int m, int k, int n, int split_k) {
    if (m < 1 || n < 1 || k < 1) return 0;
    const int split = pick_split(m, k, n, split_k);
    return split > 1 ? (size_t)split * (size_t)m * (size_t)n * sizeof(float) : 0;
}

extern "C" int nq_w4a4_gemv(const uint8_t *act_codes_dev, const uint8_t *act_beta_ids_dev,
                            const float *act_norms_dev, const float *act_betas_dev,
                            const uint8_t *w_codes_dev, const uint8_t *w_beta_ids_dev,
                            const float *w_norms_dev, const float *w_betas_dev, int m, int k, int n,
                            int64_t weight_offset, int64_t weight_seed, int split_k, void *out_dev,
                            int out_dtype, void *workspace_dev, size_t workspace_bytes,
                            void *stream) {
    NQ_REQUIRE(m >= 1 && m <= 8, NQ_ERR_SHAPE, "nq_w4a4_gemv: M = %d is outside [1, 8]", m);
    NQ_REQUIRE(k >= 32 && k % 32 == 0, NQ_ERR_SHAPE, "nq_w4a4_gemv: K = %d must be a positive multiple of 32", k);
    NQ_REQUIRE(n >= 1, NQ_ERR_SHAPE, "nq_w4a4_gemv: N must be positive");
    NQ_REQUIRE(split_k == 0 || split_k == 1 || split_k == 2 || split_k == 4 || split_k == 8,
               NQ_ERR_ARGUMENT, "nq_w4a4_gemv: split_k must be 0, 1, 2, 4 or 8");
    NQ_REQUIRE(out_dtype == NQ_F32 || out_dtype == NQ_BF16, NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv: output dtype tag %d is not F32 or BF16", out_dtype);
    NQ_REQUIRE(act_codes_dev && act_beta_ids_dev && act_norms_dev && act_betas_dev && w_codes_dev &&
                   w_beta_ids_dev && w_norms_dev && w_betas_dev && out_dev,
               NQ_ERR_ARGUMENT, "nq_w4a4_gemv: null pointer");
    NQ_REQUIRE(nq::aligned(act_codes_dev, 4) && nq::aligned(w_codes_dev, 16), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv: activation codes need 4-byte and weight codes 16-byte alignment");
    NQ_REQUIRE(weight_seed >= 0 && weight_seed < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv: seed must be in [0, 2**31)");
    NQ_REQUIRE(weight_offset >= 0 && weight_offset + (int64_t)n * (k / 8) <= ((int64_t)1 << 28),
               NQ_ERR_SHAPE, "nq_w4a4_gemv: block range exceeds the stateless dither counter space");
    const int split = pick_split(m, k, n, split_k);
    NQ_REQUIRE(k % split == 0 && (k / split) % 32 == 0, NQ_ERR_SHAPE,
               "nq_w4a4_gemv: K / split_k = %d / %d must be a multiple of 32", k, split);
    const size_t need = split > 1 ? (size_t)split * m * n * sizeof(float) : 0;
    NQ_REQUIRE(need == 0 || (workspace_dev && workspace_bytes >= need), NQ_ERR_WORKSPACE,
               "nq_w4a4_gemv: split_k = %d needs a %zu-byte workspace, got %zu", split, need,
               workspace_bytes);

    const int k_slice = k / split;
    const int m_tile = m_tile_of(m);
    const size_t lds_bytes = (size_t)m_tile * k_slice * 2;
    NQ_REQUIRE(lds_bytes <= 64 * 1024, NQ_ERR_SHAPE,
               "nq_w4a4_gemv: M = %d with K slice %d needs %zu bytes of LDS (limit 65536); raise split_k",
               m, k_slice, lds_bytes);
    const int rows_per_wg = 8;
    const dim3 grid((unsigned)((n + rows_per_wg - 1) / rows_per_wg), (unsigned)split);
    const uint32_t seed_plus_offset = (uint32_t)((uint64_t)weight_seed + (uint64_t)weight_offset * 8u);
    const float sqrt_k = (float)sqrt((double)k);
    float *target_f32 = split > 1 ? (float *)workspace_dev : (out_dtype == NQ_F32 ? (float *)out_dev : nullptr);
    uint16_t *target_bf16 = (split > 1 || out_dtype == NQ_F32) ? nullptr : (uint16_t *)out_dev;
    hipStream_t s = (hipStream_t)stream;
    const uint32_t *ac = reinterpret_cast<const uint32_t *>(act_codes_dev);
    const uint32_t *wc = reinterpret_cast<const uint32_t *>(w_codes_dev);
#define NQ_LAUNCH_GEMV(MT)                                                                          \
    hipLaunchKernelGGL(nq::w4a4_gemv_kernel<MT>, grid, dim3(nq::kGemvThreads), lds_bytes, s, ac,    \
                       act_beta_ids_dev, act_norms_dev, act_betas_dev, wc, w_beta_ids_dev,          \
                       w_norms_dev, w_betas_dev, m, k, n, k_slice, rows_per_wg, seed_plus_offset,   \
                       sqrt_k, target_f32, target_bf16)
    switch (m_tile) {
        case 1: NQ_LAUNCH_GEMV(1); break;
        case 2: NQ_LAUNCH_GEMV(2); break;
        case 4: NQ_LAUNCH_GEMV(4); break;
        default: NQ_LAUNCH_GEMV(8); break;
    }
#undef NQ_LAUNCH_GEMV
    int status = nq::check_launch("nq_w4a4_gemv");
    if (status != NQ_OK || split == 1) return status;
    const int64_t count = (int64_t)m * n;
    hipLaunchKernelGGL(nq::splitk_reduce_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s,
                       (const float *)workspace_dev, split, count,
                       out_dtype == NQ_F32 ? (float *)out_dev : nullptr,
                       out_dtype == NQ_F32 ? nullptr : (uint16_t *)out_dev);
    return nq::check_launch("nq_w4a4_gemv (split-K reduce)");
}
