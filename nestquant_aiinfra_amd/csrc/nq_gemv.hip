// Packed W4A4 linear for decode (M = 1..8 tokens): the NQRT4 weight stream is decoded in
// registers; nothing but packed words, norms, the BF16 activation and the output touches
// memory.
//
// Layout of the work.  grid = (ceil(N / rows_per_wg), split_k); a workgroup of four
// wavefronts owns `rows_per_wg` output channels and one K slice, and its wavefronts
// interleave over the slice: in every step lane l of wavefront w decodes block
// 256 * step + 64 * w + l, so a wavefront reads 256 contiguous bytes of code words (one
// 32-bit word = one E8 block = 8 weights) and the 16 beta bytes that go with them.
//   * Each lane regenerates the dither of its block, decodes it (lattice.py / codec.py
//     arithmetic, see nq_e8.hip.h), rounds to BF16 like the reference kernels
//     (nestquant/runtime/nqrt4_cooperative_device.cuh:150-171) and accumulates M dot products
//     in FP32 with v_dot2_f32_bf16.
//   * The activation is consumed as decoded BF16 [M, K]: the encoder emits it as a side
//     product, otherwise a small kernel decodes the NQA4 streams once per call (the
//     reference re-decodes it in every warp, nestquant/runtime/nqrt4_w4a4_mma.cu:914-925).
//   * Lanes are combined with a fixed butterfly, wavefronts through LDS in index order, and
//     K slices by a second kernel in ascending slice order: results are deterministic.
// The kernel is bound by vector-ALU work (about 600 instructions per 8-weight block, most
// of it the 31-bit hash and two exact E8 searches), not by the 4.25 bits per weight it reads.
#include "nq_linear_common.hip.h"

#include <math.h>

namespace nq {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / 64;
constexpr int kGemvMaxRows = 8;

template <int M, bool kHinted>
__global__ void __launch_bounds__(kGemvThreads)
w4a4_gemv_kernel(const uint4 *__restrict__ act,          // decoded BF16 [m_rows][K / 8] blocks
                 const uint32_t *__restrict__ w_codes, const uint16_t *__restrict__ w_hints,
                 const uint8_t *__restrict__ w_beta_ids,
                 const float *__restrict__ w_norms, const float *__restrict__ w_betas,
                 int m_rows, int k_size, int n_size, int k_slice, int rows_per_wg,
                 uint32_t seed_plus_offset, float sqrt_k, float *__restrict__ out_f32,
                 uint16_t *__restrict__ out_bf16) {
    __shared__ float partial[kGemvWaves][kGemvMaxRows][M];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int blocks_per_row = k_size >> 3;
    const int slice_blocks = k_slice >> 3;
    const int slice_first_block = blockIdx.y * slice_blocks;
    const float wbeta[4] = {w_betas[0], w_betas[1], w_betas[2], w_betas[3]};

    for (int r = 0; r < rows_per_wg; r++) {
        const int n = blockIdx.x * rows_per_wg + r;
        float acc[M];
#pragma unroll
        for (int m = 0; m < M; m++) acc[m] = 0.0f;
        if (n < n_size) {
            const float wscale = w_norms[n] / sqrt_k;
            const int64_t row_first_block = (int64_t)n * blocks_per_row + slice_first_block;
            for (int b = tid; b < slice_blocks; b += kGemvThreads) {
                const int64_t g = row_first_block + b;
                const uint32_t word = w_codes[g];
                const uint32_t ids = w_beta_ids[g >> 2];
                // the activation blocks do not depend on the decode: request them first
                uint4 a[M];
#pragma unroll
                for (int m = 0; m < M; m++)
                    a[m] = m < m_rows ? act[(int64_t)m * blocks_per_row + slice_first_block + b] : make_uint4(0, 0, 0, 0);
                float v[8];
                if (kHinted) {
                    uint32_t hints = w_hints[g];
                    decode_codeword<true, 1>(word, 14.0f, seed_plus_offset + (uint32_t)g * 8u, v, &hints);
                } else {
                    decode_codeword<true>(word, 14.0f, seed_plus_offset + (uint32_t)g * 8u, v);
                }
                const float scale = wbeta[(ids >> (2 * (g & 3))) & 3] * wscale;
                bf16x2 w[4];
#pragma unroll
                for (int j = 0; j < 4; j++) w[j] = pack_bf16x2(v[2 * j] * scale, v[2 * j + 1] * scale);
#pragma unroll
                for (int m = 0; m < M; m++) {
                    acc[m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a[m].x), w[0], acc[m], false);
                    acc[m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a[m].y), w[1], acc[m], false);
                    acc[m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a[m].z), w[2], acc[m], false);
                    acc[m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a[m].w), w[3], acc[m], false);
                }
            }
        }
        // fixed butterfly over the 64 lanes
#pragma unroll
        for (int m = 0; m < M; m++) {
            float v = acc[m];
#pragma unroll
            for (int offset = 32; offset >= 1; offset >>= 1) v = v + __shfl_xor(v, offset, 64);
            if (lane == 0) partial[wave][r][m] = v;
        }
    }
    __syncthreads();
    // wavefront partials in index order
    if (tid < rows_per_wg * M) {
        const int r = tid / M, m = tid - r * M;
        const int n = blockIdx.x * rows_per_wg + r;
        if (n < n_size && m < m_rows) {
            float total = partial[0][r][m];
#pragma unroll
            for (int w = 1; w < kGemvWaves; w++) total = total + partial[w][r][m];
            if (out_f32)
                out_f32[((int64_t)blockIdx.y * m_rows + m) * n_size + n] = total;
            else
                out_bf16[(int64_t)m * n_size + n] = f32_to_bf16(total);
        }
    }
}

// One lane per weight block: run both exact lattice searches once and keep their outcomes.
__global__ void __launch_bounds__(256)
make_decode_hints_kernel(const uint32_t *__restrict__ w_codes, int64_t blocks, uint32_t seed_plus_offset,
                         uint16_t *__restrict__ hints) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= blocks) return;
    float v[8];
    uint32_t h = 0u;
    decode_codeword<true, 2>(w_codes[g], 14.0f, seed_plus_offset + (uint32_t)g * 8u, v, &h);
    hints[g] = (uint16_t)h;
}

}  // namespace nq

extern "C" int nq_w4a4_make_decode_hints(const uint8_t *w_codes_dev, int64_t rows, int64_t k,
                                         int64_t weight_offset, int64_t weight_seed, uint16_t *hints_dev,
                                         void *stream) {
    NQ_REQUIRE(rows >= 1 && k >= 8 && k % 8 == 0, NQ_ERR_SHAPE,
               "nq_w4a4_make_decode_hints: rows must be positive and K a positive multiple of 8");
    NQ_REQUIRE(w_codes_dev && hints_dev && nq::aligned(w_codes_dev, 4) && nq::aligned(hints_dev, 2),
               NQ_ERR_ARGUMENT, "nq_w4a4_make_decode_hints: null or misaligned pointer");
    NQ_REQUIRE(weight_seed >= 0 && weight_seed < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
               "nq_w4a4_make_decode_hints: seed must be in [0, 2**31)");
    const int64_t blocks = rows * (k / 8);
    NQ_REQUIRE(weight_offset >= 0 && weight_offset + blocks <= ((int64_t)1 << 28), NQ_ERR_SHAPE,
               "nq_w4a4_make_decode_hints: block range exceeds the stateless dither counter space");
    const uint32_t seed_plus_offset = (uint32_t)((uint64_t)weight_seed + (uint64_t)weight_offset * 8u);
    hipLaunchKernelGGL(nq::make_decode_hints_kernel, dim3((unsigned)((blocks + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, reinterpret_cast<const uint32_t *>(w_codes_dev), blocks,
                       seed_plus_offset, hints_dev);
    return nq::check_launch("nq_w4a4_make_decode_hints");
}

namespace {

int m_tile_of(int m) { return m == 1 ? 1 : (m == 2 ? 2 : (m <= 4 ? 4 : 8)); }

// A workgroup consumes 2048 K-elements per step.  Long-K, narrow-N shapes (down_proj) are
// split until every SIMD of the 256 CUs has several wavefronts to interleave.
int pick_split(int k, int n, int requested) {
    if (requested > 0) return requested;
    int split = 1;
    while (split < 8 && (k / (split * 2)) % 32 == 0 && (int64_t)n * split < 4096 && k / (split * 2) >= 2048)
        split *= 2;
    return split;
}

}  // namespace

extern "C" size_t nq_w4a4_gemv_workspace_bytes(int m, int k, int n, int split_k, int have_decoded_activation) {
    if (m < 1 || n < 1 || k < 1) return 0;
    const int split = pick_split(k, n, split_k);
    size_t bytes = 0;
    if (!have_decoded_activation) bytes += nq::align256((size_t)m * k * 2);
    if (split > 1) bytes += (size_t)split * (size_t)m * (size_t)n * sizeof(float);
    return bytes;
}

extern "C" int nq_w4a4_gemv(const uint8_t *act_codes_dev, const uint8_t *act_beta_ids_dev,
                            const float *act_norms_dev, const float *act_betas_dev,
                            const void *act_decoded_dev, const uint8_t *w_codes_dev,
                            const uint16_t *w_hints_dev, const uint8_t *w_beta_ids_dev, const float *w_norms_dev,
                            const float *w_betas_dev, int m, int k, int n, int64_t weight_offset,
                            int64_t weight_seed, int split_k, void *out_dev, int out_dtype,
                            void *workspace_dev, size_t workspace_bytes, void *stream) {
    NQ_REQUIRE(m >= 1 && m <= 8, NQ_ERR_SHAPE, "nq_w4a4_gemv: M = %d is outside [1, 8]", m);
    NQ_REQUIRE(k >= 32 && k % 32 == 0, NQ_ERR_SHAPE, "nq_w4a4_gemv: K = %d must be a positive multiple of 32", k);
    NQ_REQUIRE(n >= 1, NQ_ERR_SHAPE, "nq_w4a4_gemv: N must be positive");
    NQ_REQUIRE(split_k == 0 || split_k == 1 || split_k == 2 || split_k == 4 || split_k == 8,
               NQ_ERR_ARGUMENT, "nq_w4a4_gemv: split_k must be 0, 1, 2, 4 or 8");
    NQ_REQUIRE(out_dtype == NQ_F32 || out_dtype == NQ_BF16, NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv: output dtype tag %d is not F32 or BF16", out_dtype);
    NQ_REQUIRE(w_codes_dev && w_beta_ids_dev && w_norms_dev && w_betas_dev && out_dev, NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv: null pointer");
    NQ_REQUIRE(act_decoded_dev || (act_codes_dev && act_beta_ids_dev && act_norms_dev && act_betas_dev),
               NQ_ERR_ARGUMENT, "nq_w4a4_gemv: neither packed nor decoded activation given");
    NQ_REQUIRE(nq::aligned(w_codes_dev, 4) && (!act_codes_dev || nq::aligned(act_codes_dev, 4)) &&
                   (!act_decoded_dev || nq::aligned(act_decoded_dev, 16)) && nq::aligned(w_hints_dev, 2),
               NQ_ERR_ARGUMENT, "nq_w4a4_gemv: code streams need 4-byte, decoded activation 16-byte alignment");
    NQ_REQUIRE(weight_seed >= 0 && weight_seed < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv: seed must be in [0, 2**31)");
    NQ_REQUIRE(weight_offset >= 0 && weight_offset + (int64_t)n * (k / 8) <= ((int64_t)1 << 28),
               NQ_ERR_SHAPE, "nq_w4a4_gemv: block range exceeds the stateless dither counter space");
    const int split = pick_split(k, n, split_k);
    NQ_REQUIRE(k % split == 0 && (k / split) % 32 == 0, NQ_ERR_SHAPE,
               "nq_w4a4_gemv: K / split_k = %d / %d must be a multiple of 32", k, split);
    const size_t decoded_bytes = act_decoded_dev ? 0 : nq::align256((size_t)m * k * 2);
    const size_t need = decoded_bytes + (split > 1 ? (size_t)split * m * n * sizeof(float) : 0);
    NQ_REQUIRE(need == 0 || (workspace_dev && workspace_bytes >= need), NQ_ERR_WORKSPACE,
               "nq_w4a4_gemv: needs a %zu-byte workspace, got %zu", need, workspace_bytes);
    NQ_REQUIRE(need == 0 || nq::aligned(workspace_dev, 16), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv: workspace must be 16-byte aligned");

    hipStream_t s = (hipStream_t)stream;
    const float sqrt_k = (float)sqrt((double)k);
    const uint4 *act = reinterpret_cast<const uint4 *>(act_decoded_dev);
    if (!act) {
        int status = nq::launch_decode_activation(act_codes_dev, act_beta_ids_dev, act_norms_dev, act_betas_dev,
                                                  m, k, workspace_dev, s);
        if (status != NQ_OK) return status;
        act = reinterpret_cast<const uint4 *>(workspace_dev);
    }
    float *partials = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace_dev) + decoded_bytes);

    const int k_slice = k / split;
    // few rows per workgroup keeps many short wavefronts in flight on every SIMD
    const int rows_per_wg = (int64_t)n * split >= 8192 ? 4 : 2;
    const dim3 grid((unsigned)((n + rows_per_wg - 1) / rows_per_wg), (unsigned)split);
    const uint32_t seed_plus_offset = (uint32_t)((uint64_t)weight_seed + (uint64_t)weight_offset * 8u);
    float *target_f32 = split > 1 ? partials : (out_dtype == NQ_F32 ? (float *)out_dev : nullptr);
    uint16_t *target_bf16 = (split > 1 || out_dtype == NQ_F32) ? nullptr : (uint16_t *)out_dev;
    const uint32_t *wc = reinterpret_cast<const uint32_t *>(w_codes_dev);
#define NQ_LAUNCH_GEMV_AS(MT, HINTED)                                                               \
    hipLaunchKernelGGL((nq::w4a4_gemv_kernel<MT, HINTED>), grid, dim3(nq::kGemvThreads), 0, s, act, \
                       wc, w_hints_dev, w_beta_ids_dev, w_norms_dev, w_betas_dev, m, k, n, k_slice, \
                       rows_per_wg, seed_plus_offset, sqrt_k, target_f32, target_bf16)
#define NQ_LAUNCH_GEMV(MT)                                                                          \
    do {                                                                                            \
        if (w_hints_dev) NQ_LAUNCH_GEMV_AS(MT, true);                                               \
        else NQ_LAUNCH_GEMV_AS(MT, false);                                                          \
    } while (0)
    switch (m_tile_of(m)) {
        case 1: NQ_LAUNCH_GEMV(1); break;
        case 2: NQ_LAUNCH_GEMV(2); break;
        case 4: NQ_LAUNCH_GEMV(4); break;
        default: NQ_LAUNCH_GEMV(8); break;
    }
#undef NQ_LAUNCH_GEMV
#undef NQ_LAUNCH_GEMV_AS
    int status = nq::check_launch("nq_w4a4_gemv");
    if (status != NQ_OK || split == 1) return status;
    return nq::launch_splitk_reduce(partials, split, (int64_t)m * n, out_dev, out_dtype, s);
}
