// Packed W4A4 linear for decode (M = 1..16 tokens): the NQRT4 weight stream is decoded in
// registers; nothing but packed words, norms, the BF16 activation and the output touches
// memory.  Two kernels share the decode: the vector-unit kernel described next (any weight
// form, up to eight tokens), and a matrix-core kernel for resolved weights (further down).
//
// Layout of the work (vector-unit kernel).  grid = (ceil(N / rows_per_wg), split_k); a workgroup of four
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
//   * Lanes are combined in rows of 16 with fixed register exchanges, rows and wavefronts
//     through LDS in index order, and K slices by a second kernel in ascending slice order:
//     results are deterministic.
// The kernel is bound by vector-ALU work, not by the bits it reads: about 600 instructions
// per 8-weight block from the NQRT4 stream (the 31-bit hash and two exact E8 searches), about
// 200 from resolved blocks (the hash and little else).
#include "nq_linear_common.hip.h"

#include <math.h>

#ifdef NQ_PHASE_STAMPS
// Measuring builds only: lane 0 of workgroup (0, 0) of the vector-unit kernel leaves the 100 MHz
// wall clock at its phase boundaries (start, first requests issued, first block decoded, loop
// done, lane sums in LDS, behind the barrier, output stored).
namespace nq { __device__ unsigned long long g_gemv_stamps[16]; }
#define NQ_GEMV_STAMP(i) do { if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) nq::g_gemv_stamps[i] = wall_clock64(); } while (0)
extern "C" int nq_debug_gemv_stamps(unsigned long long *out16) {
    if (hipDeviceSynchronize() != hipSuccess) return NQ_ERR_LAUNCH;
    return hipMemcpyFromSymbol(out16, HIP_SYMBOL(nq::g_gemv_stamps), 16 * sizeof(unsigned long long)) == hipSuccess
               ? NQ_OK : NQ_ERR_LAUNCH;
}
#else
#define NQ_GEMV_STAMP(i) do { } while (0)
#endif

namespace nq {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / 64;
constexpr int kGemvMaxRows = 8;

// kResolved: the weight comes as resolved blocks (w_words = 32-bit words, w_tails = 16-bit
// words, see nq_e8.hip.h) instead of NQRT4 code words and beta bytes.
// R: output channels per workgroup.  A lane decodes block b of all R channels against one
// load of the M activation blocks, and the R weight loads of a step are issued together.
// The work of one workgroup: channels group * R .. + R of one weight, K slice `slice`.
template <int M, int R, bool kResolved>
__device__ __forceinline__ void
gemv_rows(const uint4 *__restrict__ act,          // decoded BF16 [m_rows][K / 8] blocks
          const uint32_t *__restrict__ w_words, const uint16_t *__restrict__ w_tails,
          const uint8_t *__restrict__ w_beta_ids,
          const float *__restrict__ w_norms, const float *__restrict__ w_betas,
          int m_rows, int k_size, int n_size, int k_slice, int group, int slice,
          uint32_t seed_plus_offset, float sqrt_k, float *__restrict__ out_f32,
          uint16_t *__restrict__ out_bf16) {
    __shared__ float partial[kGemvWaves * 4][R][M];        // one entry per 16-lane row of every wavefront
    NQ_GEMV_STAMP(0);
    const int tid = threadIdx.x, lane = tid & 63;
    const int blocks_per_row = k_size >> 3;
    const int slice_blocks = k_slice >> 3;
    const int slice_first_block = slice * slice_blocks;
    const float wbeta[4] = {w_betas[0], w_betas[1], w_betas[2], w_betas[3]};
    const int n0 = group * R;

    float acc[R][M], wscale[R];
    ResolvedScales scaled_beta[R];
    int64_t row_first_block[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int n = n0 + r < n_size ? n0 + r : n_size - 1;       // channels past the end repeat the last one
        const float unit = w_norms[n] / sqrt_k;
        wscale[r] = kResolved ? unit * kResolvedUnit : unit;
        scaled_beta[r] = resolved_scales(wbeta, wscale[r]);
        row_first_block[r] = (int64_t)n * blocks_per_row + slice_first_block;
#pragma unroll
        for (int m = 0; m < M; m++) acc[r][m] = 0.0f;
    }

    // the operands of a step are requested one step ahead: a long row (down_proj: four steps)
    // waits for memory once, not once per step
    uint32_t word_next[R], side_next[R];
    uint4 a_next[M];
#pragma unroll
    for (int r = 0; r < R; r++) { word_next[r] = 0u; side_next[r] = 0u; }
#pragma unroll
    for (int m = 0; m < M; m++) a_next[m] = make_uint4(0, 0, 0, 0);
    if (tid < slice_blocks) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int64_t g = row_first_block[r] + tid;
            word_next[r] = w_words[g];
            side_next[r] = kResolved ? (uint32_t)w_tails[g] : (uint32_t)w_beta_ids[g >> 2];
        }
#pragma unroll
        for (int m = 0; m < M; m++)
            if (m < m_rows) a_next[m] = act[(int64_t)m * blocks_per_row + slice_first_block + tid];
    }
    NQ_GEMV_STAMP(1);
    for (int b = tid; b < slice_blocks; b += kGemvThreads) {
        uint32_t word[R], side[R];
        uint4 a[M];
#pragma unroll
        for (int r = 0; r < R; r++) { word[r] = word_next[r]; side[r] = side_next[r]; }
#pragma unroll
        for (int m = 0; m < M; m++) a[m] = a_next[m];
        const int ahead = b + kGemvThreads;
        if (ahead < slice_blocks) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int64_t g = row_first_block[r] + ahead;
                word_next[r] = w_words[g];
                side_next[r] = kResolved ? (uint32_t)w_tails[g] : (uint32_t)w_beta_ids[g >> 2];
            }
#pragma unroll
            for (int m = 0; m < M; m++)
                if (m < m_rows) a_next[m] = act[(int64_t)m * blocks_per_row + slice_first_block + ahead];
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int64_t g = row_first_block[r] + b;
            float v[8];
            if (kResolved) {
                decode_resolved(word[r], side[r], seed_plus_offset + (uint32_t)g * 8u,
                                resolved_scale(scaled_beta[r], word[r]), v);
            } else {
                decode_codeword<true>(word[r], 14.0f, seed_plus_offset + (uint32_t)g * 8u, v);
                const float scale = wbeta[(side[r] >> (2 * (g & 3))) & 3] * wscale[r];
#pragma unroll
                for (int j = 0; j < 8; j++) v[j] = v[j] * scale;
            }
            bf16x2 w[4];
#pragma unroll
            for (int j = 0; j < 4; j++) w[j] = pack_bf16x2(v[2 * j], v[2 * j + 1]);
#pragma unroll
            for (int m = 0; m < M; m++) {
                acc[r][m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a[m].x), w[0], acc[r][m], false);
                acc[r][m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a[m].y), w[1], acc[r][m], false);
                acc[r][m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a[m].z), w[2], acc[r][m], false);
                acc[r][m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a[m].w), w[3], acc[r][m], false);
            }
        }
#ifdef NQ_PHASE_STAMPS
        if (b == tid) { asm volatile("" :: "v"(acc[0][0])); NQ_GEMV_STAMP(2); }
#endif
    }
    NQ_GEMV_STAMP(3);
    // sums over the 16 lanes of every row with register-only lane exchanges (fixed order)
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int m = 0; m < M; m++) {
            const float v = row16_sum(acc[r][m]);
            if ((lane & 15) == 0) partial[tid >> 4][r][m] = v;
        }
    }
    NQ_GEMV_STAMP(4);
    __syncthreads();
    NQ_GEMV_STAMP(5);
    // row partials in index order
    if (tid < R * M) {
        const int r = tid / M, m = tid - r * M;
        const int n = n0 + r;
        if (n < n_size && m < m_rows) {
            float total = partial[0][r][m];
#pragma unroll
            for (int w = 1; w < kGemvWaves * 4; w++) total = total + partial[w][r][m];
            if (out_f32)
                out_f32[((int64_t)slice * m_rows + m) * n_size + n] = total;
            else
                out_bf16[(int64_t)m * n_size + n] = f32_to_bf16(total);
        }
    }
    NQ_GEMV_STAMP(6);
}

template <int M, int R, bool kResolved>
__global__ void __launch_bounds__(kGemvThreads)
w4a4_gemv_kernel(const uint4 *__restrict__ act, const uint32_t *__restrict__ w_words,
                 const uint16_t *__restrict__ w_tails, const uint8_t *__restrict__ w_beta_ids,
                 const float *__restrict__ w_norms, const float *__restrict__ w_betas,
                 int m_rows, int k_size, int n_size, int k_slice, uint32_t seed_plus_offset, float sqrt_k,
                 float *__restrict__ out_f32, uint16_t *__restrict__ out_bf16) {
    gemv_rows<M, R, kResolved>(act, w_words, w_tails, w_beta_ids, w_norms, w_betas, m_rows, k_size, n_size,
                               k_slice, blockIdx.x, blockIdx.y, seed_plus_offset, sqrt_k, out_f32, out_bf16);
}

template <int M, int R>
__global__ void __launch_bounds__(kGemvThreads)
w4a4_gemv_grouped_kernel(const uint4 *__restrict__ act, GemvWeights w, int m_rows, int k_size, float sqrt_k,
                         int out_is_f32) {
    int which = 0;
#pragma unroll
    for (int i = 1; i < kGemvMaxGroup; i++)
        if (i < w.count && (int)blockIdx.x >= w.first_group[i]) which = i;
    gemv_rows<M, R, true>(act, w.words[which], w.tails[which], nullptr, w.norms[which], w.betas[which], m_rows,
                          k_size, w.n[which], k_size, (int)blockIdx.x - w.first_group[which], 0,
                          w.seed_plus_offset[which], sqrt_k, out_is_f32 ? (float *)w.out[which] : nullptr,
                          out_is_f32 ? nullptr : (uint16_t *)w.out[which]);
}

// Five to sixteen tokens: the dot products move to the matrix cores.  A decoded E8 block is
// exactly one lane's A fragment of v_mfma_f32_16x16x32_bf16 (lane l: channel l % 16, eight
// consecutive k), so a wavefront that decodes 16 channels x 4 blocks multiplies them by the
// matching activation fragment (lane l: token l % 16, the same eight k) with no exchange, no
// LDS and no per-token work on the vector units.  A workgroup owns 16 channels; its wavefronts
// (up to 16) take super-steps of 128 k in turn and each lane reads 16 contiguous bytes of words,
// 8 of tails and 64 of activation per super-step, requested one super-step ahead.  Partial
// tiles meet in LDS and are added in wavefront order.  (The 4 x 4 x 4 block instruction would
// allow four channels per workgroup, but issues at a quarter of this one's rate.)
constexpr int kMfmaGemvMaxWaves = 16;

// R: K ranges per tile.  With R = 1 the 16 rows of the A operand are 16 channels.  Narrow
// weights would then leave part of the chip without a tile, so with R = 2 the rows are 8
// channels times two interleaved ranges of 128 k: a super-step spans 128 R k, a lane still decodes
// four consecutive blocks of its (channel, range), and every decoded block goes through R
// instructions, the r-th with the activation fragment of range r into an accumulator of its own:
// in accumulator r only the rows of range r have met their own k, and only those are taken at the
// end, where the rows of a channel are added.  (Zeroing the rows of the other ranges in the A
// operand instead cost eight selects per block on the vector units, which are this kernel's limit.)
template <int R>
__global__ void __launch_bounds__(kMfmaGemvMaxWaves * 64)
w4a4_gemv_mfma_kernel(const uint4 *__restrict__ act, GemvWeights w, int m_rows, int k_size, float sqrt_k,
                      int out_is_f32) {
    constexpr int kChannels = 16 / R;
    __shared__ float part[kMfmaGemvMaxWaves][256];
    int which = 0;
#pragma unroll
    for (int i = 1; i < kGemvMaxGroup; i++)
        if (i < w.count && (int)blockIdx.x >= w.first_group[i]) which = i;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const int n_size = w.n[which], n0 = ((int)blockIdx.x - w.first_group[which]) * kChannels;
    const int column = lane & 15, quarter = lane >> 4;
    const int range = column / kChannels;                                   // of this lane's A rows
    const int blocks_per_row = k_size >> 3, super_steps = k_size / (128 * R);
    const int n = n0 + column % kChannels < n_size ? n0 + column % kChannels : n_size - 1;   // channels past the end repeat the last one
    const float wscale = (w.norms[which][n] / sqrt_k) * kResolvedUnit;
    const float *betas = w.betas[which];
    const float wbeta[4] = {betas[0], betas[1], betas[2], betas[3]};
    const ResolvedScales scaled_beta = resolved_scales(wbeta, wscale);
    const uint32_t seed_plus_offset = w.seed_plus_offset[which];
    const int64_t row_first = (int64_t)n * blocks_per_row + 16 * range + 4 * quarter;
    const uint32_t *words = w.words[which];
    const uint16_t *tails = w.tails[which];
    const bool has_token = column < m_rows;
    const uint4 *act_row = act + (int64_t)(has_token ? column : 0) * blocks_per_row + 4 * quarter;
    const uint4 zero = make_uint4(0, 0, 0, 0);

    // acc[r]: the products with the activation of range r.  Only the rows of range r are meant in it
    // (a row of the other range has met the wrong k), and only those are read at the end.
    floatx4 acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    uint4 word_next = zero, b_next[R][4];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int t = 0; t < 4; t++) b_next[r][t] = zero;
    uint2 tail_next = make_uint2(0, 0);
    if (wave < super_steps) {
        word_next = *reinterpret_cast<const uint4 *>(words + row_first + 16 * R * wave);
        tail_next = *reinterpret_cast<const uint2 *>(tails + row_first + 16 * R * wave);
        if (has_token) {
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int t = 0; t < 4; t++) b_next[r][t] = act_row[16 * (R * wave + r) + t];
        }
    }
    for (int ss = wave; ss < super_steps; ss += waves) {
        const uint4 word4 = word_next;
        const uint2 tail2 = tail_next;
        uint4 b[R][4];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int t = 0; t < 4; t++) b[r][t] = b_next[r][t];
        if (ss + waves < super_steps) {
            word_next = *reinterpret_cast<const uint4 *>(words + row_first + 16 * R * (ss + waves));
            tail_next = *reinterpret_cast<const uint2 *>(tails + row_first + 16 * R * (ss + waves));
            if (has_token) {
#pragma unroll
                for (int r = 0; r < R; r++)
#pragma unroll
                    for (int t = 0; t < 4; t++) b_next[r][t] = act_row[16 * (R * (ss + waves) + r) + t];
            }
        }
        const uint32_t word[4] = {word4.x, word4.y, word4.z, word4.w};
        const uint32_t tail[4] = {tail2.x & 0xffffu, tail2.x >> 16, tail2.y & 0xffffu, tail2.y >> 16};
        const uint32_t first_counter = seed_plus_offset + (uint32_t)(row_first + 16 * R * ss) * 8u;
        const auto multiply = [&](int t, const float (&v)[8]) {
            const bf16x2 h0 = pack_bf16x2(v[0], v[1]), h1 = pack_bf16x2(v[2], v[3]);
            const bf16x2 h2 = pack_bf16x2(v[4], v[5]), h3 = pack_bf16x2(v[6], v[7]);
            const uint4 a = make_uint4(__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1),
                                       __builtin_bit_cast(uint32_t, h2), __builtin_bit_cast(uint32_t, h3));
#pragma unroll
            for (int r = 0; r < R; r++)
                acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                                 __builtin_bit_cast(bf16x8, b[r][t]), acc[r], 0, 0, 0);
        };
        // R = 1: the dither parts of two neighbouring blocks at a time (three aligned groups of counters
        // instead of four); R = 2 has no registers to spare for that
        if constexpr (R == 1) {
#pragma unroll
            for (int half = 0; half < 2; half++) {
                uint32_t bits[2][8];
                resolved_dither_bits_run<2>(first_counter + 16u * half, bits);
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const int t = 2 * half + i;
                    float v[8];
                    resolved_apply(word[t], tail[t], bits[i], resolved_scale(scaled_beta, word[t]), v);
                    multiply(t, v);
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < 4; t++) {
                float v[8];
                decode_resolved(word[t], tail[t], first_counter + 8u * t, resolved_scale(scaled_beta, word[t]), v);
                multiply(t, v);
            }
        }
    }
    // accumulator i of lane l: A row 4 (l / 16) + i = (range, channel), token l % 16; the row's own
    // range is (4 (l / 16) + i) / kChannels, the same for the lane's four rows
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float mine = acc[0][i];
#pragma unroll
        for (int r = 1; r < R; r++) mine = (4 * quarter) / kChannels == r ? acc[r][i] : mine;
        part[wave][(4 * quarter + i) * 16 + column] = mine;
    }
    __syncthreads();
    if (tid < kChannels * 16) {
        const int channel = tid >> 4, token = tid & 15;
        if (n0 + channel < n_size && token < m_rows) {
            float total = 0.0f;
            for (int p = 0; p < waves; p++)
#pragma unroll
                for (int r = 0; r < R; r++) total = total + part[p][(r * kChannels + channel) * 16 + token];
            const int64_t at = (int64_t)token * n_size + n0 + channel;
            if (out_is_f32) reinterpret_cast<float *>(w.out[which])[at] = total;
            else reinterpret_cast<uint16_t *>(w.out[which])[at] = f32_to_bf16(total);
        }
    }
}

// One lane per weight block: run the exact decode once and keep the lattice point it implies.
__global__ void __launch_bounds__(256)
resolve_weight_kernel(const uint32_t *__restrict__ w_codes, const uint8_t *__restrict__ w_beta_ids,
                      int64_t blocks, uint32_t seed_plus_offset, uint32_t *__restrict__ words,
                      uint16_t *__restrict__ tails, int32_t *__restrict__ out_of_range) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= blocks) return;
    const uint32_t beta_id = ((uint32_t)w_beta_ids[g >> 2] >> (2 * (g & 3))) & 3u;
    uint32_t lo, hi;
    const bool ok = resolve_codeword(w_codes[g], seed_plus_offset + (uint32_t)g * 8u, beta_id, lo, hi);
    words[g] = lo;
    tails[g] = (uint16_t)hi;
    if (!ok) atomicAdd(out_of_range, 1);
}

}  // namespace nq

extern "C" int nq_w4a4_resolve_weight(const uint8_t *w_codes_dev, const uint8_t *w_beta_ids_dev, int64_t rows,
                                      int64_t k, int64_t weight_offset, int64_t weight_seed,
                                      uint32_t *words_dev, uint16_t *tails_dev, int32_t *out_of_range_dev,
                                      void *stream) {
    NQ_REQUIRE(rows >= 1 && k >= 32 && k % 32 == 0, NQ_ERR_SHAPE,
               "nq_w4a4_resolve_weight: rows must be positive and K a positive multiple of 32");
    NQ_REQUIRE(w_codes_dev && w_beta_ids_dev && words_dev && tails_dev && out_of_range_dev, NQ_ERR_ARGUMENT,
               "nq_w4a4_resolve_weight: null pointer");
    NQ_REQUIRE(nq::aligned(w_codes_dev, 4) && nq::aligned(words_dev, 4) && nq::aligned(tails_dev, 2) &&
                   nq::aligned(out_of_range_dev, 4),
               NQ_ERR_ARGUMENT, "nq_w4a4_resolve_weight: misaligned pointer");
    NQ_REQUIRE(weight_seed >= 0 && weight_seed < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
               "nq_w4a4_resolve_weight: seed must be in [0, 2**31)");
    const int64_t blocks = rows * (k / 8);
    NQ_REQUIRE(weight_offset >= 0 && weight_offset + blocks <= ((int64_t)1 << 28), NQ_ERR_SHAPE,
               "nq_w4a4_resolve_weight: block range exceeds the stateless dither counter space");
    const uint32_t seed_plus_offset = (uint32_t)((uint64_t)weight_seed + (uint64_t)weight_offset * 8u);
    hipLaunchKernelGGL(nq::resolve_weight_kernel, dim3((unsigned)((blocks + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, reinterpret_cast<const uint32_t *>(w_codes_dev), w_beta_ids_dev,
                       blocks, seed_plus_offset, words_dev, tails_dev, out_of_range_dev);
    return nq::check_launch("nq_w4a4_resolve_weight");
}

namespace {

// The matrix-core kernel (resolved weights, 16-byte aligned streams) works in tiles of 16 / R
// channels: R = 2 interleaved K ranges (K a multiple of 256) when 16-channel tiles would number
// fewer than 192, else R = 1.  (R = 4 was measured at more than twice the time of R = 2.)  Above eight rows it is the only decode kernel; below, it is taken
// from two rows on (NQ_MFMA_FROM_ROWS), where it saves the per-token vector work (us, vector units /
// matrix cores, at 3 and 4 rows: q/k/v 7.5, 7.5 / 7.0, 7.1; down_proj 12.2, 12.1 / 11.1, 11.2; behind
// the encoder in one launch: q/k/v 11.0, 11.1 / 9.6, 9.7; o_proj 10.6, 10.8 / 9.5, 9.6; down_proj 18.4,
// 18.5 / 17.3, 17.9; at two rows the kernels alone are even, and a 1B decode step of two rows takes
// 1.235 ms on the vector units and 1.195 on the matrix cores; at one row 1.166 and 1.183), and for any
// row count when even
// R = 1 gives 512 tiles (gate/up), where it also beats the vector-unit kernel's reductions
// (measured: 25.0 against 26.2 us at one row).
constexpr int kMfmaGemvMaxRows = 16;

int mfma_gemv_ranges(int k, int64_t total_n) {
    return (total_n < 16 * 192 && k % 256 == 0) ? 2 : 1;
}

bool takes_mfma_gemv(int m, int k, int64_t total_n, bool resolved) {
    if (!resolved || k % 128 != 0 || m > kMfmaGemvMaxRows) return false;
    return m >= NQ_MFMA_FROM_ROWS || total_n >= 16 * 512;
}

int launch_mfma_gemv(const void *act, const nq::GemvWeights &w, int ranges, int groups, int m, int k,
                     int out_is_f32, hipStream_t stream) {
    // One range: two or more super-steps of 128 k per wavefront, so that the requests of the next one
    // hide behind a decode; between 4 wavefronts (the last stage wants 256 lanes) and 16.  Two ranges:
    // exactly half as many wavefronts as the same K takes in one range (the last stage wants 128
    // lanes).  Wavefront v of the two-range launch then gathers, in its accumulator r, the pieces of
    // 128 k that wavefront 2 v + r of the one-range launch gathers, in the same order, and the last
    // stage adds the accumulators in that same wavefront order: a weight gives the same bits alone
    // (two ranges) and inside a group (one range), for every K.  (down_proj at 8 rows, two ranges:
    // 12.1 us with 16 wavefronts, 11.8 to 11.9 with 8, 13.2 with 4.)
    const int pieces = k / 128;
    int waves = pieces / 2 < nq::kMfmaGemvMaxWaves ? pieces / 2 : nq::kMfmaGemvMaxWaves;
    if (waves < 4) waves = 4;
    if (ranges == 2) waves /= 2;
    const uint4 *a = reinterpret_cast<const uint4 *>(act);
    const float sqrt_k = (float)sqrt((double)k);
    const dim3 grid((unsigned)groups), block(64 * waves);
    if (ranges == 1) hipLaunchKernelGGL(nq::w4a4_gemv_mfma_kernel<1>, grid, block, 0, stream, a, w, m, k, sqrt_k, out_is_f32);
    else hipLaunchKernelGGL(nq::w4a4_gemv_mfma_kernel<2>, grid, block, 0, stream, a, w, m, k, sqrt_k, out_is_f32);
    return nq::check_launch("nq_w4a4_gemv (matrix cores)");
}

int m_tile_of(int m) { return m == 1 ? 1 : (m == 2 ? 2 : (m <= 4 ? 4 : 8)); }

// A workgroup consumes 2048 K-elements per step.  Only long-K shapes too narrow to give
// every CU a workgroup are split; the others finish in one kernel.
int pick_split(int k, int n, int requested) {
    if (requested > 0) return requested;
    int split = 1;
    while (split < 8 && (k / (split * 2)) % 32 == 0 && (int64_t)n * split < 1024 && k / (split * 2) >= 2048)
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
                            const uint8_t *w_beta_ids_dev, const uint32_t *w_resolved_words_dev,
                            const uint16_t *w_resolved_tails_dev, const float *w_norms_dev,
                            const float *w_betas_dev, int m, int k, int n, int64_t weight_offset,
                            int64_t weight_seed, int split_k, void *out_dev, int out_dtype,
                            void *workspace_dev, size_t workspace_bytes, void *stream) {
    const bool mfma = takes_mfma_gemv(m, k, n, w_resolved_words_dev != nullptr) && split_k <= 1 &&
                      nq::aligned(w_resolved_words_dev, 16) && nq::aligned(w_resolved_tails_dev, 8);
    NQ_REQUIRE(m >= 1 && (m <= 8 || mfma), NQ_ERR_SHAPE,
               "nq_w4a4_gemv: M = %d is outside [1, 8] (up to 16 with resolved weights and K a multiple of 128)", m);
    NQ_REQUIRE(k >= 32 && k % 32 == 0, NQ_ERR_SHAPE, "nq_w4a4_gemv: K = %d must be a positive multiple of 32", k);
    NQ_REQUIRE(n >= 1, NQ_ERR_SHAPE, "nq_w4a4_gemv: N must be positive");
    NQ_REQUIRE(split_k == 0 || split_k == 1 || split_k == 2 || split_k == 4 || split_k == 8,
               NQ_ERR_ARGUMENT, "nq_w4a4_gemv: split_k must be 0, 1, 2, 4 or 8");
    NQ_REQUIRE(out_dtype == NQ_F32 || out_dtype == NQ_BF16, NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv: output dtype tag %d is not F32 or BF16", out_dtype);
    const bool resolved = w_resolved_words_dev != nullptr;
    NQ_REQUIRE(w_norms_dev && w_betas_dev && out_dev, NQ_ERR_ARGUMENT, "nq_w4a4_gemv: null pointer");
    NQ_REQUIRE(resolved ? w_resolved_tails_dev != nullptr : (w_codes_dev && w_beta_ids_dev), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv: neither packed nor resolved weight streams given");
    NQ_REQUIRE(act_decoded_dev || (act_codes_dev && act_beta_ids_dev && act_norms_dev && act_betas_dev),
               NQ_ERR_ARGUMENT, "nq_w4a4_gemv: neither packed nor decoded activation given");
    NQ_REQUIRE(nq::aligned(w_codes_dev, 4) && (!act_codes_dev || nq::aligned(act_codes_dev, 4)) &&
                   (!act_decoded_dev || nq::aligned(act_decoded_dev, 16)) &&
                   nq::aligned(w_resolved_words_dev, 4) && nq::aligned(w_resolved_tails_dev, 2),
               NQ_ERR_ARGUMENT, "nq_w4a4_gemv: code streams need 4-byte, decoded activation 16-byte alignment");
    NQ_REQUIRE(weight_seed >= 0 && weight_seed < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv: seed must be in [0, 2**31)");
    NQ_REQUIRE(weight_offset >= 0 && weight_offset + (int64_t)n * (k / 8) <= ((int64_t)1 << 28),
               NQ_ERR_SHAPE, "nq_w4a4_gemv: block range exceeds the stateless dither counter space");
    const int split = mfma ? 1 : pick_split(k, n, split_k);
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
    if (mfma) {
        nq::GemvWeights one{};
        one.count = 1;
        one.words[0] = w_resolved_words_dev;
        one.tails[0] = w_resolved_tails_dev;
        one.norms[0] = w_norms_dev;
        one.betas[0] = w_betas_dev;
        one.out[0] = out_dev;
        one.n[0] = n;
        one.first_group[0] = 0;
        one.seed_plus_offset[0] = (uint32_t)((uint64_t)weight_seed + (uint64_t)weight_offset * 8u);
        const int ranges = mfma_gemv_ranges(k, n), channels = 16 / ranges;
        return launch_mfma_gemv(act, one, ranges, (n + channels - 1) / channels, m, k, out_dtype == NQ_F32, s);
    }

    const int k_slice = k / split;
    // few rows per workgroup keeps many short wavefronts in flight on every SIMD
    const int rows_per_wg = (resolved && (int64_t)n * split >= 8192) ? 4 : 2;
    const dim3 grid((unsigned)((n + rows_per_wg - 1) / rows_per_wg), (unsigned)split);
    const uint32_t seed_plus_offset = (uint32_t)((uint64_t)weight_seed + (uint64_t)weight_offset * 8u);
    float *target_f32 = split > 1 ? partials : (out_dtype == NQ_F32 ? (float *)out_dev : nullptr);
    uint16_t *target_bf16 = (split > 1 || out_dtype == NQ_F32) ? nullptr : (uint16_t *)out_dev;
    const uint32_t *wc = resolved ? w_resolved_words_dev : reinterpret_cast<const uint32_t *>(w_codes_dev);
#define NQ_LAUNCH_GEMV_AS(MT, ROWS, RESOLVED)                                                       \
    hipLaunchKernelGGL((nq::w4a4_gemv_kernel<MT, ROWS, RESOLVED>), grid, dim3(nq::kGemvThreads), 0, \
                       s, act, wc, w_resolved_tails_dev, w_beta_ids_dev, w_norms_dev, w_betas_dev,  \
                       m, k, n, k_slice, seed_plus_offset, sqrt_k, target_f32, target_bf16)
#define NQ_LAUNCH_GEMV(MT)                                                                          \
    do {                                                                                            \
        if (!resolved) NQ_LAUNCH_GEMV_AS(MT, 2, false);                                             \
        else if (rows_per_wg == 4) NQ_LAUNCH_GEMV_AS(MT, 4, true);                                  \
        else NQ_LAUNCH_GEMV_AS(MT, 2, true);                                                        \
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

extern "C" int nq_w4a4_gemv_grouped(const void *act_decoded_dev, int count, const uint32_t *const *w_resolved_words_dev,
                                    const uint16_t *const *w_resolved_tails_dev, const float *const *w_norms_dev,
                                    const float *const *w_betas_dev, const int *n, const int64_t *weight_offsets,
                                    const int64_t *weight_seeds, void *const *out_dev, int m, int k, int out_dtype,
                                    void *stream) {
    NQ_REQUIRE(count >= 1 && count <= nq::kGemvMaxGroup, NQ_ERR_SHAPE,
               "nq_w4a4_gemv_grouped: between 1 and %d weights per launch", nq::kGemvMaxGroup);
    int64_t total_n = 0;
    for (int i = 0; n && i < count; i++) total_n += n[i];
    bool mfma = takes_mfma_gemv(m, k, total_n, true);
    for (int i = 0; mfma && i < count; i++)
        mfma = w_resolved_words_dev && w_resolved_tails_dev && nq::aligned(w_resolved_words_dev[i], 16) &&
               nq::aligned(w_resolved_tails_dev[i], 8);
    NQ_REQUIRE(m >= 1 && (m <= 8 || mfma), NQ_ERR_SHAPE,
               "nq_w4a4_gemv_grouped: M = %d is outside [1, 8] (up to 16 with K a multiple of 128)", m);
    NQ_REQUIRE(k >= 32 && k % 32 == 0, NQ_ERR_SHAPE, "nq_w4a4_gemv_grouped: K = %d must be a positive multiple of 32", k);
    NQ_REQUIRE(out_dtype == NQ_F32 || out_dtype == NQ_BF16, NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv_grouped: output dtype tag %d is not F32 or BF16", out_dtype);
    NQ_REQUIRE(act_decoded_dev && nq::aligned(act_decoded_dev, 16), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv_grouped: needs the decoded BF16 activation, 16-byte aligned");
    NQ_REQUIRE(w_resolved_words_dev && w_resolved_tails_dev && w_norms_dev && w_betas_dev && n && weight_offsets &&
                   weight_seeds && out_dev, NQ_ERR_ARGUMENT, "nq_w4a4_gemv_grouped: null argument array");
    nq::GemvWeights w{};
    w.count = count;
    const int ranges = mfma ? mfma_gemv_ranges(k, total_n) : 1;
    const int rows_per_wg = mfma ? 16 / ranges : (total_n >= 8192 ? 4 : 2);
    int groups = 0;
    for (int i = 0; i < count; i++) {
        NQ_REQUIRE(n[i] >= 1, NQ_ERR_SHAPE, "nq_w4a4_gemv_grouped: N must be positive");
        NQ_REQUIRE(w_resolved_words_dev[i] && w_resolved_tails_dev[i] && w_norms_dev[i] && w_betas_dev[i] && out_dev[i],
                   NQ_ERR_ARGUMENT, "nq_w4a4_gemv_grouped: null pointer in weight %d", i);
        NQ_REQUIRE(nq::aligned(w_resolved_words_dev[i], 4) && nq::aligned(w_resolved_tails_dev[i], 2), NQ_ERR_ARGUMENT,
                   "nq_w4a4_gemv_grouped: misaligned resolved streams in weight %d", i);
        NQ_REQUIRE(weight_seeds[i] >= 0 && weight_seeds[i] < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
                   "nq_w4a4_gemv_grouped: seed must be in [0, 2**31)");
        NQ_REQUIRE(weight_offsets[i] >= 0 && weight_offsets[i] + (int64_t)n[i] * (k / 8) <= ((int64_t)1 << 28),
                   NQ_ERR_SHAPE, "nq_w4a4_gemv_grouped: block range exceeds the stateless dither counter space");
        w.words[i] = w_resolved_words_dev[i];
        w.tails[i] = w_resolved_tails_dev[i];
        w.norms[i] = w_norms_dev[i];
        w.betas[i] = w_betas_dev[i];
        w.out[i] = out_dev[i];
        w.n[i] = n[i];
        w.first_group[i] = groups;
        w.seed_plus_offset[i] = (uint32_t)((uint64_t)weight_seeds[i] + (uint64_t)weight_offsets[i] * 8u);
        groups += (n[i] + rows_per_wg - 1) / rows_per_wg;
    }
    const float sqrt_k = (float)sqrt((double)k);
    const uint4 *act = reinterpret_cast<const uint4 *>(act_decoded_dev);
    const int out_is_f32 = out_dtype == NQ_F32;
    hipStream_t s = (hipStream_t)stream;
    if (mfma) return launch_mfma_gemv(act_decoded_dev, w, ranges, groups, m, k, out_is_f32, s);
#define NQ_LAUNCH_GROUPED(MT)                                                                        \
    do {                                                                                             \
        if (rows_per_wg == 4)                                                                        \
            hipLaunchKernelGGL((nq::w4a4_gemv_grouped_kernel<MT, 4>), dim3((unsigned)groups),        \
                               dim3(nq::kGemvThreads), 0, s, act, w, m, k, sqrt_k, out_is_f32);      \
        else                                                                                         \
            hipLaunchKernelGGL((nq::w4a4_gemv_grouped_kernel<MT, 2>), dim3((unsigned)groups),        \
                               dim3(nq::kGemvThreads), 0, s, act, w, m, k, sqrt_k, out_is_f32);      \
    } while (0)
    switch (m_tile_of(m)) {
        case 1: NQ_LAUNCH_GROUPED(1); break;
        case 2: NQ_LAUNCH_GROUPED(2); break;
        case 4: NQ_LAUNCH_GROUPED(4); break;
        default: NQ_LAUNCH_GROUPED(8); break;
    }
#undef NQ_LAUNCH_GROUPED
    return nq::check_launch("nq_w4a4_gemv_grouped");
}

// ---------------------------------------------------------------------------------------
// nq_w4a4_gemv for callers that cannot allocate device memory: the workspace (decoded
// activation, split-K partials) is a fixed array in the library's own device image.
namespace {

constexpr size_t kStaticScratchBytes = (size_t)4 << 20;
constexpr int kStaticScratchMaxDevices = 64;

// One copy per GPU the library's code object is loaded on, at that GPU's own address.  In
// host code the name is only a handle for hipGetSymbolAddress: it is never passed to a kernel.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device, looked up once per device.  The lookup is a
// runtime call that a stream under capture must not see: while `stream` is capturing only an
// address that is already known is handed out (nq_w4a4_gemv_static_init makes it known).
int static_scratch_address(void **address, hipStream_t stream, bool may_be_capturing) {
    static void *known[kStaticScratchMaxDevices] = {nullptr};
    int device = -1;
    hipError_t status = hipGetDevice(&device);
    if (status != hipSuccess)
        return nq::fail(NQ_ERR_LAUNCH, "nq_w4a4_gemv_static: hipGetDevice: %s", hipGetErrorString(status));
    NQ_REQUIRE(device >= 0 && device < kStaticScratchMaxDevices, NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv_static: device ordinal %d is outside [0, %d)", device, kStaticScratchMaxDevices);
    void *pointer = __atomic_load_n(&known[device], __ATOMIC_ACQUIRE);
    if (!pointer) {
        if (may_be_capturing) {
            hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
            status = hipStreamIsCapturing(stream, &capture);
            if (status != hipSuccess)
                return nq::fail(NQ_ERR_LAUNCH, "nq_w4a4_gemv_static: hipStreamIsCapturing: %s", hipGetErrorString(status));
            NQ_REQUIRE(capture == hipStreamCaptureStatusNone, NQ_ERR_ARGUMENT,
                       "nq_w4a4_gemv_static: first use on device %d inside a stream capture; call "
                       "nq_w4a4_gemv_static_init() on this device before capturing", device);
        }
        status = hipGetSymbolAddress(&pointer, HIP_SYMBOL(scratch));
        if (status != hipSuccess || !pointer)
            return nq::fail(NQ_ERR_LAUNCH, "nq_w4a4_gemv_static: hipGetSymbolAddress(scratch): %s",
                            hipGetErrorString(status));
        __atomic_store_n(&known[device], pointer, __ATOMIC_RELEASE);    // every thread finds the same address
    }
    *address = pointer;
    return NQ_OK;
}

}  // namespace

extern "C" int nq_w4a4_gemv_static_init(void) {
    void *address = nullptr;
    return static_scratch_address(&address, nullptr, false);
}

extern "C" int nq_w4a4_gemv_static(const uint8_t *act_codes_dev, const uint8_t *act_beta_ids_dev,
                                   const float *act_norms_dev, const float *act_betas_dev,
                                   const void *act_decoded_dev, const uint8_t *w_codes_dev,
                                   const uint8_t *w_beta_ids_dev, const uint32_t *w_resolved_words_dev,
                                   const uint16_t *w_resolved_tails_dev, const float *w_norms_dev,
                                   const float *w_betas_dev, int m, int k, int n, int64_t weight_offset,
                                   int64_t weight_seed, int split_k, void *out_dev, int out_dtype, void *stream) {
    NQ_REQUIRE(m >= 1 && m <= 16 && k >= 32 && n >= 1, NQ_ERR_SHAPE,
               "nq_w4a4_gemv_static: M = %d, K = %d, N = %d: M must be in [1, 16], K at least 32, N positive", m, k, n);
    NQ_REQUIRE(split_k == 0 || split_k == 1 || split_k == 2 || split_k == 4 || split_k == 8, NQ_ERR_ARGUMENT,
               "nq_w4a4_gemv_static: split_k must be 0, 1, 2, 4 or 8");
    // what nq_w4a4_gemv will ask of its workspace (a launch on the matrix cores needs less, never more)
    const size_t need = nq_w4a4_gemv_workspace_bytes(m, k, n, split_k, act_decoded_dev != nullptr);
    NQ_REQUIRE(need <= kStaticScratchBytes, NQ_ERR_WORKSPACE,
               "nq_w4a4_gemv_static: M = %d, K = %d, N = %d, split_k = %d needs %zu bytes of scratch; the "
               "built-in buffer holds %zu (use nq_w4a4_gemv with a caller-owned workspace)",
               m, k, n, split_k, need, kStaticScratchBytes);
    void *workspace = nullptr;
    const int status = static_scratch_address(&workspace, (hipStream_t)stream, true);
    if (status != NQ_OK) return status;
    // Every partial sum and every decoded activation value a launch reads was written by that
    // same launch sequence, so what an earlier call left in the buffer needs no clearing.
    return nq_w4a4_gemv(act_codes_dev, act_beta_ids_dev, act_norms_dev, act_betas_dev, act_decoded_dev, w_codes_dev,
                        w_beta_ids_dev, w_resolved_words_dev, w_resolved_tails_dev, w_norms_dev, w_betas_dev, m, k, n,
                        weight_offset, weight_seed, split_k, out_dev, out_dtype, need ? workspace : nullptr,
                        need ? kStaticScratchBytes : 0, stream);
}
