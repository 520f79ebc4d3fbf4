// Packed W4A4 linear for prefill (M >= 9 tokens; any M) on the matrix cores.
//
// y[m, n] = sum_k a[m, k] * w[n, k]: a is the BF16 decode of the NQA4 activation [M, K]
// (emitted by the encoder, or decoded once per call), w is decoded on the fly from the
// NQRT4 stream, products accumulate in FP32 with v_mfma_f32_32x32x16_bf16.
//
// Tiling.  grid = (N / 32, split_k); a workgroup of eight wavefronts owns 32 output
// channels and one K slab and walks it in steps of 128:
//   * decode: lane t decodes one E8 block of the 32 x 128 weight tile (channel t / 16,
//     block t % 16) -- one 32-bit word per lane, 64 contiguous bytes per channel -- and
//     writes its eight BF16 values as one 16-byte LDS entry laid out as the MFMA B fragment
//     (lane l of K-step s holds channel l % 32, k = 16 s + 8 (l / 32) .. + 8).  An E8 block
//     is exactly one lane's fragment, so decoded weights never need a transpose.
//   * multiply: wavefront w owns token tiles w, w + 8, ... of 32 rows; per K-step it reads
//     the B fragment from LDS (one ds_read_b128) and takes its A fragments from registers
//     filled one trip earlier straight from the activation in global memory (L2-resident).
//   * the weight tile is double-buffered in LDS and the loop is software-pipelined: a trip
//     multiplies the previous step while it decodes the current one, with one barrier.
// Every weight block is decoded exactly once per call, whatever M is: the kernel is bound
// by the decode's vector-ALU work, and the matrix cores run in its shadow.
// M is padded up to a multiple of 32 with zero rows inside the kernel (masked loads and
// stores), so ragged M needs no copy; M above 512 is processed in chunks of 512 rows.
// Replaces: run_m16 / run_large_m_staged and the chunk-and-pad wrapper,
// nestquant/runtime/nqrt4_w4a4_mma.cu:124-171, 606-667 and nestquant/runtime/cuda_w4a4_mma.py:450-474.
#include "nq_linear_common.hip.h"

#include <math.h>

namespace nq {

constexpr int kGemmThreads = 512;
constexpr int kGemmWaves = kGemmThreads / 64;
constexpr int kGemmBN = 32;
constexpr int kGemmBK = 128;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// Up to four weights that share an activation (q, k and v; gate and up): one launch takes their
// channels one after the other, a workgroup's 32 channels always inside one weight (every weight but
// the last has a multiple of 32 channels).
constexpr int kGemmMaxGroups = 4;
struct GemmWeights {
    const uint32_t *words[kGemmMaxGroups];        // NQRT4 code words, or resolved words
    const uint16_t *tails[kGemmMaxGroups];        // resolved tails
    const uint8_t *beta_ids[kGemmMaxGroups];
    const float *norms[kGemmMaxGroups];
    const float *betas[kGemmMaxGroups];
    uint16_t *out_bf16[kGemmMaxGroups];           // BF16 [m_rows][channels of the weight], or null
    uint32_t seed_plus_offset[kGemmMaxGroups];
    int end[kGemmMaxGroups];                      // channels of the weights up to and including this one
};

// TILES: token tiles (of 32 rows) per wavefront.  kResolved: the weights come as resolved
// blocks (words / tails, see nq_e8.hip.h) instead of NQRT4 code words and beta bytes.
// FP32 results (partial sums of K slab blockIdx.y, or the output itself) are laid out weight by
// weight: out_f32[(slab * n_total + first channel of the weight) * m_rows + m * channels + n].
// CT: tiles of 32 channels per workgroup.  Every workgroup reads the whole activation of its K slab from
// L2, and those reads are what a launch of many channel tiles waits for (a 128-row gate + up launch: 512
// workgroups x 512 KB); with CT = 2 a decode lane takes two blocks per trip (channels c and c + 32) and a
// multiplying wavefront uses each activation fragment for both tiles, so half as many workgroups read it.
template <int TILES, bool kResolved, int CT = 1>
__global__ void __launch_bounds__(kGemmThreads)
w4a4_gemm_kernel(const uint16_t *__restrict__ act,        // BF16 [m_rows][K]
                 GemmWeights weights, int m_rows, int k_size, int n_total, int k_slab, float sqrt_k,
                 float *__restrict__ out_f32) {
    __shared__ uint4 b_tile[2][CT][kGemmBK / 16][64];      // 2 x CT x 8 K-steps x 64 lanes x 16 B = CT x 16 KiB
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int channel0 = blockIdx.x * (kGemmBN * CT);
    const int group = (channel0 >= weights.end[0]) + (channel0 >= weights.end[1]) + (channel0 >= weights.end[2]);
    const int group_first = group ? weights.end[group - 1] : 0;
    const int n0 = channel0 - group_first, n_size = weights.end[group] - group_first;
    const uint32_t *__restrict__ w_words = weights.words[group];
    const uint16_t *__restrict__ w_tails = weights.tails[group];
    const uint8_t *__restrict__ w_beta_ids = weights.beta_ids[group];
    const float *__restrict__ w_norms = weights.norms[group];
    const float *__restrict__ w_betas = weights.betas[group];
    uint16_t *__restrict__ out_bf16 = weights.out_bf16[group];
    const uint32_t seed_plus_offset = weights.seed_plus_offset[group];
    const int k_begin = blockIdx.y * k_slab;
    const int blocks_per_row = k_size >> 3;

    // decode role: channel n0 + 32 c + tid / 16 of every tile c, block tid % 16 of the current 128-wide step.
    // Channels past the end repeat the last one; their results are never stored.
    const int dec_kb = tid & 15;
    const float wbeta[4] = {w_betas[0], w_betas[1], w_betas[2], w_betas[3]};
    float wscale[CT];
    ResolvedScales scaled_beta[CT];
    int64_t dec_first[CT];
#pragma unroll
    for (int c = 0; c < CT; c++) {
        const int dec_n = n0 + kGemmBN * c + (tid >> 4) < n_size ? n0 + kGemmBN * c + (tid >> 4) : n_size - 1;
        const float unit = w_norms[dec_n] / sqrt_k;
        wscale[c] = kResolved ? unit * kResolvedUnit : unit;
        scaled_beta[c] = resolved_scales(wbeta, wscale[c]);
        dec_first[c] = (int64_t)dec_n * blocks_per_row + (k_begin >> 3) + dec_kb;
    }
    // LDS entry of (K-step kk, fragment lane f): [kk][f ^ (2 (kk % 4) + f / 32)].  Eight neighbouring
    // decode lanes (one channel, blocks 8 i .. 8 i + 7, i.e. four K-steps x the two halves of the
    // fragment) then write eight different 16-byte bank groups, and for the readers the mask is a
    // permutation of the 64 fragment lanes of a K-step (it leaves f / 32 alone).
    const int dec_kk = dec_kb >> 1;
    const int dec_f = (tid >> 4) + 32 * (dec_kb & 1);
    const int dec_entry = dec_f ^ (2 * (dec_kk & 3) + (dec_kb & 1));
    uint4 *dec_slot0 = &b_tile[0][0][dec_kk][dec_entry];
    uint4 *dec_slot1 = &b_tile[1][0][dec_kk][dec_entry];
    constexpr int kTileEntries = (kGemmBK / 16) * 64;

    // multiply role: A fragment rows of this lane, one per owned tile (rows past the end
    // repeat the last one; their results are never stored)
    const uint16_t *a_row[TILES];
#pragma unroll
    for (int t = 0; t < TILES; t++) {
        const int m = (wave + t * kGemmWaves) * 32 + (lane & 31);
        a_row[t] = act + (int64_t)(m < m_rows ? m : m_rows - 1) * k_size + k_begin + 8 * (lane >> 5);
    }
    const bool multiplies = wave * 32 < m_rows;
    floatx16 acc[TILES][CT];
#pragma unroll
    for (int t = 0; t < TILES; t++)
#pragma unroll
        for (int c = 0; c < CT; c++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[t][c][i] = 0.0f;

    // Software pipeline, one barrier per trip: trip s multiplies step s - 1 (weights from
    // LDS, activation fragments requested one trip earlier) while it decodes step s, and
    // requests the code words of step s + 1 and the fragments of step s.
    const int steps = k_slab / kGemmBK;
    uint32_t word_next[CT], side_next[CT];
#pragma unroll
    for (int c = 0; c < CT; c++) {
        word_next[c] = w_words[dec_first[c]];
        side_next[c] = kResolved ? (uint32_t)w_tails[dec_first[c]] : (uint32_t)w_beta_ids[dec_first[c] >> 2];
    }
    uint4 a_next[TILES][kGemmBK / 16];
#pragma unroll
    for (int t = 0; t < TILES; t++)
#pragma unroll
        for (int kk = 0; kk < kGemmBK / 16; kk++) a_next[t][kk] = make_uint4(0, 0, 0, 0);

    for (int s = 0; s <= steps; s++) {
        uint32_t word[CT], side[CT];
#pragma unroll
        for (int c = 0; c < CT; c++) { word[c] = word_next[c]; side[c] = side_next[c]; }
        uint4 a_now[TILES][kGemmBK / 16];
#pragma unroll
        for (int t = 0; t < TILES; t++)
#pragma unroll
            for (int kk = 0; kk < kGemmBK / 16; kk++) a_now[t][kk] = a_next[t][kk];
        int64_t g[CT];
#pragma unroll
        for (int c = 0; c < CT; c++) {
            g[c] = dec_first[c] + (int64_t)s * (kGemmBK / 8);
            if (s + 1 < steps) {
                word_next[c] = w_words[g[c] + kGemmBK / 8];
                side_next[c] = kResolved ? (uint32_t)w_tails[g[c] + kGemmBK / 8] : (uint32_t)w_beta_ids[(g[c] + kGemmBK / 8) >> 2];
            }
        }
        if (s < steps && multiplies) {
#pragma unroll
            for (int t = 0; t < TILES; t++)
#pragma unroll
                for (int kk = 0; kk < kGemmBK / 16; kk++)
                    a_next[t][kk] = *reinterpret_cast<const uint4 *>(a_row[t] + s * kGemmBK + kk * 16);
        }
        if (s > 0 && multiplies) {
#pragma unroll
            for (int kk = 0; kk < kGemmBK / 16; kk++) {
#pragma unroll
                for (int c = 0; c < CT; c++) {
                    const bf16x8 b = __builtin_bit_cast(bf16x8, b_tile[(s - 1) & 1][c][kk][lane ^ (2 * (kk & 3) + (lane >> 5))]);
#pragma unroll
                    for (int t = 0; t < TILES; t++)
                        acc[t][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a_now[t][kk]), b,
                                                                            acc[t][c], 0, 0, 0);
                }
            }
        }
        if (s < steps) {
#pragma unroll
            for (int c = 0; c < CT; c++) {
                float v[8];
                if (kResolved) {
                    decode_resolved(word[c], side[c], seed_plus_offset + (uint32_t)g[c] * 8u,
                                    resolved_scale(scaled_beta[c], word[c]), v);
                } else {
                    decode_codeword<true>(word[c], 14.0f, seed_plus_offset + (uint32_t)g[c] * 8u, v);
                    const float scale = wbeta[(side[c] >> (2 * (g[c] & 3))) & 3] * wscale[c];
#pragma unroll
                    for (int j = 0; j < 8; j++) v[j] = v[j] * scale;
                }
                const bf16x2 h0 = pack_bf16x2(v[0], v[1]), h1 = pack_bf16x2(v[2], v[3]);
                const bf16x2 h2 = pack_bf16x2(v[4], v[5]), h3 = pack_bf16x2(v[6], v[7]);
                ((s & 1) ? dec_slot1 : dec_slot0)[c * kTileEntries] =
                    make_uint4(__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1),
                               __builtin_bit_cast(uint32_t, h2), __builtin_bit_cast(uint32_t, h3));
            }
        }
        __syncthreads();
    }

    // accumulator register r of lane l holds token row (r % 4) + 8 * (r / 4) + 4 * (l / 32)
    // of the tile and channel n0 + l % 32
#pragma unroll
    for (int c = 0; c < CT; c++) {
        const int n = n0 + kGemmBN * c + (lane & 31);
        if (n >= n_size) continue;
#pragma unroll
        for (int t = 0; t < TILES; t++) {
            const int m_base = (wave + t * kGemmWaves) * 32 + 4 * (lane >> 5);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m_base + (r & 3) + 8 * (r >> 2);
                if (m < m_rows) {
                    if (out_f32)
                        out_f32[((int64_t)blockIdx.y * n_total + group_first) * m_rows + (int64_t)m * n_size + n] = acc[t][c][r];
                    else
                        out_bf16[(int64_t)m * n_size + n] = f32_to_bf16(acc[t][c][r]);
                }
            }
        }
    }
}


// The BF16 weight [N][K] the linear kernels multiply by, written out: the same decode, scale and
// rounding as the decode role of the kernel above.  Long prefills decode the weight once with the
// whole chip and multiply with the dense BF16 GEMM.  The packed form: one lane per E8 block.
__global__ void __launch_bounds__(256)
decode_weight_kernel(const uint32_t *__restrict__ w_words, const uint8_t *__restrict__ w_beta_ids,
                     const float *__restrict__ w_norms, const float *__restrict__ w_betas, int64_t blocks,
                     int blocks_per_row, uint32_t seed_plus_offset, float sqrt_k, uint4 *__restrict__ out) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= blocks) return;
    const int64_t row = g / blocks_per_row;
    const uint32_t word = w_words[g];
    const float unit = w_norms[row] / sqrt_k;
    float v[8];
    decode_codeword<true>(word, 14.0f, seed_plus_offset + (uint32_t)g * 8u, v);
    const float scale = w_betas[(w_beta_ids[g >> 2] >> (2 * (g & 3))) & 3] * unit;
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = v[j] * scale;
    const bf16x2 h0 = pack_bf16x2(v[0], v[1]), h1 = pack_bf16x2(v[2], v[3]);
    const bf16x2 h2 = pack_bf16x2(v[4], v[5]), h3 = pack_bf16x2(v[6], v[7]);
    out[g] = make_uint4(__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1),
                        __builtin_bit_cast(uint32_t, h2), __builtin_bit_cast(uint32_t, h3));
}

// The resolved form of the weight, four blocks per lane.  A wavefront takes 256 consecutive blocks,
// lane l the blocks l, 64 + l, 128 + l and 192 + l of them: every load and store instruction of the
// wavefront covers one contiguous stretch, the four word loads of a lane are in flight together and
// the hashes of the next block overlap the stores of the last.  kWholeStretch: the blocks of a row
// are a multiple of 256, so a wavefront's stretch lies in one row and the lane keeps that row's four
// beta scales in registers.
constexpr int kDecodeBlocksPerLane = 4;

template <bool kWholeStretch>
__global__ void __launch_bounds__(256)
decode_resolved_weight_kernel(const uint32_t *__restrict__ w_words, const uint16_t *__restrict__ w_tails,
                              const float *__restrict__ w_norms, const float *__restrict__ w_betas, uint32_t blocks,
                              uint32_t blocks_per_row, uint32_t seed_plus_offset, float sqrt_k,
                              uint4 *__restrict__ out) {
    const uint32_t first = (blockIdx.x * 4u + (threadIdx.x >> 6)) * (64u * kDecodeBlocksPerLane) + (threadIdx.x & 63u);
    if (first >= blocks) return;
    uint32_t word[kDecodeBlocksPerLane], tail[kDecodeBlocksPerLane];
#pragma unroll
    for (int i = 0; i < kDecodeBlocksPerLane; i++) {
        const uint32_t g = first + 64u * i;
        const bool live = g < blocks;
        word[i] = live ? w_words[g] : 0u;
        tail[i] = live ? (uint32_t)w_tails[g] : 0u;
    }
    const float beta[4] = {w_betas[0], w_betas[1], w_betas[2], w_betas[3]};
    ResolvedScales scales = resolved_scales(beta, (w_norms[first / blocks_per_row] / sqrt_k) * kResolvedUnit);
#pragma unroll
    for (int i = 0; i < kDecodeBlocksPerLane; i++) {
        const uint32_t g = first + 64u * i;
        if (g >= blocks) break;
        if (!kWholeStretch && i > 0)
            scales = resolved_scales(beta, (w_norms[g / blocks_per_row] / sqrt_k) * kResolvedUnit);
        float v[8];
        decode_resolved(word[i], tail[i], seed_plus_offset + g * 8u, resolved_scale(scales, word[i]), v);
        const bf16x2 h0 = pack_bf16x2(v[0], v[1]), h1 = pack_bf16x2(v[2], v[3]);
        const bf16x2 h2 = pack_bf16x2(v[4], v[5]), h3 = pack_bf16x2(v[6], v[7]);
        out[g] = make_uint4(__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1),
                            __builtin_bit_cast(uint32_t, h2), __builtin_bit_cast(uint32_t, h3));
    }
}

}  // namespace nq

namespace nq {
int dense_split_for(int m, int n, int k, size_t partial_bytes);
struct DenseOutputs;
int launch_bf16_gemm(const void *a, const void *b, void *c, int m, int n, int k, int forced_tile, int forced_split,
                     void *partials, size_t partial_bytes, hipStream_t stream, const DenseOutputs *split_outputs);
}

namespace {

constexpr int kChunkRows = 512;    // 8 wavefronts x 2 tiles x 32 rows
// From this many rows on (BF16 output, automatic split) the weight is decoded once into a BF16
// scratch [N][K] in the workspace and a dense BF16 GEMM multiplies: the fused kernel decodes a
// block once per 512 rows and re-reads the activation once per 32 channels.
constexpr int kDecodeOnceRows = 257;

bool decodes_once(int m, int k, int split_k) { return split_k == 0 && m >= kDecodeOnceRows && k % 128 == 0; }

// enough workgroups for 256 CUs; slabs stay multiples of 128
int pick_gemm_split(int k, int n, int requested) {
    if (requested > 0) return requested;
    const int groups = (n + nq::kGemmBN - 1) / nq::kGemmBN;
    int split = 1;
    while (split < 16 && groups * split < 256 && (k / (split * 2)) % nq::kGemmBK == 0) split *= 2;
    return split;
}

// The form of one launch of the fused kernel: 32- or 64-channel tiles, and the K slabs.
// Two channel tiles per workgroup halve the reads of the activation, which every workgroup makes for
// its whole K slab and which a launch of many tiles or of long rows waits for; they are taken from 96
// rows on (below, the launch waits for the decode of its slowest workgroup, and twice the workgroups
// share that better), where enough workgroups are left
//   * without a K split (gate + up of a short prefill; us, 32- / 64-channel tiles: 96 rows 34.6 / 33.7,
//     128 rows 40.3 / 35.7, 200 rows 58.6 / 47.0, 256 rows 68.4 / 50.4, 64 rows 27.8 / 30.3), or
//   * with twice the slabs when a row of the activation has 4096 values or more (down_proj, K = 8192:
//     128 rows 26.7 / 24.8, 256 rows 40.1 / 33.5; a 4096 x 4096 weight at 256 rows 41.2 / 33.8): the halved
//     reads outweigh the doubled partial sums, which they do not for rows of 2048 values (q/k/v at 128
//     rows 17.6 / 22.0, o_proj 13.1 / 14.6), or
//   * with the slabs of the 32-channel form where 192 workgroups remain (q/k/v: 128 rows 17.6 / 16.6,
//     256 rows 27.8 / 23.1; not o_proj, 128 workgroups: 12.9 / 14.4).
// A split the caller names is kept.  Every split gives the same bits in both forms.
struct GemmPlan {
    bool wide;
    int split;
};

GemmPlan plan_fused_gemm(int rows, int k, int n_total, int requested, bool resolved, bool whole_tiles) {
    GemmPlan plan{false, pick_gemm_split(k, n_total, requested)};
    if (!resolved || !whole_tiles || rows < 96 || rows > 8 * 32) return plan;
    const int tiles = (n_total + 63) / 64;
    if (requested > 0) {
        plan.wide = tiles * requested >= 192;
        return plan;
    }
    int split = 1;
    while (split < 16 && tiles * split < 256 && (k / (split * 2)) % nq::kGemmBK == 0) split *= 2;
    if (tiles * split >= 256 && (split == 1 || k >= 4096)) plan = GemmPlan{true, split};
    else if (tiles * plan.split >= 192) plan.wide = true;
    return plan;
}

// whether every weight of a launch but the last has a multiple of 64 channels (a workgroup's tiles lie in one weight)
bool whole_wide_tiles(const nq::GemmWeights &weights, int n_total) {
    bool whole = true;
    for (int g = 0; g < nq::kGemmMaxGroups; g++) whole = whole && (weights.end[g] % 64 == 0 || weights.end[g] == n_total);
    return whole;
}

// One launch of the fused kernel over `rows` tokens and the n_total channels of `weights`.
int launch_fused_gemm(const uint16_t *act, const nq::GemmWeights &weights, bool resolved, int rows, int k, int n_total,
                      const GemmPlan &plan, float *out_f32, hipStream_t s) {
    const float sqrt_k = (float)sqrt((double)k);
    const int split = plan.split;
    if (plan.wide) {
        hipLaunchKernelGGL((nq::w4a4_gemm_kernel<1, true, 2>), dim3((unsigned)((n_total + 63) / 64), (unsigned)split),
                           dim3(nq::kGemmThreads), 0, s, act, weights, rows, k, n_total, k / split, sqrt_k, out_f32);
        return nq::check_launch("nq_w4a4_gemm");
    }
    const dim3 grid((unsigned)((n_total + nq::kGemmBN - 1) / nq::kGemmBN), (unsigned)split);
#define NQ_LAUNCH_GEMM(TILES, RESOLVED)                                                                     \
    hipLaunchKernelGGL((nq::w4a4_gemm_kernel<TILES, RESOLVED>), grid, dim3(nq::kGemmThreads), 0, s, act,    \
                       weights, rows, k, n_total, k / split, sqrt_k, out_f32)
    if (rows <= 8 * 32) {
        if (resolved) NQ_LAUNCH_GEMM(1, true);
        else NQ_LAUNCH_GEMM(1, false);
    } else {
        if (resolved) NQ_LAUNCH_GEMM(2, true);
        else NQ_LAUNCH_GEMM(2, false);
    }
#undef NQ_LAUNCH_GEMM
    return nq::check_launch("nq_w4a4_gemm");
}

}  // namespace

extern "C" size_t nq_w4a4_gemm_workspace_bytes(int m, int k, int n, int split_k, int have_decoded_activation) {
    if (m < 1 || n < 1 || k < 1) return 0;
    size_t bytes = 0;
    if (!have_decoded_activation) bytes += nq::align256((size_t)m * k * 2);
    // the output dtype is not known here: enough for the decode-once scratch (BF16 output) and for the
    // fused kernel's partial sums (FP32 output) alike
    const int chunk = m < kChunkRows ? m : kChunkRows;
    // (nor the weight's form: the larger of the two forms' splits)
    const int narrow = pick_gemm_split(k, n, split_k), other = plan_fused_gemm(chunk, k, n, split_k, true, true).split;
    const int split = narrow > other ? narrow : other;
    const size_t partials = split > 1 ? (size_t)split * (size_t)chunk * (size_t)n * sizeof(float) : 0;
    // decode-once: the BF16 weight, then the partial results of the dense product's own K split
    size_t scratch = 0;
    if (decodes_once(m, k, split_k)) {
        const int dense_split = nq::dense_split_for(m, n, k, ~(size_t)0);
        scratch = nq::align256((size_t)n * k * 2) + (dense_split > 1 ? (size_t)dense_split * m * n * sizeof(float) : 0);
    }
    return bytes + (scratch > partials ? scratch : partials);
}

extern "C" int nq_w4a4_gemm(const uint8_t *act_codes_dev, const uint8_t *act_beta_ids_dev,
                            const float *act_norms_dev, const float *act_betas_dev,
                            const void *act_decoded_dev, const uint8_t *w_codes_dev,
                            const uint8_t *w_beta_ids_dev, const uint32_t *w_resolved_words_dev,
                            const uint16_t *w_resolved_tails_dev, const float *w_norms_dev,
                            const float *w_betas_dev, int m, int k, int n, int64_t weight_offset,
                            int64_t weight_seed, int split_k, void *out_dev, int out_dtype,
                            void *workspace_dev, size_t workspace_bytes, void *stream) {
    NQ_REQUIRE(m >= 1, NQ_ERR_SHAPE, "nq_w4a4_gemm: M must be positive");
    NQ_REQUIRE(k >= nq::kGemmBK && k % nq::kGemmBK == 0, NQ_ERR_SHAPE,
               "nq_w4a4_gemm: K = %d must be a positive multiple of 128", k);
    NQ_REQUIRE(n >= 1, NQ_ERR_SHAPE, "nq_w4a4_gemm: N must be positive");
    NQ_REQUIRE(split_k == 0 || split_k == 1 || split_k == 2 || split_k == 4 || split_k == 8 || split_k == 16,
               NQ_ERR_ARGUMENT, "nq_w4a4_gemm: split_k must be 0, 1, 2, 4, 8 or 16");
    NQ_REQUIRE(out_dtype == NQ_F32 || out_dtype == NQ_BF16, NQ_ERR_ARGUMENT,
               "nq_w4a4_gemm: output dtype tag %d is not F32 or BF16", out_dtype);
    const bool resolved = w_resolved_words_dev != nullptr;
    NQ_REQUIRE(w_norms_dev && w_betas_dev && out_dev, NQ_ERR_ARGUMENT, "nq_w4a4_gemm: null pointer");
    NQ_REQUIRE(resolved ? w_resolved_tails_dev != nullptr : (w_codes_dev && w_beta_ids_dev), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemm: neither packed nor resolved weight streams given");
    NQ_REQUIRE(act_decoded_dev || (act_codes_dev && act_beta_ids_dev && act_norms_dev && act_betas_dev),
               NQ_ERR_ARGUMENT, "nq_w4a4_gemm: neither packed nor decoded activation given");
    NQ_REQUIRE(nq::aligned(w_codes_dev, 4) && (!act_codes_dev || nq::aligned(act_codes_dev, 4)) &&
                   (!act_decoded_dev || nq::aligned(act_decoded_dev, 16)) &&
                   nq::aligned(w_resolved_words_dev, 4) && nq::aligned(w_resolved_tails_dev, 2),
               NQ_ERR_ARGUMENT, "nq_w4a4_gemm: code streams need 4-byte, decoded activation 16-byte alignment");
    NQ_REQUIRE(weight_seed >= 0 && weight_seed < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemm: seed must be in [0, 2**31)");
    NQ_REQUIRE(weight_offset >= 0 && weight_offset + (int64_t)n * (k / 8) <= ((int64_t)1 << 28),
               NQ_ERR_SHAPE, "nq_w4a4_gemm: block range exceeds the stateless dither counter space");
    const bool once = decodes_once(m, k, split_k) && out_dtype == NQ_BF16;
    const int chunk_rows = m < kChunkRows ? m : kChunkRows;
    const GemmPlan plan = once ? GemmPlan{false, 1} : plan_fused_gemm(chunk_rows, k, n, split_k, resolved, true);
    const int split = plan.split;
    NQ_REQUIRE(k % split == 0 && (k / split) % nq::kGemmBK == 0, NQ_ERR_SHAPE,
               "nq_w4a4_gemm: K / split_k = %d / %d must be a multiple of 128", k, split);
    const size_t decoded_bytes = act_decoded_dev ? 0 : nq::align256((size_t)m * k * 2);
    const size_t need = decoded_bytes + (once ? nq::align256((size_t)n * k * 2)
                                              : (split > 1 ? (size_t)split * chunk_rows * n * sizeof(float) : 0));
    NQ_REQUIRE(need == 0 || (workspace_dev && workspace_bytes >= need), NQ_ERR_WORKSPACE,
               "nq_w4a4_gemm: needs a %zu-byte workspace, got %zu", need, workspace_bytes);
    NQ_REQUIRE(need == 0 || nq::aligned(workspace_dev, 16), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemm: workspace must be 16-byte aligned");

    hipStream_t s = (hipStream_t)stream;
    const uint16_t *act = reinterpret_cast<const uint16_t *>(act_decoded_dev);
    if (!act) {
        int status = nq::launch_decode_activation(act_codes_dev, act_beta_ids_dev, act_norms_dev, act_betas_dev,
                                                  m, k, workspace_dev, s);
        if (status != NQ_OK) return status;
        act = reinterpret_cast<const uint16_t *>(workspace_dev);
    }
    float *partials = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace_dev) + decoded_bytes);
    if (once) {
        void *weight_bf16 = partials;
        const int status = nq_w4a4_decode_weight(w_codes_dev, w_beta_ids_dev, w_resolved_words_dev, w_resolved_tails_dev,
                                                 w_norms_dev, w_betas_dev, n, k, weight_offset, weight_seed, weight_bf16,
                                                 stream);
        if (status != NQ_OK) return status;
        char *dense_partials = reinterpret_cast<char *>(weight_bf16) + nq::align256((size_t)n * k * 2);
        const size_t used = (size_t)(dense_partials - reinterpret_cast<char *>(workspace_dev));
        return nq::launch_bf16_gemm(act, weight_bf16, out_dev, m, n, k, -1, 0, dense_partials,
                                    workspace_bytes > used ? workspace_bytes - used : 0, s, nullptr);
    }
    nq::GemmWeights weights = {};
    weights.words[0] = resolved ? w_resolved_words_dev : reinterpret_cast<const uint32_t *>(w_codes_dev);
    weights.tails[0] = w_resolved_tails_dev;
    weights.beta_ids[0] = w_beta_ids_dev;
    weights.norms[0] = w_norms_dev;
    weights.betas[0] = w_betas_dev;
    weights.seed_plus_offset[0] = (uint32_t)((uint64_t)weight_seed + (uint64_t)weight_offset * 8u);
    for (int g = 0; g < nq::kGemmMaxGroups; g++) weights.end[g] = n;
    const size_t out_row_bytes = (size_t)n * (out_dtype == NQ_F32 ? 4 : 2);
    for (int m0 = 0; m0 < m; m0 += kChunkRows) {
        const int rows = m - m0 < kChunkRows ? m - m0 : kChunkRows;
        char *out_chunk = reinterpret_cast<char *>(out_dev) + (size_t)m0 * out_row_bytes;
        float *target_f32 = split > 1 ? partials : (out_dtype == NQ_F32 ? (float *)out_chunk : nullptr);
        weights.out_bf16[0] = (split > 1 || out_dtype == NQ_F32) ? nullptr : (uint16_t *)out_chunk;
        int status = launch_fused_gemm(act + (size_t)m0 * k, weights, resolved, rows, k, n, plan, target_f32, s);
        if (status != NQ_OK) return status;
        if (split > 1) {
            status = nq::launch_splitk_reduce(partials, split, (int64_t)rows * n, out_chunk, out_dtype, s);
            if (status != NQ_OK) return status;
        }
    }
    return NQ_OK;
}

extern "C" size_t nq_w4a4_gemm_grouped_workspace_bytes(int m, int k, int n_total) {
    if (m < 1 || n_total < 1 || k < 1) return 0;
    const int narrow = pick_gemm_split(k, n_total, 0), other = plan_fused_gemm(m, k, n_total, 0, true, true).split;
    const int split = narrow > other ? narrow : other;
    return split > 1 ? (size_t)split * (size_t)m * (size_t)n_total * sizeof(float) : 0;
}

extern "C" int nq_w4a4_gemm_grouped(const void *act_decoded_dev, int count, const uint32_t *const *w_resolved_words_dev,
                                    const uint16_t *const *w_resolved_tails_dev, const float *const *w_norms_dev,
                                    const float *const *w_betas_dev, const int *n, const int64_t *weight_offsets,
                                    const int64_t *weight_seeds, void *const *out_bf16_dev, int m, int k,
                                    void *workspace_dev, size_t workspace_bytes, void *stream) {
    NQ_REQUIRE(count >= 1 && count <= nq::kGemmMaxGroups, NQ_ERR_ARGUMENT,
               "nq_w4a4_gemm_grouped: between one and four weights, got %d", count);
    NQ_REQUIRE(m >= 1 && m <= kChunkRows, NQ_ERR_SHAPE, "nq_w4a4_gemm_grouped: M = %d is outside [1, 512]", m);
    NQ_REQUIRE(k >= nq::kGemmBK && k % nq::kGemmBK == 0, NQ_ERR_SHAPE,
               "nq_w4a4_gemm_grouped: K = %d must be a positive multiple of 128", k);
    NQ_REQUIRE(act_decoded_dev && w_resolved_words_dev && w_resolved_tails_dev && w_norms_dev && w_betas_dev && n &&
                   weight_offsets && weight_seeds && out_bf16_dev,
               NQ_ERR_ARGUMENT, "nq_w4a4_gemm_grouped: null pointer");
    NQ_REQUIRE(nq::aligned(act_decoded_dev, 16), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemm_grouped: the decoded activation must be 16-byte aligned");
    nq::GemmWeights weights = {};
    nq::ReduceOutputs outputs = {};
    int64_t n_total = 0;
    for (int g = 0; g < count; g++) {
        NQ_REQUIRE(n[g] >= 32 && n[g] % 32 == 0, NQ_ERR_SHAPE,
                   "nq_w4a4_gemm_grouped: N = %d of weight %d is not a positive multiple of 32", n[g], g);
        NQ_REQUIRE(w_resolved_words_dev[g] && w_resolved_tails_dev[g] && w_norms_dev[g] && w_betas_dev[g] &&
                       out_bf16_dev[g], NQ_ERR_ARGUMENT, "nq_w4a4_gemm_grouped: null pointer for weight %d", g);
        NQ_REQUIRE(nq::aligned(w_resolved_words_dev[g], 4) && nq::aligned(w_resolved_tails_dev[g], 2) &&
                       nq::aligned(out_bf16_dev[g], 2), NQ_ERR_ARGUMENT,
                   "nq_w4a4_gemm_grouped: misaligned stream or output of weight %d", g);
        NQ_REQUIRE(weight_seeds[g] >= 0 && weight_seeds[g] < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
                   "nq_w4a4_gemm_grouped: seed must be in [0, 2**31)");
        NQ_REQUIRE(weight_offsets[g] >= 0 && weight_offsets[g] + (int64_t)n[g] * (k / 8) <= ((int64_t)1 << 28),
                   NQ_ERR_SHAPE, "nq_w4a4_gemm_grouped: block range exceeds the stateless dither counter space");
        n_total += n[g];
        NQ_REQUIRE(n_total <= ((int64_t)1 << 24), NQ_ERR_SHAPE, "nq_w4a4_gemm_grouped: too many channels");
        weights.words[g] = w_resolved_words_dev[g];
        weights.tails[g] = w_resolved_tails_dev[g];
        weights.norms[g] = w_norms_dev[g];
        weights.betas[g] = w_betas_dev[g];
        weights.out_bf16[g] = reinterpret_cast<uint16_t *>(out_bf16_dev[g]);
        weights.seed_plus_offset[g] = (uint32_t)((uint64_t)weight_seeds[g] + (uint64_t)weight_offsets[g] * 8u);
        weights.end[g] = (int)n_total;
        outputs.out[g] = weights.out_bf16[g];
        outputs.end[g] = (int64_t)m * n_total;
    }
    for (int g = count; g < nq::kGemmMaxGroups; g++) {
        weights.end[g] = (int)n_total;
        outputs.out[g] = outputs.out[count - 1];
        outputs.end[g] = (int64_t)m * n_total;
    }
    const GemmPlan plan = plan_fused_gemm(m, k, (int)n_total, 0, true, whole_wide_tiles(weights, (int)n_total));
    const int split = plan.split;
    const size_t need = split > 1 ? (size_t)split * m * n_total * sizeof(float) : 0;
    NQ_REQUIRE(need == 0 || (workspace_dev && workspace_bytes >= need), NQ_ERR_WORKSPACE,
               "nq_w4a4_gemm_grouped: needs a %zu-byte workspace, got %zu", need, workspace_bytes);
    NQ_REQUIRE(need == 0 || nq::aligned(workspace_dev, 16), NQ_ERR_ARGUMENT,
               "nq_w4a4_gemm_grouped: workspace must be 16-byte aligned");
    const hipStream_t s = (hipStream_t)stream;
    float *partials = split > 1 ? reinterpret_cast<float *>(workspace_dev) : nullptr;
    if (split > 1)
        for (int g = 0; g < nq::kGemmMaxGroups; g++) weights.out_bf16[g] = nullptr;
    int status = launch_fused_gemm(reinterpret_cast<const uint16_t *>(act_decoded_dev), weights, true, m, k, (int)n_total,
                                   plan, partials, s);
    if (status != NQ_OK || split == 1) return status;
    return nq::launch_splitk_reduce_grouped(partials, split, (int64_t)m * n_total, outputs, s);
}

extern "C" int nq_w4a4_decode_weight(const uint8_t *w_codes_dev, const uint8_t *w_beta_ids_dev,
                                     const uint32_t *w_resolved_words_dev, const uint16_t *w_resolved_tails_dev,
                                     const float *w_norms_dev, const float *w_betas_dev, int64_t n, int64_t k,
                                     int64_t weight_offset, int64_t weight_seed, void *out_bf16_dev, void *stream) {
    NQ_REQUIRE(n >= 1 && k >= 32 && k % 32 == 0, NQ_ERR_SHAPE,
               "nq_w4a4_decode_weight: N must be positive and K a positive multiple of 32");
    const bool resolved = w_resolved_words_dev != nullptr;
    NQ_REQUIRE(w_norms_dev && w_betas_dev && out_bf16_dev, NQ_ERR_ARGUMENT, "nq_w4a4_decode_weight: null pointer");
    NQ_REQUIRE(resolved ? w_resolved_tails_dev != nullptr : (w_codes_dev && w_beta_ids_dev), NQ_ERR_ARGUMENT,
               "nq_w4a4_decode_weight: neither packed nor resolved weight streams given");
    NQ_REQUIRE(nq::aligned(w_codes_dev, 4) && nq::aligned(w_resolved_words_dev, 4) &&
                   nq::aligned(w_resolved_tails_dev, 2) && nq::aligned(out_bf16_dev, 16),
               NQ_ERR_ARGUMENT, "nq_w4a4_decode_weight: code streams need 4-byte, the output 16-byte alignment");
    NQ_REQUIRE(weight_seed >= 0 && weight_seed < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
               "nq_w4a4_decode_weight: seed must be in [0, 2**31)");
    const int64_t blocks = n * (k / 8);
    NQ_REQUIRE(weight_offset >= 0 && weight_offset + blocks <= ((int64_t)1 << 28), NQ_ERR_SHAPE,
               "nq_w4a4_decode_weight: block range exceeds the stateless dither counter space");
    const uint32_t seed_plus_offset = (uint32_t)((uint64_t)weight_seed + (uint64_t)weight_offset * 8u);
    const float sqrt_k = (float)sqrt((double)k);
    const hipStream_t s = (hipStream_t)stream;
    const uint32_t blocks_per_row = (uint32_t)(k / 8);
    if (resolved) {
        constexpr int64_t per_group = 256 * nq::kDecodeBlocksPerLane;
        const dim3 grid((unsigned)((blocks + per_group - 1) / per_group));
        if (blocks_per_row % (64 * nq::kDecodeBlocksPerLane) == 0)
            hipLaunchKernelGGL(nq::decode_resolved_weight_kernel<true>, grid, dim3(256), 0, s, w_resolved_words_dev,
                               w_resolved_tails_dev, w_norms_dev, w_betas_dev, (uint32_t)blocks, blocks_per_row,
                               seed_plus_offset, sqrt_k, reinterpret_cast<uint4 *>(out_bf16_dev));
        else
            hipLaunchKernelGGL(nq::decode_resolved_weight_kernel<false>, grid, dim3(256), 0, s, w_resolved_words_dev,
                               w_resolved_tails_dev, w_norms_dev, w_betas_dev, (uint32_t)blocks, blocks_per_row,
                               seed_plus_offset, sqrt_k, reinterpret_cast<uint4 *>(out_bf16_dev));
    } else {
        hipLaunchKernelGGL(nq::decode_weight_kernel, dim3((unsigned)((blocks + 255) / 256)), dim3(256), 0, s,
                           reinterpret_cast<const uint32_t *>(w_codes_dev), w_beta_ids_dev, w_norms_dev, w_betas_dev,
                           blocks, (int)blocks_per_row, seed_plus_offset, sqrt_k,
                           reinterpret_cast<uint4 *>(out_bf16_dev));
    }
    return nq::check_launch("nq_w4a4_decode_weight");
}
