// BF16 linear for a few rows against a large BF16 weight ([rows <= 16, K] x [N, K]^T: the LM
// head of a decode step, or a packed projection whose weight has been expanded to the BF16
// values its kernels multiply by): a stream over the weight, 2 N K bytes, with the products on
// the matrix cores.
//
// A weight row's eight consecutive k are one lane's A fragment of v_mfma_f32_16x16x32_bf16 (lane l:
// weight row l % 16, k = 32 step + 8 (l / 16) .. + 8), the activation's the B fragment (token l % 16,
// the same k), so nothing is transposed and nothing staged.  A workgroup of four wavefronts walks
// a run of consecutive tiles of 16 weight rows, K in chunks of 2048; wavefront w owns quarter w of
// a chunk and requests the next (tile, chunk)'s weight fragments before it multiplies the current
// ones.  With one chunk the activation fragments stay in registers for the whole launch; with
// more they are read again per chunk (from the L2, behind the weight requests already in flight).
// The four partial tiles meet in LDS and are added in wavefront order (deterministic), one lane per
// output.  The N rows may belong to up to three outputs of their own (q, k and v of one activation).
// A weight with fewer tiles than there are compute units is walked in half tiles.
#include "nq_e8.hip.h"
#include "nq_host.h"

namespace nq {

typedef float lm_floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 lm_bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t lm_u32x4 __attribute__((ext_vector_type(4)));

constexpr int kLmWaves = 4;
constexpr int kLmSteps = 16;                   // K-steps of 32 per wavefront and chunk: 4 x 16 x 32 = 2048
constexpr int kLmChunkBlocks = 256;            // blocks of eight per row and chunk
constexpr int kLmMaxGroups = 3;

// Rows [end[g - 1], end[g]) of the weight produce out[g], BF16 [rows][end[g] - end[g - 1]].
struct LmOutputs {
    uint16_t *out[kLmMaxGroups];
    int end[kLmMaxGroups];
};

template <int kChunks>
__global__ void __launch_bounds__(64 * kLmWaves)
bf16_rows_linear_kernel(const uint4 *__restrict__ act,          // BF16 [rows][K / 8] blocks of eight
                        const lm_u32x4 *__restrict__ weight,    // BF16 [N][K / 8]
                        LmOutputs outputs, int rows, int n_size, int tiles, int split) {
    __shared__ float part[kLmWaves][16 * 17];                  // [weight row][token], rows padded to 17
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int column = lane & 15, quarter = lane >> 4;
    constexpr int blocks_per_row = kLmChunkBlocks * kChunks;    // K / 8
    // this lane's first block of a chunk: quarter `wave`, then 4 blocks per K-step, one per lane quarter
    const int lane_block = wave * (kLmSteps * 4) + quarter;

    // a workgroup's tiles are consecutive; its turns are (tile, chunk) pairs, chunks innermost
    const int per = (tiles + gridDim.x - 1) / gridDim.x;
    const int tile_begin = blockIdx.x * per;
    const int tile_end = tile_begin + per < tiles ? tile_begin + per : tiles;
    const int turns = tile_end > tile_begin ? (tile_end - tile_begin) * kChunks : 0;

    // tokens past `rows` read row 0 and multiply by nothing
    const uint4 *act_row = act + (int64_t)(column < rows ? column : 0) * blocks_per_row + lane_block;
    const uint32_t keep = column < rows ? 0xffffffffu : 0u;
    uint4 b[kLmSteps];
    if (kChunks == 1) {
#pragma unroll
        for (int s = 0; s < kLmSteps; s++) {
            const uint4 raw = act_row[4 * s];
            b[s] = make_uint4(raw.x & keep, raw.y & keep, raw.z & keep, raw.w & keep);
        }
    }

    // with `split` of 2 a tile is shared by two workgroups, eight of its rows each (a weight with
    // few rows then occupies every compute unit): the lanes of the other eight rows request nothing
    const int rows_each = 16 / split;
    const lm_u32x4 nothing = lm_u32x4{0u, 0u, 0u, 0u};
    lm_u32x4 a_next[kLmSteps];
    if (turns > 0) {
        const int n = (tile_begin / split) * 16 + column < n_size ? (tile_begin / split) * 16 + column : n_size - 1;   // rows past the end repeat the last
        const lm_u32x4 *row = weight + (int64_t)n * blocks_per_row + lane_block;
        const bool mine = column / rows_each == tile_begin % split;
#pragma unroll
        for (int s = 0; s < kLmSteps; s++) a_next[s] = mine ? row[4 * s] : nothing;
    }
    lm_floatx4 acc = lm_floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    for (int turn = 0; turn < turns; turn++) {
        const int tile = tile_begin + turn / kChunks, chunk = turn % kChunks;
        lm_u32x4 a[kLmSteps];
#pragma unroll
        for (int s = 0; s < kLmSteps; s++) a[s] = a_next[s];
        if (kChunks > 1) {
#pragma unroll
            for (int s = 0; s < kLmSteps; s++) {
                const uint4 raw = act_row[chunk * kLmChunkBlocks + 4 * s];
                b[s] = make_uint4(raw.x & keep, raw.y & keep, raw.z & keep, raw.w & keep);
            }
        }
        if (turn + 1 < turns) {
            const int ahead_tile = tile_begin + (turn + 1) / kChunks, ahead_chunk = (turn + 1) % kChunks;
            const int n = (ahead_tile / split) * 16 + column < n_size ? (ahead_tile / split) * 16 + column : n_size - 1;
            const lm_u32x4 *row = weight + (int64_t)n * blocks_per_row + ahead_chunk * kLmChunkBlocks + lane_block;
            const bool mine = column / rows_each == ahead_tile % split;
#pragma unroll
            for (int s = 0; s < kLmSteps; s++) a_next[s] = mine ? row[4 * s] : nothing;
        }
#pragma unroll
        for (int s = 0; s < kLmSteps; s++)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lm_bf16x8, a[s]),
                                                          __builtin_bit_cast(lm_bf16x8, b[s]), acc, 0, 0, 0);
        if (chunk != kChunks - 1) continue;
        // accumulator i of lane l: weight row 4 (l / 16) + i of the tile, token l % 16
        __syncthreads();                                        // the previous tile's readers are done
#pragma unroll
        for (int i = 0; i < 4; i++) part[wave][(4 * quarter + i) * 17 + column] = acc[i];
        acc = lm_floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        __syncthreads();
        {
            // sixteen lanes write one token's sixteen consecutive outputs
            const int row_in_tile = tid & 15, token = tid >> 4;
            const int n = (tile / split) * 16 + row_in_tile;
            if (n < n_size && token < rows && row_in_tile / rows_each == tile % split) {
                float total = part[0][row_in_tile * 17 + token];
#pragma unroll
                for (int w = 1; w < kLmWaves; w++) total = total + part[w][row_in_tile * 17 + token];
                const bool first = n < outputs.end[0], second = n < outputs.end[1];
                uint16_t *out = first ? outputs.out[0] : (second ? outputs.out[1] : outputs.out[2]);
                const int begin = first ? 0 : (second ? outputs.end[0] : outputs.end[1]);
                const int width = (first ? outputs.end[0] : (second ? outputs.end[1] : outputs.end[2])) - begin;
                out[(int64_t)token * width + (n - begin)] = f32_to_bf16(total);
            }
        }
    }
}

}  // namespace nq

extern "C" int nq_bf16_rows_linear_grouped(const void *act_bf16_dev, const void *weight_bf16_dev, int rows, int64_t k,
                                           int groups, const int64_t *group_n, void *const *outs_bf16_dev,
                                           void *stream) {
    NQ_REQUIRE(rows >= 1 && rows <= 16, NQ_ERR_SHAPE, "nq_bf16_rows_linear: rows = %d is outside [1, 16]", rows);
    NQ_REQUIRE(k == 2048 || k == 4096 || k == 8192, NQ_ERR_SHAPE, "nq_bf16_rows_linear: K = %lld is not 2048, 4096 or 8192",
               (long long)k);
    NQ_REQUIRE(groups >= 1 && groups <= nq::kLmMaxGroups && group_n && outs_bf16_dev, NQ_ERR_ARGUMENT,
               "nq_bf16_rows_linear: between one and three outputs with their sizes");
    NQ_REQUIRE(act_bf16_dev && weight_bf16_dev, NQ_ERR_ARGUMENT, "nq_bf16_rows_linear: null pointer");
    NQ_REQUIRE(nq::aligned(act_bf16_dev, 16) && nq::aligned(weight_bf16_dev, 16), NQ_ERR_ARGUMENT,
               "nq_bf16_rows_linear: activation and weight must be 16-byte aligned");
    nq::LmOutputs outputs;
    int64_t n = 0;
    for (int g = 0; g < nq::kLmMaxGroups; g++) {
        if (g < groups) {
            NQ_REQUIRE(group_n[g] >= 1 && n + group_n[g] <= ((int64_t)1 << 27), NQ_ERR_SHAPE,
                       "nq_bf16_rows_linear: N must be in [1, 2**27]");
            NQ_REQUIRE(outs_bf16_dev[g], NQ_ERR_ARGUMENT, "nq_bf16_rows_linear: null pointer");
            n += group_n[g];
        }
        outputs.out[g] = reinterpret_cast<uint16_t *>(outs_bf16_dev[g < groups ? g : groups - 1]);
        outputs.end[g] = (int)n;
    }
    // two workgroups per compute unit take the tiles in runs; a weight with at most 128 tiles (fewer
    // than compute units) is walked in half tiles, one workgroup each (2048 x 8192 at 8 rows: 12.6
    // against 14.2 us; with 192 tiles halves were slower, 6.9 against 5.6 us)
    const int split = (n + 15) / 16 <= 128 ? 2 : 1;
    const int tiles = (int)((n + 15) / 16) * split;
    const int grid = tiles < 512 ? tiles : 512;
    const hipStream_t s = (hipStream_t)stream;
#define NQ_LAUNCH_ROWS_LINEAR(CHUNKS)                                                                              \
    hipLaunchKernelGGL(nq::bf16_rows_linear_kernel<CHUNKS>, dim3(grid), dim3(64 * nq::kLmWaves), 0, s,             \
                       reinterpret_cast<const uint4 *>(act_bf16_dev),                                              \
                       reinterpret_cast<const nq::lm_u32x4 *>(weight_bf16_dev), outputs, rows, (int)n, tiles, split)
    if (k == 2048) NQ_LAUNCH_ROWS_LINEAR(1);
    else if (k == 4096) NQ_LAUNCH_ROWS_LINEAR(2);
    else NQ_LAUNCH_ROWS_LINEAR(4);
#undef NQ_LAUNCH_ROWS_LINEAR
    return nq::check_launch("nq_bf16_rows_linear");
}

extern "C" int nq_bf16_rows_linear(const void *act_bf16_dev, const void *weight_bf16_dev, int rows, int64_t k,
                                   int64_t n, void *out_bf16_dev, void *stream) {
    void *const outs[1] = {out_bf16_dev};
    return nq_bf16_rows_linear_grouped(act_bf16_dev, weight_bf16_dev, rows, k, 1, &n, outs, stream);
}
