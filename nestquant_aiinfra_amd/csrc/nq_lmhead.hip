// BF16 linear for a few rows against a large BF16 weight (the LM head of a decode step:
// [rows <= 16, K] x [N, K]^T with N = 128 K): a stream over the weight, 2 N K bytes, with the
// products on the matrix cores.
//
// A weight row's eight consecutive k are one lane's A fragment of v_mfma_f32_16x16x32_bf16 (lane l:
// weight row l % 16, k = 32 step + 8 (l / 16) .. + 8), the activation's the B fragment (token l % 16,
// the same k), so nothing is transposed and nothing staged.  A workgroup of four wavefronts walks
// tiles of 16 weight rows; wavefront w owns the K quarter w, keeps its activation fragments in
// registers for the whole launch and requests the next tile's weight fragments before it
// multiplies the current ones; a workgroup's tiles are consecutive.  The four partial tiles meet in LDS and are added in wavefront
// order (deterministic), one lane per output.
#include "nq_e8.hip.h"
#include "nq_host.h"

namespace nq {

typedef float lm_floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 lm_bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t lm_u32x4 __attribute__((ext_vector_type(4)));

constexpr int kLmWaves = 4;
constexpr int kLmSteps = 16;                   // K-steps of 32 per wavefront: K = 4 x 16 x 32 = 2048 per pass

// kPasses: K = 2048 kPasses (the activation fragments of all passes stay in registers).
template <int kPasses>
__global__ void __launch_bounds__(64 * kLmWaves)
bf16_rows_linear_kernel(const uint4 *__restrict__ act,          // BF16 [rows][K / 8] blocks of eight
                        const lm_u32x4 *__restrict__ weight,    // BF16 [N][K / 8]
                        uint16_t *__restrict__ out, int rows, int n_size, int tiles) {
    constexpr int kSteps = kLmSteps * kPasses;
    __shared__ float part[kLmWaves][16 * 17];                  // [weight row][token], rows padded to 17
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int column = lane & 15, quarter = lane >> 4;
    const int blocks_per_row = 256 * kPasses;                   // K / 8
    // this lane's first block of a row: K quarter `wave`, then 4 blocks per K-step, one per lane quarter
    const int first_block = wave * (kSteps * 4) + quarter;

    // tokens past `rows` read row 0 and multiply by nothing
    uint4 b[kSteps];
    {
        const uint4 *row = act + (int64_t)(column < rows ? column : 0) * blocks_per_row + first_block;
        const uint32_t keep = column < rows ? 0xffffffffu : 0u;
#pragma unroll
        for (int s = 0; s < kSteps; s++) {
            const uint4 raw = row[4 * s];
            b[s] = make_uint4(raw.x & keep, raw.y & keep, raw.z & keep, raw.w & keep);
        }
    }

    const int per = (tiles + gridDim.x - 1) / gridDim.x;
    int tile = blockIdx.x * per;
    const int tiles_end = tile + per < tiles ? tile + per : tiles;
    lm_u32x4 a_next[kSteps];
    if (tile < tiles_end) {
        const int n = tile * 16 + column < n_size ? tile * 16 + column : n_size - 1;   // rows past the end repeat the last
        const lm_u32x4 *row = weight + (int64_t)n * blocks_per_row + first_block;
#pragma unroll
        for (int s = 0; s < kSteps; s++) a_next[s] = row[4 * s];
    }
    for (; tile < tiles_end; tile += 1) {
        lm_u32x4 a[kSteps];
#pragma unroll
        for (int s = 0; s < kSteps; s++) a[s] = a_next[s];
        const int ahead = tile + 1;
        if (ahead < tiles_end) {
            const int n = ahead * 16 + column < n_size ? ahead * 16 + column : n_size - 1;
            const lm_u32x4 *row = weight + (int64_t)n * blocks_per_row + first_block;
#pragma unroll
            for (int s = 0; s < kSteps; s++) a_next[s] = row[4 * s];
        }
        lm_floatx4 acc = lm_floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < kSteps; s++)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lm_bf16x8, a[s]),
                                                          __builtin_bit_cast(lm_bf16x8, b[s]), acc, 0, 0, 0);
        // accumulator i of lane l: weight row 4 (l / 16) + i of the tile, token l % 16
        __syncthreads();                                        // the previous tile's readers are done
#pragma unroll
        for (int i = 0; i < 4; i++) part[wave][(4 * quarter + i) * 17 + column] = acc[i];
        __syncthreads();
        {
            // sixteen lanes write one token's sixteen consecutive outputs
            const int row_in_tile = tid & 15, token = tid >> 4;
            const int n = tile * 16 + row_in_tile;
            if (n < n_size && token < rows) {
                float total = part[0][row_in_tile * 17 + token];
#pragma unroll
                for (int w = 1; w < kLmWaves; w++) total = total + part[w][row_in_tile * 17 + token];
                out[(int64_t)token * n_size + n] = f32_to_bf16(total);
            }
        }
    }
}

}  // namespace nq

extern "C" int nq_bf16_rows_linear(const void *act_bf16_dev, const void *weight_bf16_dev, int rows, int64_t k,
                                   int64_t n, void *out_bf16_dev, void *stream) {
    NQ_REQUIRE(rows >= 1 && rows <= 16, NQ_ERR_SHAPE, "nq_bf16_rows_linear: rows = %d is outside [1, 16]", rows);
    NQ_REQUIRE(k == 2048 || k == 4096, NQ_ERR_SHAPE, "nq_bf16_rows_linear: K = %lld is not 2048 or 4096", (long long)k);
    NQ_REQUIRE(n >= 1 && n <= ((int64_t)1 << 27), NQ_ERR_SHAPE, "nq_bf16_rows_linear: N must be in [1, 2**27]");
    NQ_REQUIRE(act_bf16_dev && weight_bf16_dev && out_bf16_dev, NQ_ERR_ARGUMENT, "nq_bf16_rows_linear: null pointer");
    NQ_REQUIRE(nq::aligned(act_bf16_dev, 16) && nq::aligned(weight_bf16_dev, 16), NQ_ERR_ARGUMENT,
               "nq_bf16_rows_linear: activation and weight must be 16-byte aligned");
    const int tiles = (int)((n + 15) / 16);
    // the workgroups a compute unit holds at once (two for K = 2048, one for 4096) take the tiles in turn
    const int resident = k == 2048 ? 512 : 256;
    const int grid = tiles < resident ? tiles : resident;
    const hipStream_t s = (hipStream_t)stream;
    if (k == 2048)
        hipLaunchKernelGGL(nq::bf16_rows_linear_kernel<1>, dim3(grid), dim3(64 * nq::kLmWaves), 0, s,
                           reinterpret_cast<const uint4 *>(act_bf16_dev), reinterpret_cast<const nq::lm_u32x4 *>(weight_bf16_dev),
                           reinterpret_cast<uint16_t *>(out_bf16_dev), rows, (int)n, tiles);
    else
        hipLaunchKernelGGL(nq::bf16_rows_linear_kernel<2>, dim3(grid), dim3(64 * nq::kLmWaves), 0, s,
                           reinterpret_cast<const uint4 *>(act_bf16_dev), reinterpret_cast<const nq::lm_u32x4 *>(weight_bf16_dev),
                           reinterpret_cast<uint16_t *>(out_bf16_dev), rows, (int)n, tiles);
    return nq::check_launch("nq_bf16_rows_linear");
}
