// Dense BF16 GEMM on the matrix cores for long prefills: C[M, N] = A[M, K] * B[N, K]^T, both
// operands K-contiguous, FP32 accumulation, BF16 out.  A is the decoded NQA4 activation, B the
// BF16 weight nq_w4a4_decode_weight wrote once for the call, so that a prefill of hundreds or
// thousands of rows decodes every weight block once and multiplies at matrix-core speed.
//
// Tiling.  A workgroup of four wavefronts (2 x 2) owns a (64 WM) x (64 WN) tile of C; each
// wavefront owns WM x WN tiles of 32 x 32 (v_mfma_f32_32x32x16_bf16), e.g. 4 x 4 = 128 x 128 with
// 256 accumulator registers.  K is walked in steps of 64: the A and B slabs of a step sit in LDS
// as rows of 128 bytes whose eight 16-byte pieces are stored at piece ^ ((row / 2) % 8).  The LDS
// has 64 banks and serves sixteen lanes of a 16-byte read per cycle: sixteen consecutive rows of
// one fragment read (lane l: row l % 32, piece 2 s + l / 32) then fall on sixteen different groups
// of four banks (even rows in one half of the banks, odd rows in the other, eight different pieces
// in each), and so do the eight lanes that store one row.  LDS is double-buffered: the loads of step s + 1 are
// requested before the products of step s and stored after them, one barrier per step.
// Workgroups are numbered so that the ones that run together on one XCD (every eighth) form a
// compact block of tiles, i.e. share rows of A and of B in that XCD's L2.
// Replaces (together with nq_w4a4_decode_weight): run_large_m_staged and the chunk-and-pad wrapper for
// M beyond a few hundred rows, nestquant/runtime/nqrt4_w4a4_mma.cu:606-667 and
// nestquant/runtime/cuda_w4a4_mma.py:450-474.
#include "nq_linear_common.hip.h"

#include <stdint.h>

namespace nq {

typedef __bf16 gemm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gemm_floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // a native vector: stays in registers across the loop

constexpr int kDenseBK = 64;

__device__ __forceinline__ uint16_t dense_f32_to_bf16(float x) {
    uint32_t bits = __float_as_uint(x);
    bits += 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)(bits >> 16);
}

// The order a step's instructions should issue in (a hint to the scheduler, sched_group_barrier):
// the first fragments, then kGroups groups of four matrix instructions, each followed by its share
// of the kReads LDS reads of the next fragments, of the kMoves LDS stores of the next slab and of
// the kMoves global requests.  Left to itself the compiler issues the step as requests, reads and
// matrix instructions, stores: with the phases interleaved a wavefront's waits fall behind matrix
// instructions that are still running (8192^3: 1049 -> 945 us).
template <int kGroups, int kReads, int kMoves, int g = 0>
__device__ __forceinline__ void issue_order_groups() {
    if constexpr (g < kGroups) {
        constexpr int reads = kReads / kGroups + (g >= kGroups - kReads % kGroups ? 1 : 0);
        constexpr int moves = kMoves / kGroups + (g >= kGroups - kMoves % kGroups ? 1 : 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);                       // matrix instructions
        if constexpr (reads > 0) __builtin_amdgcn_sched_group_barrier(0x100, reads, 0);       // LDS reads
        if constexpr (moves > 0) {
            __builtin_amdgcn_sched_group_barrier(0x200, moves, 0);              // LDS stores
            __builtin_amdgcn_sched_group_barrier(0x020, moves, 0);              // global loads
        }
        issue_order_groups<kGroups, kReads, kMoves, g + 1>();
    }
}
template <int kGroups, int kReads, int kMoves>
__device__ __forceinline__ void issue_order(int) {
    __builtin_amdgcn_sched_group_barrier(0x100, kReads / 3, 0);
    issue_order_groups<kGroups, kReads, kMoves>();
}

// Column ranges of the product that go to outputs of their own (q, k and v of one activation
// multiplied by their weights stacked in B): range i starts at column first[i] and goes to out[i],
// a row-major matrix of its own width.  The host keeps every boundary a multiple of 256, so that no
// workgroup tile straddles one.  count == 0: the single output c.
struct DenseOutputs {
    uint16_t *out[3];
    int first[3], width[3];
    int count;
};

// The output a workgroup whose tile starts at column n0 stores to, its width, and n0 inside it.
__device__ __forceinline__ void tile_output(const DenseOutputs &outputs, int n0, uint16_t *&c, int &width, int &column0) {
    if (outputs.count == 0) return;
    int which = 0;
#pragma unroll
    for (int i = 1; i < 3; i++)
        if (i < outputs.count && n0 >= outputs.first[i]) which = i;
    c = which == 0 ? outputs.out[0] : (which == 1 ? outputs.out[1] : outputs.out[2]);
    width = which == 0 ? outputs.width[0] : (which == 1 ? outputs.width[1] : outputs.width[2]);
    column0 = n0 - (which == 0 ? outputs.first[0] : (which == 1 ? outputs.first[1] : outputs.first[2]));
}

// The wavefront's tiles go to C.  The products are taken as B A^T (the weight fragment is the matrix
// instruction's first operand), so accumulator r of lane l belongs to row l % 32 and column
// (r % 4) + 8 (r / 4) + 4 (l / 32) of its 32 x 32 tile: four neighbouring columns per lane and group of
// four accumulators, which leave as one 8-byte piece of BF16 (16 bytes of a float32 partial result).
// With one column per lane (A B^T) the same tile took 16 two-byte stores per lane instead of 4 wide
// ones, and the store instructions of a 256 x 128 tile took 7 us of the 44 us its workgroup ran.
template <int WM, int WN>
__device__ __forceinline__ void store_tiles(const gemm_floatx16 (&acc)[WM][WN], int row0, int col0, int lane,
                                            uint16_t *__restrict__ c, float *__restrict__ partial, int m_size,
                                            int n_size) {
    const bool wide = (n_size & 3) == 0 && (reinterpret_cast<uintptr_t>(c) & 7) == 0 &&
                      (reinterpret_cast<uintptr_t>(partial) & 15) == 0;
#pragma unroll
    for (int i = 0; i < WM; i++) {
        const int row = row0 + 32 * i + (lane & 31);
        if (row >= m_size) continue;
#pragma unroll
        for (int j = 0; j < WN; j++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int col = col0 + 32 * j + 8 * g + 4 * (lane >> 5);
                const float v0 = acc[i][j][4 * g], v1 = acc[i][j][4 * g + 1], v2 = acc[i][j][4 * g + 2],
                            v3 = acc[i][j][4 * g + 3];
                const int64_t at = (int64_t)row * n_size + col;
                if (wide && col + 3 < n_size) {
                    if (partial) {
                        *reinterpret_cast<float4 *>(partial + at) = make_float4(v0, v1, v2, v3);
                    } else {
                        uint2 packed;
                        packed.x = __builtin_bit_cast(uint32_t, pack_bf16x2(v0, v1));
                        packed.y = __builtin_bit_cast(uint32_t, pack_bf16x2(v2, v3));
                        *reinterpret_cast<uint2 *>(c + at) = packed;
                    }
                } else {
                    const float v[4] = {v0, v1, v2, v3};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if (col + e >= n_size) continue;
                        if (partial) partial[at + e] = v[e];
                        else c[at + e] = dense_f32_to_bf16(v[e]);
                    }
                }
            }
        }
    }
}

// The same tiles as BF16 by way of LDS, for whole rows of C: the wavefront parks its 32 WM x 32 WN
// values in `stage` (its own 2048 WM WN bytes, rows of 64 WN bytes whose 16-byte pieces sit at
// piece ^ (row % pieces)), then every lane takes one piece and the wavefront stores whole rows of its
// tile: 64 WN contiguous bytes per row instead of 16, a quarter of the requests to the L2 (which,
// with every workgroup of a round storing at once, is what the direct form waits for: 3.5 us per
// 256 x 128 tile against 7 us with two-byte stores).  Needs rows of C that are multiples of 16 bytes.
template <int WM, int WN>
__device__ __forceinline__ void store_tiles_by_rows(const gemm_floatx16 (&acc)[WM][WN], int row0, int col0, int lane,
                                                    uint16_t *__restrict__ c, int m_size, int n_size,
                                                    u32x4 *__restrict__ stage) {
    constexpr int kPieces = 4 * WN;                                // 16-byte pieces per row of the wavefront's tile
    uint2 *halves = reinterpret_cast<uint2 *>(stage);
#pragma unroll
    for (int i = 0; i < WM; i++) {
        const int row = 32 * i + (lane & 31);
#pragma unroll
        for (int j = 0; j < WN; j++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                uint2 packed;
                packed.x = __builtin_bit_cast(uint32_t, pack_bf16x2(acc[i][j][4 * g], acc[i][j][4 * g + 1]));
                packed.y = __builtin_bit_cast(uint32_t, pack_bf16x2(acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]));
                const int piece = (4 * j + g) ^ (row & (kPieces - 1));
                halves[(row * kPieces + piece) * 2 + (lane >> 5)] = packed;
            }
        }
    }
    // the pieces are read by other lanes than wrote them: LDS serves a wavefront's accesses in order,
    // and the compiler must keep them in this order too
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    constexpr int kRowsPerStore = 64 / kPieces;
#pragma unroll
    for (int pass = 0; pass < 32 * WM / kRowsPerStore; pass++) {
        const int row = pass * kRowsPerStore + lane / kPieces, piece = lane % kPieces;
        const u32x4 value = stage[row * kPieces + (piece ^ (row & (kPieces - 1)))];
        const int out_row = row0 + row, out_col = col0 + 8 * piece;
        if (out_row < m_size && out_col < n_size)                   // n_size is a multiple of 8 here
            *reinterpret_cast<u32x4 *>(c + (int64_t)out_row * n_size + out_col) = value;
    }
}

// WM x WN: 32 x 32 tiles per wavefront; GM x GN: wavefronts per workgroup along M and N.
template <int WM, int WN, int GM, int GN>
__global__ void __launch_bounds__(64 * GM * GN)
bf16_gemm_kernel(const uint16_t *__restrict__ a, const uint16_t *__restrict__ b, uint16_t *__restrict__ c,
                 int m_size, int n_size, int k_size, int tiles_m, int tiles_n, int group_m, int k_slab,
                 float *__restrict__ partials, DenseOutputs outputs) {
    constexpr int kThreads = 64 * GM * GN;
    constexpr int BM = 32 * WM * GM, BN = 32 * WN * GN;
    constexpr int kRowsPerPass = kThreads / 8;                     // rows one pass of 16-byte loads covers
    constexpr int kLoadsA = BM / kRowsPerPass, kLoadsB = BN / kRowsPerPass;
    static_assert(BM % kRowsPerPass == 0 && BN % kRowsPerPass == 0 && kRowsPerPass % 8 == 0, "tile and workgroup shapes");
    extern __shared__ u32x4 lds[];                                 // [2][BM + BN][8] pieces
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / GN, wave_n = wave % GN;

    // tile of this workgroup: every eighth workgroup shares an XCD; within an XCD's share, tiles are
    // walked in groups of group_m rows of tiles so that neighbours in time share operands
    int pid = blockIdx.x;
    const int total = tiles_m * tiles_n;
    if (total % 8 == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
    const int per_group = group_m * tiles_n;
    const int group = pid / per_group, first_m = group * group_m;
    const int rows_in_group = tiles_m - first_m < group_m ? tiles_m - first_m : group_m;
    const int in_group = pid - group * per_group;
    const int tile_m = first_m + in_group % rows_in_group, tile_n = in_group / rows_in_group;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // with a K split, workgroup row blockIdx.y multiplies the K range [k_begin, k_begin + k_slab) and
    // leaves a float32 partial result
    const int k_begin = blockIdx.y * k_slab;

    // global -> LDS role: piece (tid & 7) of rows (tid >> 3) + kRowsPerPass i
    const int load_row = tid >> 3, load_piece = tid & 7;
    const int store_slot = load_row * 8 + (load_piece ^ ((load_row >> 1) & 7));
    int a_offset[kLoadsA], b_offset[kLoadsB];                      // in elements, below 2^31 (checked by the host)
#pragma unroll
    for (int i = 0; i < kLoadsA; i++) {
        const int row = m0 + load_row + kRowsPerPass * i;
        a_offset[i] = (row < m_size ? row : m_size - 1) * k_size + k_begin + load_piece * 8;
    }
#pragma unroll
    for (int i = 0; i < kLoadsB; i++) {
        const int row = n0 + load_row + kRowsPerPass * i;
        b_offset[i] = (row < n_size ? row : n_size - 1) * k_size + k_begin + load_piece * 8;
    }

    // fragment role: A rows wave_m * 32 WM + 32 i + lane % 32, B rows likewise; piece 2 s + lane / 32
    const int frag_row = lane & 31, frag_half = lane >> 5, frag_mask = (lane >> 1) & 7;
    const int a_frag_base = (wave_m * 32 * WM + frag_row) * 8;
    const int b_frag_base = (BM + wave_n * 32 * WN + frag_row) * 8;

    gemm_floatx16 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < WN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // Slabs are requested two steps ahead: registers `early` hold slab s + 1 (requested a step ago,
    // stored to LDS at the end of step s), registers `late` receive slab s + 2 at the top of step s.
    // A step of 64 k lasts about as long as a trip to the L2 and back under load, so one step of
    // lead leaves the matrix cores waiting for the stores.
    const int steps = k_slab / kDenseBK;
    u32x4 pa0[kLoadsA], pa1[kLoadsA], pb0[kLoadsB], pb1[kLoadsB];
    {
        u32x4 ra[kLoadsA], rb[kLoadsB];
#pragma unroll
        for (int i = 0; i < kLoadsA; i++) ra[i] = *reinterpret_cast<const u32x4 *>(a + a_offset[i]);
#pragma unroll
        for (int i = 0; i < kLoadsB; i++) rb[i] = *reinterpret_cast<const u32x4 *>(b + b_offset[i]);
        const int k_one = steps > 1 ? kDenseBK : 0;
#pragma unroll
        for (int i = 0; i < kLoadsA; i++) pa1[i] = *reinterpret_cast<const u32x4 *>(a + a_offset[i] + k_one);
#pragma unroll
        for (int i = 0; i < kLoadsB; i++) pb1[i] = *reinterpret_cast<const u32x4 *>(b + b_offset[i] + k_one);
#pragma unroll
        for (int i = 0; i < kLoadsA; i++) lds[store_slot + kRowsPerPass * 8 * i] = ra[i];
#pragma unroll
        for (int i = 0; i < kLoadsB; i++) lds[BM * 8 + store_slot + kRowsPerPass * 8 * i] = rb[i];
    }
    __syncthreads();

    // one step: request slab step + 2 into set `late`, multiply slab `step` from LDS, store set `early`
    // (slab step + 1) into the other LDS buffer
    auto dense_step = [&](int step, u32x4 (&late_a)[kLoadsA], u32x4 (&late_b)[kLoadsB],
                          const u32x4 (&early_a)[kLoadsA], const u32x4 (&early_b)[kLoadsB]) {
        const u32x4 *now = lds + (step & 1) * (BM + BN) * 8;
        u32x4 *next = lds + ((step + 1) & 1) * (BM + BN) * 8;
        const int ahead = step + 2 < steps ? step + 2 : steps - 1;      // past the end: any valid slab
#pragma unroll
        for (int i = 0; i < kLoadsA; i++) late_a[i] = *reinterpret_cast<const u32x4 *>(a + a_offset[i] + ahead * kDenseBK);
#pragma unroll
        for (int i = 0; i < kLoadsB; i++) late_b[i] = *reinterpret_cast<const u32x4 *>(b + b_offset[i] + ahead * kDenseBK);
        // fragments of sub-step s + 1 are read while the products of sub-step s run
        gemm_bf16x8 fa[2][WM], fb[2][WN];
#pragma unroll
        for (int i = 0; i < WM; i++) fa[0][i] = __builtin_bit_cast(gemm_bf16x8, now[a_frag_base + 256 * i + (frag_half ^ frag_mask)]);
#pragma unroll
        for (int j = 0; j < WN; j++) fb[0][j] = __builtin_bit_cast(gemm_bf16x8, now[b_frag_base + 256 * j + (frag_half ^ frag_mask)]);
#pragma unroll
        for (int s = 0; s < kDenseBK / 16; s++) {
            if (s + 1 < kDenseBK / 16) {
                const int piece = (2 * (s + 1) + frag_half) ^ frag_mask;
#pragma unroll
                for (int i = 0; i < WM; i++)
                    fa[(s + 1) & 1][i] = __builtin_bit_cast(gemm_bf16x8, now[a_frag_base + 256 * i + piece]);
#pragma unroll
                for (int j = 0; j < WN; j++)
                    fb[(s + 1) & 1][j] = __builtin_bit_cast(gemm_bf16x8, now[b_frag_base + 256 * j + piece]);
            }
#pragma unroll
            for (int i = 0; i < WM; i++)
#pragma unroll
                for (int j = 0; j < WN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[s & 1][j], fa[s & 1][i], acc[i][j], 0, 0, 0);
        }
        // (after the last step this stores a slab nobody reads, into the buffer nobody is reading)
#pragma unroll
        for (int i = 0; i < kLoadsA; i++) next[store_slot + kRowsPerPass * 8 * i] = early_a[i];
#pragma unroll
        for (int i = 0; i < kLoadsB; i++) next[BM * 8 + store_slot + kRowsPerPass * 8 * i] = early_b[i];
        issue_order<WM * WN, 3 * (WM + WN), kLoadsA + kLoadsB>(WM + WN);
        // a barrier that orders LDS traffic only: the requests for slab step + 2 stay in flight across it
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    };
    for (int step = 0; step < steps; step += 2) {          // the host checks that the step count is even
        dense_step(step, pa0, pb0, pa1, pb1);
        dense_step(step + 1, pa1, pb1, pa0, pb0);
    }

    // (the last step's barrier has passed: nobody reads the slabs any more)
    uint16_t *c_out = c;
    int width = n_size, column0 = n0;
    tile_output(outputs, n0, c_out, width, column0);
    if (!partials && (width & 7) == 0 && (reinterpret_cast<uintptr_t>(c_out) & 15) == 0)
        store_tiles_by_rows<WM, WN>(acc, m0 + wave_m * 32 * WM, column0 + wave_n * 32 * WN, lane, c_out, m_size, width,
                                    lds + wave * (128 * WM * WN));
    else
        store_tiles<WM, WN>(acc, m0 + wave_m * 32 * WM, column0 + wave_n * 32 * WN, lane, c_out,
                            partials ? partials + (int64_t)blockIdx.y * m_size * n_size : nullptr, m_size, width);
}


// The same product with the wavefronts of a workgroup split by role: four of the eight (one per
// SIMD) only move data -- global loads three steps ahead into a ring of registers, then into a ring
// of three LDS stages -- and four only multiply, each a quarter (WM x WN tiles of 32 x 32) of the
// workgroup's 64 WM x 64 WN tile.  A wavefront that waits for memory therefore never holds back
// matrix instructions: the multiplying wavefront of its SIMD keeps issuing.  One barrier per step of
// 64 k; before it the movers wait for their LDS stores only (their global loads stay in flight).
template <int WM, int WN>
__global__ void __launch_bounds__(512)
bf16_gemm_roles_kernel(const uint16_t *__restrict__ a, const uint16_t *__restrict__ b, uint16_t *__restrict__ c,
                       int m_size, int n_size, int k_size, int tiles_m, int tiles_n, int group_m, int k_slab,
                       float *__restrict__ partials, DenseOutputs outputs) {
    constexpr int BM = 64 * WM, BN = 64 * WN;
    constexpr int kStage = (BM + BN) * 8;                          // 16-byte pieces per LDS stage
    constexpr int kLoadsA = BM / 32, kLoadsB = BN / 32;            // 256 mover lanes cover 32 rows of 128 bytes per pass
    constexpr int kLoads = kLoadsA + kLoadsB;
    extern __shared__ u32x4 lds[];                                 // [3][BM + BN][8] pieces
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    int pid = blockIdx.x;
    const int total = tiles_m * tiles_n;
    if (total % 8 == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
    const int per_group = group_m * tiles_n;
    const int group = pid / per_group, first_m = group * group_m;
    const int rows_in_group = tiles_m - first_m < group_m ? tiles_m - first_m : group_m;
    const int in_group = pid - group * per_group;
    const int tile_m = first_m + in_group % rows_in_group, tile_n = in_group / rows_in_group;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int k_begin = blockIdx.y * k_slab;
    const int steps = k_slab / kDenseBK;
    // a workgroup barrier that orders LDS traffic only: the movers' global loads stay in flight across it
    auto lds_barrier = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    };

    if (wave >= 4) {
        // ---- movers ---------------------------------------------------------------------------------
        const int mover = tid - 256;
        const int load_row = mover >> 3, load_piece = mover & 7;
        const int store_slot = load_row * 8 + (load_piece ^ ((load_row >> 1) & 7));
        int offset[kLoads], slot[kLoads];
#pragma unroll
        for (int i = 0; i < kLoadsA; i++) {
            const int row = m0 + load_row + 32 * i;
            offset[i] = (row < m_size ? row : m_size - 1) * k_size + k_begin + load_piece * 8;
            slot[i] = store_slot + 256 * i;
        }
#pragma unroll
        for (int i = 0; i < kLoadsB; i++) {
            const int row = n0 + load_row + 32 * i;
            offset[kLoadsA + i] = (row < n_size ? row : n_size - 1) * k_size + k_begin + load_piece * 8;
            slot[kLoadsA + i] = BM * 8 + store_slot + 256 * i;
        }
        auto request = [&](int step, u32x4 (&into)[kLoads]) {
            const int at = (step < steps ? step : steps - 1) * kDenseBK;        // past the end: any valid slab, never stored
#pragma unroll
            for (int i = 0; i < kLoads; i++) {
                const uint16_t *base = i < kLoadsA ? a : b;
                into[i] = *reinterpret_cast<const u32x4 *>(base + offset[i] + at);
            }
        };
        auto park = [&](int step, const u32x4 (&from)[kLoads]) {
            if (step < steps) {
                u32x4 *stage = lds + (step % 3) * kStage;
#pragma unroll
                for (int i = 0; i < kLoads; i++) stage[slot[i]] = from[i];
            }
        };
        u32x4 r0[kLoads], r1[kLoads], r2[kLoads];
        request(0, r0);
        request(1, r1);
        request(2, r2);
        park(0, r0);
        park(1, r1);
        request(3, r0);
        request(4, r1);
        lds_barrier();
        // at step s: slab s + 2 goes to its stage (the one the multipliers finished with at step s - 1),
        // slab s + 5 is requested into the registers that held it
        for (int s = 0; s < steps; s += 3) {
            park(s + 2, r2);
            request(s + 5, r2);
            lds_barrier();
            if (s + 1 < steps) {
                park(s + 3, r0);
                request(s + 6, r0);
                lds_barrier();
            }
            if (s + 2 < steps) {
                park(s + 4, r1);
                request(s + 7, r1);
                lds_barrier();
            }
        }
        return;
    }

    // ---- multipliers --------------------------------------------------------------------------------
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const int frag_row = lane & 31, frag_half = lane >> 5, frag_mask = (lane >> 1) & 7;
    const int a_frag_base = (wave_m * 32 * WM + frag_row) * 8;
    const int b_frag_base = (BM + wave_n * 32 * WN + frag_row) * 8;
    gemm_floatx16 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < WN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
    lds_barrier();                                                 // slabs 0 and 1 are parked
    for (int step = 0; step < steps; step++) {
        const u32x4 *now = lds + (step % 3) * kStage;
        gemm_bf16x8 fa[2][WM], fb[2][WN];
#pragma unroll
        for (int i = 0; i < WM; i++) fa[0][i] = __builtin_bit_cast(gemm_bf16x8, now[a_frag_base + 256 * i + (frag_half ^ frag_mask)]);
#pragma unroll
        for (int j = 0; j < WN; j++) fb[0][j] = __builtin_bit_cast(gemm_bf16x8, now[b_frag_base + 256 * j + (frag_half ^ frag_mask)]);
#pragma unroll
        for (int s = 0; s < kDenseBK / 16; s++) {
            if (s + 1 < kDenseBK / 16) {
                const int piece = (2 * (s + 1) + frag_half) ^ frag_mask;
#pragma unroll
                for (int i = 0; i < WM; i++)
                    fa[(s + 1) & 1][i] = __builtin_bit_cast(gemm_bf16x8, now[a_frag_base + 256 * i + piece]);
#pragma unroll
                for (int j = 0; j < WN; j++)
                    fb[(s + 1) & 1][j] = __builtin_bit_cast(gemm_bf16x8, now[b_frag_base + 256 * j + piece]);
            }
#pragma unroll
            for (int i = 0; i < WM; i++)
#pragma unroll
                for (int j = 0; j < WN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[s & 1][j], fa[s & 1][i], acc[i][j], 0, 0, 0);
        }
        issue_order<WM * WN, 3 * (WM + WN), 0>(WM + WN);
        lds_barrier();                                             // every fragment of the stage has arrived
    }
    // (the last step's barrier has passed: nobody reads the slabs any more)
    uint16_t *c_out = c;
    int width = n_size, column0 = n0;
    tile_output(outputs, n0, c_out, width, column0);
    if (!partials && (width & 7) == 0 && (reinterpret_cast<uintptr_t>(c_out) & 15) == 0)
        store_tiles_by_rows<WM, WN>(acc, m0 + wave_m * 32 * WM, column0 + wave_n * 32 * WN, lane, c_out, m_size, width,
                                    lds + wave * (128 * WM * WN));
    else
        store_tiles<WM, WN>(acc, m0 + wave_m * 32 * WM, column0 + wave_n * 32 * WN, lane, c_out,
                            partials ? partials + (int64_t)blockIdx.y * m_size * n_size : nullptr, m_size, width);
}

}  // namespace nq

namespace {

struct DenseTile { int bm, bn; float efficiency, alone; };

// Workgroup tiles from the fastest per product to the slowest; `efficiency` is the measured rate
// relative to the 256 x 256 tile on a problem that fills the chip (8192^3: 1.13, 0.92, 0.99, 0.93,
// 0.74, 0.74, 0.61 PFLOP/s).  The 256 x 128 tile always runs on the kernel with movers and
// multipliers (0.94 PFLOP/s with every wavefront doing both).  For 128 x 128, 64 x 128 and 64 x 64
// that kernel's three LDS stages leave room for one workgroup per compute unit where the plain
// kernel fits two or more, so it loses when a product has more tiles than compute units (M = 1024,
// N = 8192, K = 2048 at 128 x 128: 52 against 45 us) and wins when every compute unit holds at
// most one tile, because it keeps five slabs in flight instead of two and a lone workgroup is bound
// by the latency of its loads (M = 384, same N and K: 24.6 against 27.7 us; M = 128 at 64 x 64:
// 16.5 against 20.1 us): `alone` is the rate in that case, 0 where the plain kernel stays.
// All of them sit at the LDS's 128 bytes per clock: a wavefront that owns 2 x 4 tiles reads 0.75 KB
// of fragments per matrix instruction, which with the stores of the next slab is about 125 bytes
// per clock at full matrix rate.
const DenseTile kDenseTiles[] = {
    {256, 256, 1.00f, 0.0f}, {128, 256, 0.81f, 0.0f}, {256, 128, 0.89f, 0.0f}, {128, 128, 0.82f, 0.92f},
    {64, 128, 0.65f, 0.73f}, {128, 64, 0.65f, 0.0f},  {64, 64, 0.55f, 0.67f},
};

template <int WM, int WN, int GM, int GN>
void launch_dense(const void *a, const void *b, void *c, int m, int n, int k, int split, float *partials,
                  const nq::DenseOutputs &outputs, hipStream_t stream) {
    constexpr int BM = 32 * WM * GM, BN = 32 * WN * GN;
    const int tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    const size_t lds_bytes = (size_t)2 * (BM + BN) * 128;
    static bool raised = false;                  // once per process: permission for more than 64 KiB of LDS
    if (!raised) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(nq::bf16_gemm_kernel<WM, WN, GM, GN>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        raised = true;
    }
    const int group_m = tiles_m < 4 ? tiles_m : 4;
    hipLaunchKernelGGL((nq::bf16_gemm_kernel<WM, WN, GM, GN>), dim3((unsigned)(tiles_m * tiles_n), (unsigned)split),
                       dim3(64 * GM * GN), lds_bytes, stream, reinterpret_cast<const uint16_t *>(a),
                       reinterpret_cast<const uint16_t *>(b), reinterpret_cast<uint16_t *>(c), m, n, k, tiles_m, tiles_n,
                       group_m, k / split, split > 1 ? partials : nullptr, outputs);
}

template <int WM, int WN>
void launch_roles(const void *a, const void *b, void *c, int m, int n, int k, int split, float *partials,
                  const nq::DenseOutputs &outputs, hipStream_t stream) {
    constexpr int BM = 64 * WM, BN = 64 * WN;
    const int tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    const size_t lds_bytes = (size_t)3 * (BM + BN) * 128;
    static bool raised = false;
    if (!raised) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(nq::bf16_gemm_roles_kernel<WM, WN>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        raised = true;
    }
    const int group_m = tiles_m < 4 ? tiles_m : 4;
    hipLaunchKernelGGL((nq::bf16_gemm_roles_kernel<WM, WN>), dim3((unsigned)(tiles_m * tiles_n), (unsigned)split),
                       dim3(512), lds_bytes, stream, reinterpret_cast<const uint16_t *>(a),
                       reinterpret_cast<const uint16_t *>(b), reinterpret_cast<uint16_t *>(c), m, n, k, tiles_m, tiles_n,
                       group_m, k / split, split > 1 ? partials : nullptr, outputs);
}

}  // namespace

namespace nq {

// K split of a product whose tiles would leave most of the chip idle: 1 (none), 2, 4 or 8 slabs of
// at least 2048 k, as long as the 128 x 128 tiles times the slabs stay within one per compute unit,
// within a partial-result buffer of `partial_bytes`.  (Measured at 384 rows: K = 8192, N = 2048 runs
// in 29 us with four slabs against 42 us without; at K = 2048, N = 8192 the partial results cost
// more than the idle units, 35 against 27 us.)
int dense_split_for(int m, int n, int k, size_t partial_bytes) {
    const int64_t tiles = (int64_t)((m + 127) / 128) * ((n + 127) / 128);
    int split = 1;
    while (split < 8 && tiles * split * 2 <= 256 && k / (split * 2) >= 2048 && k % (split * 2 * 128) == 0 &&
           (size_t)(split * 2) * m * n * sizeof(float) <= partial_bytes)
        split *= 2;
    return split;
}

// Shared with nq_w4a4_gemm: picks the tile shape with the least estimated time (and, given a buffer
// for partial results, a K split) and launches.
int launch_bf16_gemm(const void *a, const void *b, void *c, int m, int n, int k, int forced_tile, int forced_split,
                     void *partials, size_t partial_bytes, hipStream_t stream, const DenseOutputs *split_outputs) {
    DenseOutputs outputs;
    outputs.count = 0;
    if (split_outputs) outputs = *split_outputs;
    // column ranges with outputs of their own are stored by the product's own launch: no K split
    if (outputs.count > 0) forced_split = 1;
    int split = forced_split > 0 ? forced_split : dense_split_for(m, n, k, partials ? partial_bytes : 0);
    if (split > 1 && (k % (split * 128) != 0 || !partials || (size_t)split * m * n * sizeof(float) > partial_bytes))
        return fail(NQ_ERR_WORKSPACE, "nq_bf16_gemm: a K split of %d needs K a multiple of %d and %zu bytes for partial results",
                    split, split * 128, (size_t)split * m * n * sizeof(float));
    int best = 0;
    float best_cost = 0.0f;
    bool best_alone = false;
    const int count = (int)(sizeof(kDenseTiles) / sizeof(kDenseTiles[0]));
    for (int t = 0; t < count; t++) {
        const DenseTile &tile = kDenseTiles[t];
        const int64_t tiles = (int64_t)((m + tile.bm - 1) / tile.bm) * ((n + tile.bn - 1) / tile.bn) * split;
        // the busiest of the 256 compute units works through ceil(tiles / 256) tiles, whether one
        // after the other or side by side at a share of its rate
        const bool alone = tiles <= 256 && tile.alone > 0.0f;
        const float cost = (float)((tiles + 255) / 256) * (float)(tile.bm * tile.bn) / (alone ? tile.alone : tile.efficiency);
        if (t == 0 || cost < best_cost) { best = t; best_cost = cost; best_alone = alone; }
    }
    // measurements may force a tile: 0..6 the table's entries on their usual kernel, 7..9 the 128 x 128,
    // 64 x 128 and 64 x 64 tiles on the kernel with movers and multipliers
    if (forced_tile >= 0 && forced_tile < count) { best = forced_tile; best_alone = false; }
    if (forced_tile == 7) { best = 3; best_alone = true; }
    if (forced_tile == 8) { best = 4; best_alone = true; }
    if (forced_tile == 9) { best = 6; best_alone = true; }
    float *p = reinterpret_cast<float *>(partials);
    switch (best) {
        case 0: launch_dense<2, 4, 4, 2>(a, b, c, m, n, k, split, p, outputs, stream); break;
        case 1: launch_dense<2, 4, 2, 2>(a, b, c, m, n, k, split, p, outputs, stream); break;
        case 2: launch_roles<4, 2>(a, b, c, m, n, k, split, p, outputs, stream); break;      // movers and multipliers
        case 3:
            if (best_alone) launch_roles<2, 2>(a, b, c, m, n, k, split, p, outputs, stream);
            else launch_dense<2, 2, 2, 2>(a, b, c, m, n, k, split, p, outputs, stream);
            break;
        case 4:
            if (best_alone) launch_roles<1, 2>(a, b, c, m, n, k, split, p, outputs, stream);
            else launch_dense<1, 2, 2, 2>(a, b, c, m, n, k, split, p, outputs, stream);
            break;
        case 5: launch_dense<2, 1, 2, 2>(a, b, c, m, n, k, split, p, outputs, stream); break;
        default:
            if (best_alone) launch_roles<1, 1>(a, b, c, m, n, k, split, p, outputs, stream);
            else launch_dense<1, 1, 2, 2>(a, b, c, m, n, k, split, p, outputs, stream);
            break;
    }
    const int status = check_launch("nq_bf16_gemm");
    if (status != NQ_OK || split == 1) return status;
    return launch_splitk_reduce(p, split, (int64_t)m * n, c, NQ_BF16, stream);
}

}  // namespace nq

extern "C" int nq_bf16_gemm(const void *a_bf16_dev, const void *b_bf16_dev, int64_t m, int64_t n, int64_t k,
                            void *c_bf16_dev, int tile, int split_k, void *workspace_dev, size_t workspace_bytes,
                            void *stream) {
    NQ_REQUIRE(m >= 1 && n >= 1 && m < ((int64_t)1 << 30) && n < ((int64_t)1 << 30), NQ_ERR_SHAPE,
               "nq_bf16_gemm: M and N must be positive");
    NQ_REQUIRE(k >= 2 * nq::kDenseBK && k % (2 * nq::kDenseBK) == 0 && k < ((int64_t)1 << 30), NQ_ERR_SHAPE,
               "nq_bf16_gemm: K = %lld must be a positive multiple of 128", (long long)k);
    NQ_REQUIRE(a_bf16_dev && b_bf16_dev && c_bf16_dev, NQ_ERR_ARGUMENT, "nq_bf16_gemm: null pointer");
    NQ_REQUIRE(nq::aligned(a_bf16_dev, 16) && nq::aligned(b_bf16_dev, 16) && nq::aligned(c_bf16_dev, 2), NQ_ERR_ARGUMENT,
               "nq_bf16_gemm: operands must be 16-byte aligned");
    NQ_REQUIRE(m * k < ((int64_t)1 << 31) && n * k < ((int64_t)1 << 31), NQ_ERR_SHAPE,
               "nq_bf16_gemm: operands of 2^31 elements or more are not supported");
    NQ_REQUIRE(tile >= -1 && tile <= 9, NQ_ERR_ARGUMENT, "nq_bf16_gemm: tile must be -1 (automatic) or 0..9");
    NQ_REQUIRE(split_k == 0 || split_k == 1 || split_k == 2 || split_k == 4 || split_k == 8, NQ_ERR_ARGUMENT,
               "nq_bf16_gemm: split_k must be 0 (automatic), 1, 2, 4 or 8");
    NQ_REQUIRE(!workspace_dev || nq::aligned(workspace_dev, 16), NQ_ERR_ARGUMENT, "nq_bf16_gemm: workspace must be 16-byte aligned");
    return nq::launch_bf16_gemm(a_bf16_dev, b_bf16_dev, c_bf16_dev, (int)m, (int)n, (int)k, tile, split_k, workspace_dev,
                                workspace_dev ? workspace_bytes : 0, (hipStream_t)stream, nullptr);
}

extern "C" int nq_bf16_gemm_split(const void *a_bf16_dev, const void *b_bf16_dev, int64_t m, int64_t k,
                                  void *const *outs_bf16_dev, const int64_t *widths, int count, int tile, void *stream) {
    NQ_REQUIRE(count >= 1 && count <= 3 && outs_bf16_dev && widths, NQ_ERR_ARGUMENT,
               "nq_bf16_gemm_split: one to three outputs");
    nq::DenseOutputs outputs;
    outputs.count = count;
    int64_t n = 0;
    for (int i = 0; i < 3; i++) {
        outputs.out[i] = nullptr; outputs.first[i] = 0; outputs.width[i] = 0;
        if (i >= count) continue;
        NQ_REQUIRE(widths[i] >= 256 && widths[i] % 256 == 0 && widths[i] < ((int64_t)1 << 30), NQ_ERR_SHAPE,
                   "nq_bf16_gemm_split: width %lld of output %d is not a positive multiple of 256", (long long)widths[i], i);
        NQ_REQUIRE(outs_bf16_dev[i] && nq::aligned(outs_bf16_dev[i], 16), NQ_ERR_ARGUMENT,
                   "nq_bf16_gemm_split: outputs must be 16-byte aligned");
        outputs.out[i] = reinterpret_cast<uint16_t *>(outs_bf16_dev[i]);
        outputs.first[i] = (int)n;
        outputs.width[i] = (int)widths[i];
        n += widths[i];
    }
    NQ_REQUIRE(m >= 1 && m < ((int64_t)1 << 30) && n < ((int64_t)1 << 30), NQ_ERR_SHAPE,
               "nq_bf16_gemm_split: M and N must be positive");
    NQ_REQUIRE(k >= 2 * nq::kDenseBK && k % (2 * nq::kDenseBK) == 0 && k < ((int64_t)1 << 30), NQ_ERR_SHAPE,
               "nq_bf16_gemm_split: K = %lld must be a positive multiple of 128", (long long)k);
    NQ_REQUIRE(a_bf16_dev && b_bf16_dev && nq::aligned(a_bf16_dev, 16) && nq::aligned(b_bf16_dev, 16), NQ_ERR_ARGUMENT,
               "nq_bf16_gemm_split: operands must be given and 16-byte aligned");
    NQ_REQUIRE(m * k < ((int64_t)1 << 31) && n * k < ((int64_t)1 << 31), NQ_ERR_SHAPE,
               "nq_bf16_gemm_split: operands of 2^31 elements or more are not supported");
    NQ_REQUIRE(tile >= -1 && tile <= 9, NQ_ERR_ARGUMENT, "nq_bf16_gemm_split: tile must be -1 (automatic) or 0..9");
    return nq::launch_bf16_gemm(a_bf16_dev, b_bf16_dev, outputs.out[0], (int)m, (int)n, (int)k, tile, 1, nullptr, 0,
                                (hipStream_t)stream, &outputs);
}
