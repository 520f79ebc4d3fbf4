// A decode step's row encoder and the packed linear that consumes its row, in one launch.
//
// In a decode step the encoder of a Linear's input (residual + RMSNorm, SwiGLU or the attention
// merge, then Hadamard, norm and the A4 encode) is a chain of latencies on a few compute units,
// and the linear behind it spends most of its time regenerating and decoding weights, work that
// does not depend on the activation.  Here the first `producers` workgroups of the grid are the
// encoder's (row_lanes_encode, the same device code as the stand-alone kernel), the others the
// linear's: a consumer decodes all of its weight blocks into registers first, then waits until
// every producer has flagged its slice of the decoded row, and only then multiplies.
//
// Hand-over.  Producers store the decoded BF16 row written through to memory at device scope
// (sc1), wait for those stores, meet at a barrier and set their flag word, also written through.
// One wavefront per consumer workgroup polls the flag words with device-scope loads and the
// consumers then read the row with device-scope loads: neither side needs a cache write-back or
// invalidation (the XCDs' L2 caches are not coherent with each other for ordinary accesses).
// Every launch owns its flag words and clears those of the launch before it on the stream, which
// has finished; nothing is counted, so nothing has to be reset by a last workgroup.
//
// Progress.  Workgroups are dispatched in index order, so every producer is resident before a
// consumer can occupy the slot it needs, and producers wait for nothing.  The consumers' wait is
// bounded all the same: after `spin_limit` polls a workgroup writes 1 to the status word, skips
// its outputs and exits; the host sees the status and goes back to two launches.
//
// Results are those of the two-launch form bit for bit: the encoder is the same code, and the
// consumers add the same products in the same order as w4a4_gemv_kernel (up to four rows, except
// for weights that fill the chip in 16-channel tiles) and w4a4_gemv_mfma_kernel (the rest).
// Replaces: FusedNQRTLinear.forward's input stage followed by its kernel dispatch
// (nestquant/models/fused_linear.py:287-306, 316-407).
#include "nq_rowlanes.hip.h"
#include "nq_linear_common.hip.h"

#include <math.h>

#ifdef NQ_PHASE_STAMPS
// Measuring builds only: lane 0 of the first and last producer and of the first and last consumer
// (slots 0 to 3, eight stamps each) leave the 100 MHz wall clock at their phase boundaries.
namespace nq { __device__ unsigned long long g_pair_stamps[32]; }
#define NQ_PAIR_STAMP(slot, i) do { if ((slot) >= 0 && threadIdx.x == 0) nq::g_pair_stamps[(slot) * 8 + (i)] = wall_clock64(); } while (0)
extern "C" int nq_debug_pair_stamps(unsigned long long *out32) {
    if (hipDeviceSynchronize() != hipSuccess) return NQ_ERR_LAUNCH;
    return hipMemcpyFromSymbol(out32, HIP_SYMBOL(nq::g_pair_stamps), 32 * sizeof(unsigned long long)) == hipSuccess
               ? NQ_OK : NQ_ERR_LAUNCH;
}
#else
#define NQ_PAIR_STAMP(slot, i) do { } while (0)
#endif

namespace nq {

// Every consumer workgroup polls the flags at once, and polls of one cache line queue up at the one
// memory channel that holds it: the flag words therefore exist in several copies, a producer sets
// its word in all of them (one store instruction) and consumer g reads copy g % copies.  A launch of
// up to 256 producers lays its kFlagWords out as 16 copies 256 words apart, a larger one (up to 512)
// as 8 copies 512 words apart.
constexpr int kFlagWords = 4096;
constexpr int kMaxProducers = 512;

struct PairSync {
    uint32_t *flags;         // copies x stride = kFlagWords words, one per producer workgroup and copy, zero when the launch starts
    int copies, stride;
    uint32_t *previous;      // the flag words of the launch before this one on the stream (cleared here), or null
    int previous_count;
    uint32_t *status;        // set to 1 when a consumer's wait runs out (device or pinned host memory)
    int spin_limit;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t load_word_device_scope(const uint32_t *at) {
    uint32_t value;
    asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(value) : "v"(at) : "memory");
    return value;
}

__device__ __forceinline__ void store_word_device_scope(uint32_t *at, uint32_t value) {
    asm volatile("global_store_dword %0, %1, off sc1" :: "v"(at), "v"(value) : "memory");
}

// Four consecutive 16-byte pieces from each of two addresses, read at device scope; returns when all
// eight have arrived.  (One statement: the compiler must not touch a destination before the wait.)
__device__ __forceinline__ void load_2x4_device_scope(const uint4 *a0, const uint4 *a1, u32x4 (&out)[2][4]) {
    asm volatile(
        "global_load_dwordx4 %0, %8, off sc1\n\t"
        "global_load_dwordx4 %1, %8, off offset:16 sc1\n\t"
        "global_load_dwordx4 %2, %8, off offset:32 sc1\n\t"
        "global_load_dwordx4 %3, %8, off offset:48 sc1\n\t"
        "global_load_dwordx4 %4, %9, off sc1\n\t"
        "global_load_dwordx4 %5, %9, off offset:16 sc1\n\t"
        "global_load_dwordx4 %6, %9, off offset:32 sc1\n\t"
        "global_load_dwordx4 %7, %9, off offset:48 sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(out[0][0]), "=&v"(out[0][1]), "=&v"(out[0][2]), "=&v"(out[0][3]), "=&v"(out[1][0]), "=&v"(out[1][1]),
          "=&v"(out[1][2]), "=&v"(out[1][3])
        : "v"(a0), "v"(a1)
        : "memory");
}

// One 16-byte piece from each of kCount (1, 2, 4 or 8) addresses, read at device scope.
template <int kCount>
__device__ __forceinline__ void load_pieces_device_scope(const uint4 *const (&at)[kCount], u32x4 (&out)[kCount]) {
    static_assert(kCount == 1 || kCount == 2 || kCount == 4 || kCount == 8, "1, 2, 4 or 8 pieces");
    if constexpr (kCount == 1) {
        asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(out[0]) : "v"(at[0]) : "memory");
    } else if constexpr (kCount == 2) {
        asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %3, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(out[0]), "=&v"(out[1]) : "v"(at[0]), "v"(at[1]) : "memory");
    } else if constexpr (kCount == 4) {
        asm volatile("global_load_dwordx4 %0, %4, off sc1\n\tglobal_load_dwordx4 %1, %5, off sc1\n\t"
                     "global_load_dwordx4 %2, %6, off sc1\n\tglobal_load_dwordx4 %3, %7, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(out[0]), "=&v"(out[1]), "=&v"(out[2]), "=&v"(out[3])
                     : "v"(at[0]), "v"(at[1]), "v"(at[2]), "v"(at[3]) : "memory");
    } else {
        asm volatile("global_load_dwordx4 %0, %8, off sc1\n\tglobal_load_dwordx4 %1, %9, off sc1\n\t"
                     "global_load_dwordx4 %2, %10, off sc1\n\tglobal_load_dwordx4 %3, %11, off sc1\n\t"
                     "global_load_dwordx4 %4, %12, off sc1\n\tglobal_load_dwordx4 %5, %13, off sc1\n\t"
                     "global_load_dwordx4 %6, %14, off sc1\n\tglobal_load_dwordx4 %7, %15, off sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(out[0]), "=&v"(out[1]), "=&v"(out[2]), "=&v"(out[3]), "=&v"(out[4]), "=&v"(out[5]),
                       "=&v"(out[6]), "=&v"(out[7])
                     : "v"(at[0]), "v"(at[1]), "v"(at[2]), "v"(at[3]), "v"(at[4]), "v"(at[5]), "v"(at[6]), "v"(at[7])
                     : "memory");
    }
}

// All lanes of a consumer workgroup: true once every producer's flag is set, false when the first
// wavefront's polls ran out (it has then written the status word).  Ends behind a barrier.  A poll is
// one 16-byte load per lane, two for more than 256 producers, both requested before either is waited
// for: four flag words each, so that the flags of a launch cost one trip to memory per poll (a load
// per flag and lane in turn made a poll of 256 flags four trips long).
__device__ __forceinline__ bool wait_for_producers(const PairSync &sync, int producers) {
    __shared__ __align__(16) int ready_shared[4];        // a multiple of 16 bytes, like every static array here
    if (threadIdx.x < 64) {
        const int first = 4 * (int)threadIdx.x;
        const uint32_t *flags = sync.flags + ((int)blockIdx.x % sync.copies) * sync.stride;
        const bool polls = first < producers;             // the flag words come in multiples of four
        const bool polls_twice = first + 256 < producers;
        int spins = 0;
        bool ready;
        for (;;) {
            u32x4 four = u32x4{1u, 1u, 1u, 1u}, more = u32x4{1u, 1u, 1u, 1u};
            if (polls_twice)
                asm volatile("global_load_dwordx4 %0, %2, off sc1\n\tglobal_load_dwordx4 %1, %2, off offset:1024 sc1\n\t"
                             "s_waitcnt vmcnt(0)" : "=&v"(four), "=&v"(more) : "v"(flags + first) : "memory");
            else if (polls)
                asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)"
                             : "=&v"(four) : "v"(flags + first) : "memory");
            const bool mine = four.x != 0u && four.y != 0u && four.z != 0u && four.w != 0u && more.x != 0u &&
                              more.y != 0u && more.z != 0u && more.w != 0u;
            ready = __builtin_amdgcn_ballot_w64(!mine) == 0;
            if (ready || ++spins > sync.spin_limit) break;
            __builtin_amdgcn_s_sleep(4);
        }
        if (threadIdx.x == 0) {
            ready_shared[0] = ready ? 1 : 0;
            if (!ready) __hip_atomic_store(sync.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
    __syncthreads();
    return ready_shared[0] != 0;
}

constexpr int kPairSubgroup = 256;       // lanes that share a group of channels in the vector form

// Vector-unit consumer (w4a4_gemv_kernel's products and sums): the workgroup's subgroups of 256 lanes
// own R channels each; lane t of a subgroup decodes blocks t, t + 256, ... of those channels.
template <int MT, int R, int kSteps>
__device__ __forceinline__ void
consume_on_vector_units(const uint4 *__restrict__ act, const GemvWeights &w, int which, int group, int m_rows, int k_size,
                        float sqrt_k, int out_is_f32, const PairSync &sync, int producers) {
    __shared__ float partial[4][16][R][MT];
    [[maybe_unused]] const int stamp_slot = (int)blockIdx.x == producers ? 2 : ((int)blockIdx.x == (int)gridDim.x - 1 ? 3 : -1);
    NQ_PAIR_STAMP(stamp_slot, 0);
    const int tid = threadIdx.x, sub = tid >> 8, t = tid & 255;
    const int subgroups = (int)blockDim.x >> 8;
    const int blocks_per_row = k_size >> 3;
    const int n_size = w.n[which];
    const int n0 = (group * subgroups + sub) * R;
    const float *betas = w.betas[which];
    const float wbeta[4] = {betas[0], betas[1], betas[2], betas[3]};
    const uint32_t *words = w.words[which];
    const uint16_t *tails = w.tails[which];
    const uint32_t seed_plus_offset = w.seed_plus_offset[which];

    // The weight words of a step are requested one step ahead, and a step's blocks are decoded before the
    // next step's words are unpacked: few registers beyond the decoded weights themselves stay live.
    uint32_t word_next[R], tail_next[R];
    int64_t row_first[R];
    ResolvedScales scaled_beta[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int n = n0 + r < n_size ? n0 + r : n_size - 1;        // channels past the end repeat the last one
        row_first[r] = (int64_t)n * blocks_per_row;
        word_next[r] = words[row_first[r] + t];
        tail_next[r] = (uint32_t)tails[row_first[r] + t];
        scaled_beta[r] = resolved_scales(wbeta, (w.norms[which][n] / sqrt_k) * kResolvedUnit);
    }
    uint32_t weight[kSteps][R][4];
#pragma unroll
    for (int s = 0; s < kSteps; s++) {
        uint32_t word[R], tail[R];
#pragma unroll
        for (int r = 0; r < R; r++) { word[r] = word_next[r]; tail[r] = tail_next[r]; }
        if (s + 1 < kSteps) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                word_next[r] = words[row_first[r] + t + kPairSubgroup * (s + 1)];
                tail_next[r] = (uint32_t)tails[row_first[r] + t + kPairSubgroup * (s + 1)];
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int64_t g = row_first[r] + t + kPairSubgroup * s;
            float v[8];
            decode_resolved(word[r], tail[r], seed_plus_offset + (uint32_t)g * 8u, resolved_scale(scaled_beta[r], word[r]), v);
#pragma unroll
            for (int j = 0; j < 4; j++) weight[s][r][j] = __builtin_bit_cast(uint32_t, pack_bf16x2(v[2 * j], v[2 * j + 1]));
            // packed here, not where the products are (the compiler would otherwise carry the eight floats across the wait)
            asm volatile("" : "+v"(weight[s][r][0]), "+v"(weight[s][r][1]), "+v"(weight[s][r][2]), "+v"(weight[s][r][3]));
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    NQ_PAIR_STAMP(stamp_slot, 1);
    const bool ready = wait_for_producers(sync, producers);
    NQ_PAIR_STAMP(stamp_slot, 2);

    float acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < MT; m++) acc[r][m] = 0.0f;
    if (ready) {
        // the activation blocks of (step, row), eight at a time at most; steps in order, as the sums want them
        constexpr int kPieces = kSteps * MT, kBatch = kPieces < 8 ? kPieces : 8, kStepsPerBatch = kBatch / MT;
#pragma unroll
        for (int first = 0; first < kSteps; first += kStepsPerBatch) {
            const uint4 *at[kBatch];
            u32x4 a[kBatch];
#pragma unroll
            for (int i = 0; i < kBatch; i++) {
                const int s = first + i / MT, m = i % MT;
                at[i] = act + (int64_t)(m < m_rows ? m : 0) * blocks_per_row + t + kPairSubgroup * s;
            }
            load_pieces_device_scope<kBatch>(at, a);
#pragma unroll
            for (int i = 0; i < kBatch; i++) {
                const int s = first + i / MT, m = i % MT;
                // by component: indexing the vector with the loop variable read component 0 four times
                const bool live = m < m_rows;
                const uint32_t row[4] = {live ? a[i].x : 0u, live ? a[i].y : 0u, live ? a[i].z : 0u, live ? a[i].w : 0u};
#pragma unroll
                for (int r = 0; r < R; r++) {
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        acc[r][m] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, row[j]),
                                                                    __builtin_bit_cast(bf16x2, weight[s][r][j]), acc[r][m], false);
                }
            }
        }
    }
    NQ_PAIR_STAMP(stamp_slot, 3);
    // sums over the 16 lanes of every row with register-only lane exchanges, then rows in index order
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const float v = row16_sum(acc[r][m]);
            if ((tid & 15) == 0) partial[sub][t >> 4][r][m] = v;
        }
    }
    __syncthreads();
    if (ready && t < R * MT) {
        const int r = t / MT, m = t - r * MT;
        const int n = n0 + r;
        if (n < n_size && m < m_rows) {
            float total = partial[sub][0][r][m];
#pragma unroll
            for (int i = 1; i < 16; i++) total = total + partial[sub][i][r][m];
            if (out_is_f32) reinterpret_cast<float *>(w.out[which])[(int64_t)m * n_size + n] = total;
            else reinterpret_cast<uint16_t *>(w.out[which])[(int64_t)m * n_size + n] = f32_to_bf16(total);
        }
    }
    NQ_PAIR_STAMP(stamp_slot, 4);
}

// Matrix-core consumer (w4a4_gemv_mfma_kernel<1>'s products and sums): a tile of 16 channels.  The
// stand-alone kernel runs kVirtual wavefronts on a K of this length, wavefront v taking the pieces of
// 128 k numbered v, v + kVirtual, ...; here a wavefront plays kVirtual / (lanes / 64) of them in turn,
// each with an accumulator of its own, so that the same pieces meet in the same order.
template <int kVirtualPerWave, int kStepsPerVirtual>
__device__ __forceinline__ void
consume_on_matrix_cores(const uint4 *__restrict__ act, const GemvWeights &w, int which, int tile, int m_rows, int k_size,
                        float sqrt_k, int out_is_f32, const PairSync &sync, int producers) {
    static_assert(kVirtualPerWave * kStepsPerVirtual == 4, "a lane holds sixteen decoded blocks");
    __shared__ float part[16][256];
    [[maybe_unused]] const int stamp_slot = (int)blockIdx.x == producers ? 2 : ((int)blockIdx.x == (int)gridDim.x - 1 ? 3 : -1);
    NQ_PAIR_STAMP(stamp_slot, 0);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = (int)blockDim.x >> 6;
    const int virtual_waves = waves * kVirtualPerWave;
    const int n_size = w.n[which], n0 = tile * 16;
    const int column = lane & 15, quarter = lane >> 4;
    const int blocks_per_row = k_size >> 3;
    const int n = n0 + column < n_size ? n0 + column : n_size - 1;      // channels past the end repeat the last one
    const float *betas = w.betas[which];
    const float wbeta[4] = {betas[0], betas[1], betas[2], betas[3]};
    const ResolvedScales scaled_beta = resolved_scales(wbeta, (w.norms[which][n] / sqrt_k) * kResolvedUnit);
    const uint32_t seed_plus_offset = w.seed_plus_offset[which];
    const int64_t row_first = (int64_t)n * blocks_per_row + 4 * quarter;
    const uint32_t *words = w.words[which];
    const uint16_t *tails = w.tails[which];

    // the words of a piece of K are requested one piece ahead of their decode
    const auto piece = [&](int e) { return wave + (e / kStepsPerVirtual) * waves + (e % kStepsPerVirtual) * virtual_waves; };
    uint4 word4_next = *reinterpret_cast<const uint4 *>(words + row_first + 16 * piece(0));
    uint2 tail2_next = *reinterpret_cast<const uint2 *>(tails + row_first + 16 * piece(0));
    uint4 a_fragment[4][4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const uint4 word4 = word4_next;
        const uint2 tail2 = tail2_next;
        if (e + 1 < 4) {
            word4_next = *reinterpret_cast<const uint4 *>(words + row_first + 16 * piece(e + 1));
            tail2_next = *reinterpret_cast<const uint2 *>(tails + row_first + 16 * piece(e + 1));
        }
        const uint32_t word[4] = {word4.x, word4.y, word4.z, word4.w};
        const uint32_t tail[4] = {tail2.x & 0xffffu, tail2.x >> 16, tail2.y & 0xffffu, tail2.y >> 16};
        const uint32_t first_counter = seed_plus_offset + (uint32_t)(row_first + 16 * piece(e)) * 8u;
        uint32_t bits[2][8];                     // the dither parts of two neighbouring blocks at a time
#pragma unroll
        for (int t = 0; t < 4; t++) {
            if (t % 2 == 0) resolved_dither_bits_run<2>(first_counter + 8u * t, bits);
            float x[8];
            resolved_apply(word[t], tail[t], bits[t % 2], resolved_scale(scaled_beta, word[t]), x);
            a_fragment[e][t] = make_uint4(__builtin_bit_cast(uint32_t, pack_bf16x2(x[0], x[1])),
                                          __builtin_bit_cast(uint32_t, pack_bf16x2(x[2], x[3])),
                                          __builtin_bit_cast(uint32_t, pack_bf16x2(x[4], x[5])),
                                          __builtin_bit_cast(uint32_t, pack_bf16x2(x[6], x[7])));
            // packed here, not where the products are (the compiler would otherwise carry the eight floats across the wait)
            asm volatile("" : "+v"(a_fragment[e][t].x), "+v"(a_fragment[e][t].y), "+v"(a_fragment[e][t].z), "+v"(a_fragment[e][t].w));
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    NQ_PAIR_STAMP(stamp_slot, 1);
    const bool ready = wait_for_producers(sync, producers);
    NQ_PAIR_STAMP(stamp_slot, 2);

    if (ready) {
        const bool has_token = column < m_rows;
        const uint4 *act_row = act + (int64_t)(has_token ? column : 0) * blocks_per_row + 4 * quarter;
        floatx4 acc = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        // the activation fragments of two pieces at a time (32 registers beside the 64 of decoded weights)
#pragma unroll
        for (int half = 0; half < 2; half++) {
            // lanes whose column is no token of this launch request nothing and multiply zeros
            u32x4 b[2][4];
#pragma unroll
            for (int pair = 0; pair < 2; pair++)
#pragma unroll
                for (int t = 0; t < 4; t++) b[pair][t] = u32x4{0u, 0u, 0u, 0u};
            if (has_token) load_2x4_device_scope(act_row + 16 * piece(2 * half), act_row + 16 * piece(2 * half + 1), b);
#pragma unroll
            for (int pair = 0; pair < 2; pair++) {
                const int e = 2 * half + pair;
                if (e % kStepsPerVirtual == 0) acc = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int t = 0; t < 4; t++)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a_fragment[e][t]),
                                                                  __builtin_bit_cast(bf16x8, b[pair][t]), acc, 0, 0, 0);
                if (e % kStepsPerVirtual == kStepsPerVirtual - 1) {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        part[wave + (e / kStepsPerVirtual) * waves][(4 * quarter + i) * 16 + column] = acc[i];
                }
            }
        }
    }
    NQ_PAIR_STAMP(stamp_slot, 3);
    __syncthreads();
    if (ready && tid < 256) {
        const int channel = tid >> 4, token = tid & 15;
        if (n0 + channel < n_size && token < m_rows) {
            float total = 0.0f;
            for (int p = 0; p < virtual_waves; p++) total = total + part[p][channel * 16 + token];
            const int64_t at = (int64_t)token * n_size + n0 + channel;
            if (out_is_f32) reinterpret_cast<float *>(w.out[which])[at] = total;
            else reinterpret_cast<uint16_t *>(w.out[which])[at] = f32_to_bf16(total);
        }
    }
    NQ_PAIR_STAMP(stamp_slot, 4);
}

struct EncoderArgs {
    const void *x;
    int64_t rows;
    int n;
    const float *betas;
    int beta_count;
    float sqrt_n;
    uint32_t *codes;
    uint8_t *beta_ids;
    float *norms;
    uint4 *decoded;
    int slices, rotate;
    InputPrologue prologue;
};

// kConsumer: 0 = vector units (MT rows, R channels per subgroup), 1 = matrix cores.
template <int kPrologue, int kForm, int kConsumer, int MT, int R>
__global__ void __launch_bounds__(kForm == kFirstLanes ? 1024 : 256)
fused_stage_linear_kernel(EncoderArgs e, GemvWeights w, int producers, int late_first, int late_count, int m_rows,
                          float sqrt_k, int out_is_f32, PairSync sync) {
    const int block = (int)blockIdx.x;
    int group = block - producers;
    if (block < producers) {
        __builtin_amdgcn_s_setprio(3);           // a chain of latencies that the consumers' vector work would stretch
        [[maybe_unused]] const int stamp_slot = block == 0 ? 0 : (block == producers - 1 ? 1 : -1);
        NQ_PAIR_STAMP(stamp_slot, 0);
        row_lanes_encode<kPrologue, kForm, true>(e.x, 0, e.rows, e.n, e.betas, e.beta_count, e.sqrt_n, e.codes, e.beta_ids,
                                                 e.norms, e.decoded, e.slices, e.rotate, e.prologue, block);
        NQ_PAIR_STAMP(stamp_slot, 1);
        __builtin_amdgcn_s_waitcnt(0);           // this wavefront's write-through stores have been acknowledged
        NQ_PAIR_STAMP(stamp_slot, 2);
        __syncthreads();
        NQ_PAIR_STAMP(stamp_slot, 3);
        if ((int)threadIdx.x < sync.copies) store_word_device_scope(sync.flags + (int)threadIdx.x * sync.stride + block, 1u);
        // the groups of channels that found no free slot beside the others are the producers' second job
        if (block >= late_count) return;
        __builtin_amdgcn_s_setprio(0);
        group = late_first + block;
    }
    // the flag words of the launch before this one (finished: it came earlier on the stream) are cleared
    // by a workgroup that has time to spare: the first consumer
    if (block == producers && sync.previous)
        for (int i = (int)threadIdx.x; i < sync.previous_count; i += (int)blockDim.x) sync.previous[i] = 0u;
    int which = 0;
#pragma unroll
    for (int i = 1; i < kGemvMaxGroup; i++)
        if (i < w.count && group >= w.first_group[i]) which = i;
    group -= w.first_group[which];
    const uint4 *act = e.decoded;
    if (kConsumer == 0) {
        constexpr int kSteps = kForm == kFirstLanes ? 4 : 1;       // n = 8192 : n = 2048
        consume_on_vector_units<MT, R, kSteps>(act, w, which, group, m_rows, e.n, sqrt_k, out_is_f32, sync, producers);
    } else {
        if (kForm == kFirstLanes) consume_on_matrix_cores<1, 4>(act, w, which, group, m_rows, e.n, sqrt_k, out_is_f32, sync, producers);
        else consume_on_matrix_cores<2, 2>(act, w, which, group, m_rows, e.n, sqrt_k, out_is_f32, sync, producers);
    }
}

}  // namespace nq

namespace {

constexpr int kComputeUnits = 256;

// mirrors the choice nq_w4a4_gemv_grouped makes between its two kernels
bool pair_takes_matrix_cores(int m, int64_t total_n) { return m >= NQ_MFMA_FROM_ROWS || total_n >= 16 * 512; }

template <int kPrologue, int kForm>
int launch_pair(const nq::EncoderArgs &e, const nq::GemvWeights &w, int consumer, int m_tile, int r, int producers,
                int consumers, int late, int m, float sqrt_k, int out_is_f32, const nq::PairSync &sync, size_t lds_bytes,
                hipStream_t stream) {
    using Kernel = void (*)(nq::EncoderArgs, nq::GemvWeights, int, int, int, int, float, int, nq::PairSync);
    Kernel kernel = nullptr;
#define NQ_PAIR(C, MT, R) (Kernel)nq::fused_stage_linear_kernel<kPrologue, kForm, C, MT, R>
    if (consumer == 1) kernel = NQ_PAIR(1, 1, 1);
    else if (r == 4) kernel = m_tile == 1 ? NQ_PAIR(0, 1, 4) : (m_tile == 2 ? NQ_PAIR(0, 2, 4) : NQ_PAIR(0, 4, 4));
    else kernel = m_tile == 1 ? NQ_PAIR(0, 1, 3) : (m_tile == 2 ? NQ_PAIR(0, 2, 3) : NQ_PAIR(0, 4, 3));
#undef NQ_PAIR
    if (lds_bytes > 48 * 1024) {
        hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (status != hipSuccess)
            return nq::fail(NQ_ERR_LAUNCH, "nq_fused_stage_linear: cannot reserve %zu bytes of LDS: %s", lds_bytes,
                            hipGetErrorString(status));
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)(producers + consumers - late)), dim3(e.n / 8), lds_bytes, stream, e, w,
                       producers, consumers - late, late, m, sqrt_k, out_is_f32, sync);
    return nq::check_launch("nq_fused_stage_linear");
}

}  // namespace

namespace {
// encoder workgroups of a launch: rows x slices (a multiple of four, at most kMaxProducers); `tiles`:
// the linear's workgroups when they take 16 channels each
int pair_producers(int64_t rows, int64_t n, int64_t tiles) {
    // rows of 8192 values: slices of 512 values, one pass each, up to eight rows; slices of 1024 values
    // beyond, so that the consumers still find free compute units beside the encoder
    if (n > 4096) return (int)(rows * (rows <= 8 ? n / 512 : n / 1024));
    // rows of 2048 values: 32 slices of one pass each up to eight rows, and beyond while the launch as
    // a whole still fits the chip (four 256-lane workgroups per compute unit); else 16 of two passes
    return (int)(rows * (rows * 32 <= 256 || rows * 32 + tiles <= 4 * kComputeUnits ? 32 : 16));
}
}  // namespace

extern "C" int nq_fused_stage_linear_flag_words(int64_t rows, int64_t n) {
    if (rows < 1 || rows > 16 || (n != 2048 && n != 8192)) return 0;
    return nq::kFlagWords;
}

extern "C" int nq_fused_stage_linear(
    const void *x_dev, int64_t rows, int64_t n, int mode, const void *residual_dev, void *residual_out_dev,
    const void *norm_weight_dev, float eps, const void *gate_dev, const void *attention_workspace_dev, int q_heads,
    int parts, void *staged_out_dev, const float *betas_dev, int beta_count, uint8_t *codes_dev, uint8_t *beta_ids_dev,
    float *norms_dev, void *decoded_bf16_dev, int count, const uint32_t *const *w_resolved_words_dev,
    const uint16_t *const *w_resolved_tails_dev, const float *const *w_norms_dev, const float *const *w_betas_dev,
    const int *w_n, const int64_t *weight_offsets, const int64_t *weight_seeds, void *const *out_dev, int out_dtype,
    uint32_t *flags_dev, uint32_t *previous_flags_dev, int previous_flag_words, uint32_t *status_dev, int spin_limit,
    void *stream) {
    NQ_REQUIRE(rows >= 1 && rows <= 16, NQ_ERR_SHAPE, "nq_fused_stage_linear: between 1 and 16 rows (a decode step)");
    NQ_REQUIRE(n == 2048 || n == 8192, NQ_ERR_SHAPE, "nq_fused_stage_linear: rows of 2048 or 8192 values, got %lld", (long long)n);
    NQ_REQUIRE(mode >= 0 && mode <= 4, NQ_ERR_ARGUMENT,
               "nq_fused_stage_linear: mode must be 0 (the rows as they are), 1 (residual + RMSNorm), 2 (SiLU(gate) * x), "
               "3 (attention merge) or 4 (the rows as they are, already rotated)");
    NQ_REQUIRE((mode != 0 && mode != 4) || x_dev, NQ_ERR_ARGUMENT, "nq_fused_stage_linear: modes 0 and 4 need the rows");
    NQ_REQUIRE(mode != 1 || (x_dev && norm_weight_dev && eps >= 0.0f && eps < 1.0f), NQ_ERR_ARGUMENT,
               "nq_fused_stage_linear: mode 1 needs the rows, the norm weight and an eps in [0, 1)");
    NQ_REQUIRE(mode != 2 || (x_dev && gate_dev), NQ_ERR_ARGUMENT, "nq_fused_stage_linear: mode 2 needs the rows and the gate rows");
    NQ_REQUIRE(mode != 3 || (attention_workspace_dev && q_heads >= 1 && (int64_t)q_heads * 64 == n && parts >= 1 && parts <= 512),
               NQ_ERR_ARGUMENT, "nq_fused_stage_linear: mode 3 needs the attention workspace, heads * 64 = n and 1..512 parts");
    NQ_REQUIRE(nq::aligned(x_dev, 16) && nq::aligned(residual_dev, 16) && nq::aligned(residual_out_dev, 16) &&
                   nq::aligned(norm_weight_dev, 16) && nq::aligned(gate_dev, 16) && nq::aligned(staged_out_dev, 16) &&
                   nq::aligned(attention_workspace_dev, 16),
               NQ_ERR_ARGUMENT, "nq_fused_stage_linear: rows must be 16-byte aligned");
    NQ_REQUIRE(betas_dev && beta_count == 4 && codes_dev && beta_ids_dev && norms_dev && decoded_bf16_dev, NQ_ERR_ARGUMENT,
               "nq_fused_stage_linear: needs a table of four betas and the four outputs of the encoder");
    NQ_REQUIRE(nq::aligned(codes_dev, 4) && nq::aligned(decoded_bf16_dev, 16), NQ_ERR_ARGUMENT,
               "nq_fused_stage_linear: codes need 4-byte, the decoded row 16-byte alignment");
    NQ_REQUIRE(count >= 1 && count <= nq::kGemvMaxGroup, NQ_ERR_SHAPE, "nq_fused_stage_linear: between 1 and %d weights",
               nq::kGemvMaxGroup);
    NQ_REQUIRE(w_resolved_words_dev && w_resolved_tails_dev && w_norms_dev && w_betas_dev && w_n && weight_offsets &&
                   weight_seeds && out_dev, NQ_ERR_ARGUMENT, "nq_fused_stage_linear: null argument array");
    NQ_REQUIRE(out_dtype == NQ_F32 || out_dtype == NQ_BF16, NQ_ERR_ARGUMENT,
               "nq_fused_stage_linear: output dtype tag %d is not F32 or BF16", out_dtype);
    NQ_REQUIRE(flags_dev && status_dev && nq::aligned(flags_dev, 16) && nq::aligned(previous_flags_dev, 4) &&
                   nq::aligned(status_dev, 4), NQ_ERR_ARGUMENT,
               "nq_fused_stage_linear: needs flag words (16-byte aligned) and a status word");
    NQ_REQUIRE(previous_flag_words >= 0 && previous_flag_words <= 65536 && (previous_flag_words == 0 || previous_flags_dev),
               NQ_ERR_ARGUMENT, "nq_fused_stage_linear: at most 65536 flag words of the launch before");
    NQ_REQUIRE(spin_limit >= 0, NQ_ERR_ARGUMENT, "nq_fused_stage_linear: spin_limit must not be negative");

    const int k = (int)n;
    int64_t total_n = 0;
    for (int i = 0; i < count; i++) {
        NQ_REQUIRE(w_n[i] >= 1, NQ_ERR_SHAPE, "nq_fused_stage_linear: N must be positive");
        total_n += w_n[i];
    }
    const int m = (int)rows;
    const int consumer = pair_takes_matrix_cores(m, total_n) ? 1 : 0;
    int64_t tiles = 0;
    for (int i = 0; i < count; i++) tiles += (w_n[i] + 15) / 16;
    const int producers = pair_producers(rows, n, tiles);
    const int slices = producers / m;
    const int lanes = k / 8, subgroups = lanes / nq::kPairSubgroup;
    // Every workgroup of the launch must be resident at once: a consumer that started after another
    // had finished would pay the whole of its decode behind the encoder instead of beside it.  A
    // 256-lane workgroup fits four times on a compute unit, a 1024-lane one once (its row needs 66 KB
    // of LDS); the vector form takes as few channels per subgroup as that allows.
    const int slots = kComputeUnits * (lanes == 256 ? 4 : 1);
    int r = 3;
    if (consumer == 0)
        while (r < 4 && producers + (total_n + (int64_t)r * subgroups - 1) / ((int64_t)r * subgroups) + count > slots) r++;
    const int per_group = consumer == 1 ? 16 : r * subgroups;
    nq::GemvWeights w{};
    w.count = count;
    int groups = 0;
    for (int i = 0; i < count; i++) {
        NQ_REQUIRE(w_resolved_words_dev[i] && w_resolved_tails_dev[i] && w_norms_dev[i] && w_betas_dev[i] && out_dev[i],
                   NQ_ERR_ARGUMENT, "nq_fused_stage_linear: null pointer in weight %d", i);
        NQ_REQUIRE(nq::aligned(w_resolved_words_dev[i], 16) && nq::aligned(w_resolved_tails_dev[i], 8), NQ_ERR_ARGUMENT,
                   "nq_fused_stage_linear: resolved streams of weight %d need 16- and 8-byte alignment", i);
        NQ_REQUIRE(weight_seeds[i] >= 0 && weight_seeds[i] < ((int64_t)1 << 31), NQ_ERR_ARGUMENT,
                   "nq_fused_stage_linear: seed must be in [0, 2**31)");
        NQ_REQUIRE(weight_offsets[i] >= 0 && weight_offsets[i] + (int64_t)w_n[i] * (k / 8) <= ((int64_t)1 << 28),
                   NQ_ERR_SHAPE, "nq_fused_stage_linear: block range exceeds the stateless dither counter space");
        w.words[i] = w_resolved_words_dev[i];
        w.tails[i] = w_resolved_tails_dev[i];
        w.norms[i] = w_norms_dev[i];
        w.betas[i] = w_betas_dev[i];
        w.out[i] = out_dev[i];
        w.n[i] = w_n[i];
        w.first_group[i] = groups;
        w.seed_plus_offset[i] = (uint32_t)((uint64_t)weight_seeds[i] + (uint64_t)weight_offsets[i] * 8u);
        groups += (w_n[i] + per_group - 1) / per_group;
    }

    nq::EncoderArgs e{};
    e.x = mode == 3 ? attention_workspace_dev : x_dev;
    e.rows = rows;
    e.n = k;
    e.betas = betas_dev;
    e.beta_count = beta_count;
    e.sqrt_n = (float)sqrt((double)k);
    e.codes = reinterpret_cast<uint32_t *>(codes_dev);
    e.beta_ids = beta_ids_dev;
    e.norms = norms_dev;
    e.decoded = reinterpret_cast<uint4 *>(decoded_bf16_dev);
    e.slices = slices;
    e.rotate = mode == 4 ? 0 : 1;
    e.prologue.residual = reinterpret_cast<const uint16_t *>(residual_dev);
    e.prologue.weight = reinterpret_cast<const uint16_t *>(norm_weight_dev);
    e.prologue.gate = reinterpret_cast<const uint16_t *>(gate_dev);
    e.prologue.residual_out = reinterpret_cast<uint16_t *>(residual_out_dev);
    e.prologue.normed_out = reinterpret_cast<uint16_t *>(staged_out_dev);
    e.prologue.eps = eps;
    if (mode == 3) {
        const size_t heads_total = (size_t)rows * q_heads;
        e.prologue.part_max = reinterpret_cast<const float *>(attention_workspace_dev);
        e.prologue.part_sum = e.prologue.part_max + heads_total * parts;
        e.prologue.part_acc = e.prologue.part_sum + heads_total * parts;
        e.prologue.parts = parts;
        e.prologue.heads = q_heads;
    }
    // Groups of channels beyond the slots of the chip would start when others finish and pay their
    // whole decode behind the rest of the launch: as many of them as there are producers become the
    // producers' second job (an encoder workgroup is done long before the first consumer).
    const int late = groups + producers > slots ? (groups + producers - slots < producers ? groups + producers - slots : producers) : 0;
    const int flag_stride = producers > 256 ? nq::kMaxProducers : 256;
    nq::PairSync sync{flags_dev, nq::kFlagWords / flag_stride, flag_stride, previous_flags_dev, previous_flag_words, status_dev,
                      spin_limit};
    const size_t lds_bytes = (size_t)(8 * ((k >> 3) + 8) + k + 4 + 8) * sizeof(float);
    const float sqrt_k = (float)sqrt((double)k);
    const int m_tile = m == 1 ? 1 : (m == 2 ? 2 : 4);
    const int out_is_f32 = out_dtype == NQ_F32;
    hipStream_t s = (hipStream_t)stream;
#define NQ_LAUNCH_PAIR(PRO, FORM) \
    launch_pair<PRO, FORM>(e, w, consumer, m_tile, r, producers, groups, late, m, sqrt_k, out_is_f32, sync, lds_bytes, s)
    if (k == 8192) {
        if (mode == 0 || mode == 4) return NQ_LAUNCH_PAIR(0, nq::kFirstLanes);
        if (mode == 1) return NQ_LAUNCH_PAIR(1, nq::kFirstLanes);
        if (mode == 2) return NQ_LAUNCH_PAIR(2, nq::kFirstLanes);
        return NQ_LAUNCH_PAIR(3, nq::kFirstLanes);
    }
    if (mode == 0 || mode == 4) return NQ_LAUNCH_PAIR(0, nq::kEightLanes);
    if (mode == 1) return NQ_LAUNCH_PAIR(1, nq::kEightLanes);
    if (mode == 2) return NQ_LAUNCH_PAIR(2, nq::kEightLanes);
    return NQ_LAUNCH_PAIR(3, nq::kEightLanes);
#undef NQ_LAUNCH_PAIR
}
