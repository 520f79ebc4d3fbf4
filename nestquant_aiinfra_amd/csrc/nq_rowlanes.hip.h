// The decode-step row encoder (one lane per eight neighbouring values) as device code, so that it can
// run as a kernel of its own (nq_codec.hip) and as the producing part of a launch whose other
// workgroups are the linear that consumes the row (nq_fused_pair.hip).
// Reference: nestquant/core/quantizer.py:214-301, nestquant/runtime/nqkv_page.py:97-185,
// nestquant/models/fused_linear.py:287-306.
#pragma once

#include "nq_rowquant.hip.h"

namespace nq {

// Optional element-wise stage in front of the quantiser (BF16 rows only), in the arithmetic
// of BF16 tensor operations: every tensor-level result is rounded to BF16.
//   mode 1  h = x + residual (residual may be null); residual_out = h;
//           y = weight * bf16(h * rsqrt(mean(h^2) + eps))      (LlamaRMSNorm)
//   mode 2  y = bf16(silu(gate)) * x                            (the SwiGLU product)
//   mode 3  y = the attention output [rows, heads * 64] merged from the per-chunk partial results
//           of the decode attention (online-softmax maxima, sums and numerators of `parts` chunks
//           per head), rounded to BF16: stage 2 of the attention, done where its result is consumed
// normed_out (optional) receives y; rows are then rotated / quantised as usual.
struct InputPrologue {
    const uint16_t *residual, *weight, *gate;
    uint16_t *residual_out, *normed_out;
    float eps;
    const float *part_max, *part_sum, *part_acc;       // mode 3: [rows * heads][parts] (x 64 for part_acc)
    int parts, heads;
};


__device__ __forceinline__ void unpack_bf16x8(const uint4 raw, float (&v)[8]) {
    v[0] = __uint_as_float(raw.x << 16); v[1] = __uint_as_float(raw.x & 0xffff0000u);
    v[2] = __uint_as_float(raw.y << 16); v[3] = __uint_as_float(raw.y & 0xffff0000u);
    v[4] = __uint_as_float(raw.z << 16); v[5] = __uint_as_float(raw.z & 0xffff0000u);
    v[6] = __uint_as_float(raw.w << 16); v[7] = __uint_as_float(raw.w & 0xffff0000u);
}

// eight float32 values -> packed BF16, round to nearest even
__device__ __forceinline__ uint4 pack_bf16x8(const float (&v)[8]) {
    return make_uint4(__builtin_bit_cast(uint32_t, pack_bf16x2(v[0], v[1])), __builtin_bit_cast(uint32_t, pack_bf16x2(v[2], v[3])),
                      __builtin_bit_cast(uint32_t, pack_bf16x2(v[4], v[5])), __builtin_bit_cast(uint32_t, pack_bf16x2(v[6], v[7])));
}

// eight float32 values that are exact BF16 numbers -> packed BF16
__device__ __forceinline__ uint4 pack_bf16x8_exact(const float (&v)[8]) {
    return make_uint4((__float_as_uint(v[0]) >> 16) | (__float_as_uint(v[1]) & 0xffff0000u),
                      (__float_as_uint(v[2]) >> 16) | (__float_as_uint(v[3]) & 0xffff0000u),
                      (__float_as_uint(v[4]) >> 16) | (__float_as_uint(v[5]) & 0xffff0000u),
                      (__float_as_uint(v[6]) >> 16) | (__float_as_uint(v[7]) & 0xffff0000u));
}

// ---------------------------------------------------------------------------------------
// One BF16 row per launch slice, one lane per eight neighbouring values (n / 8 lanes, n a power of
// two from 2048 to 8192, q = 14): the form for decode steps, where the latency of one row is all
// that counts.  The row never makes the trip through LDS that the general kernel's phases are built
// around:
//   * the element-wise stage (residual + RMSNorm, SwiGLU, attention merge) runs on the lane's eight
//     values in registers; the RMS sum is a sum per lane, a DPP tree per wavefront, one barrier;
//   * the rotation's butterflies of distance 1 .. 256 follow in the same registers (hadamard_chunk);
//     rows above 512 values need one pass through LDS for the distances from 512 up;
//   * the last writer leaves the row in LDS transposed -- element i at (i % 8) * pitch + i / 8 -- so
//     that each of the eight fused-multiply-add chains of the row norm (element i feeds chain i % 8)
//     reads its operands four at a time with 128-bit loads instead of one 32-bit load per step;
//   * the wavefronts that encode run the chains themselves (no hand-over through LDS), and divide
//     by beta through its reciprocal where that gives the IEEE quotient.
// Every workgroup of a row repeats all of this and encodes its own slice of the blocks.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float wave_sum_in_lane_order(float v) {
    // sum over the 64 lanes: pairs, quads, eights and sixteens by DPP, then the four rows of 16 in order
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    const int bits = __builtin_bit_cast(int, v);
    return ((__builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0)) +
             __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16))) +
            __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32))) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
}

// The lane's eight values after the element-wise stage of `pro` (see InputPrologue); g is the index
// of the first of them in the row-major input.  Mode 1 needs the whole workgroup (one barrier);
// `wave_sums` is LDS for one float per wavefront.
template <int kPrologue>
__device__ __forceinline__ void lane_prologue(const uint16_t *__restrict__ x, const InputPrologue &pro, int64_t row, int n,
                                              bool writes_outputs, float *wave_sums, float (&y)[8]) {
    const int chunk = threadIdx.x;
    const int64_t g = row * n + 8 * chunk;
    if (kPrologue == 3) {
        // Parts are taken four at a time, and the next four are requested before the current four are
        // used: the workspace was written by the previous launch on other XCDs, so a round of loads
        // costs over a microsecond and the rounds of a long table would otherwise add up.
        constexpr int kBatch = 4;
        const float kNone = -__builtin_inff();
#pragma unroll
        for (int j = 0; j < 8; j++) y[j] = 0.0f;
        const int64_t head = row * pro.heads + (chunk >> 3);      // eight lanes per head of 64
        const float *m = pro.part_max + head * pro.parts, *sum = pro.part_sum + head * pro.parts;
        const float *acc = pro.part_acc + head * pro.parts * 64 + 8 * (chunk & 7);
        struct Batch { float mc[kBatch], sc[kBatch]; float4 lo[kBatch], hi[kBatch]; };
        const auto request = [&](int c0, Batch &b) {
#pragma unroll
            for (int j = 0; j < kBatch; j++) {
                const int c = min(c0 + j, pro.parts - 1);
                b.mc[j] = m[c];
                b.sc[j] = sum[c];
                b.lo[j] = *reinterpret_cast<const float4 *>(acc + (int64_t)c * 64);
                b.hi[j] = *reinterpret_cast<const float4 *>(acc + (int64_t)c * 64 + 4);
            }
        };
        float top = kNone, denom = 0.0f;
        const auto fold = [&](int c0, Batch &b) {
            float batch_top = kNone;
#pragma unroll
            for (int j = 0; j < kBatch; j++) {
                if (c0 + j >= pro.parts) b.sc[j] = 0.0f;
                batch_top = fmaxf(batch_top, b.mc[j]);
            }
            const float next_top = fmaxf(top, batch_top);
            if (next_top > kNone) {
                const float keep = top > kNone ? __expf(top - next_top) : 0.0f;
                denom = denom * keep;
#pragma unroll
                for (int i = 0; i < 8; i++) y[i] = y[i] * keep;
#pragma unroll
                for (int j = 0; j < kBatch; j++) {
                    const float w = b.sc[j] > 0.0f ? __expf(b.mc[j] - next_top) : 0.0f;
                    denom = denom + b.sc[j] * w;
                    const bool used = w > 0.0f;
                    y[0] += used ? b.lo[j].x * w : 0.0f; y[1] += used ? b.lo[j].y * w : 0.0f;
                    y[2] += used ? b.lo[j].z * w : 0.0f; y[3] += used ? b.lo[j].w * w : 0.0f;
                    y[4] += used ? b.hi[j].x * w : 0.0f; y[5] += used ? b.hi[j].y * w : 0.0f;
                    y[6] += used ? b.hi[j].z * w : 0.0f; y[7] += used ? b.hi[j].w * w : 0.0f;
                }
                top = next_top;
            }
        };
        Batch even, odd;
        request(0, even);
        for (int c0 = 0; c0 < pro.parts; c0 += 2 * kBatch) {
            if (c0 + kBatch < pro.parts) request(c0 + kBatch, odd);
            fold(c0, even);
            if (c0 + kBatch >= pro.parts) break;
            if (c0 + 2 * kBatch < pro.parts) request(c0 + 2 * kBatch, even);
            fold(c0 + kBatch, odd);
        }
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            y[j] = denom > 0.0f ? y[j] / denom : 0.0f;               // inactive or empty rows give zeros
            y[j + 1] = denom > 0.0f ? y[j + 1] / denom : 0.0f;
            round_pair<1>(y[j], y[j + 1]);
        }
        if (writes_outputs && pro.normed_out) reinterpret_cast<uint4 *>(pro.normed_out)[g >> 3] = pack_bf16x8_exact(y);
        return;
    }
    // every global operand is requested before any is used: one memory round trip
    const uint4 zero = make_uint4(0, 0, 0, 0);
    const uint4 raw_x = reinterpret_cast<const uint4 *>(x)[g >> 3];
    uint4 raw_a = zero, raw_w = zero;
    if (kPrologue == 1) {
        if (pro.residual) raw_a = reinterpret_cast<const uint4 *>(pro.residual)[g >> 3];
        raw_w = reinterpret_cast<const uint4 *>(pro.weight)[chunk];
    } else if (kPrologue == 2) {
        raw_a = reinterpret_cast<const uint4 *>(pro.gate)[g >> 3];
    }
    unpack_bf16x8(raw_x, y);
    if (kPrologue == 0) return;
    float a[8];
    unpack_bf16x8(raw_a, a);
    if (kPrologue == 2) {
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            float s0 = a[j] / (1.0f + __expf(-a[j])), s1 = a[j + 1] / (1.0f + __expf(-a[j + 1]));
            round_pair<1>(s0, s1);
            y[j] = s0 * y[j];
            y[j + 1] = s1 * y[j + 1];
            round_pair<1>(y[j], y[j + 1]);
        }
        if (writes_outputs && pro.normed_out) reinterpret_cast<uint4 *>(pro.normed_out)[g >> 3] = pack_bf16x8_exact(y);
        return;
    }
    // LlamaRMSNorm: bf16(weight * bf16(h * rsqrt(mean(h^2) + eps))) with h = x + residual
    if (pro.residual) {
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            y[j] = y[j] + a[j];
            y[j + 1] = y[j + 1] + a[j + 1];
            round_pair<1>(y[j], y[j + 1]);
        }
    }
    if (writes_outputs && pro.residual_out) reinterpret_cast<uint4 *>(pro.residual_out)[g >> 3] = pack_bf16x8_exact(y);
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) sum = __builtin_fmaf(y[j], y[j], sum);
    sum = wave_sum_in_lane_order(sum);
    const int waves = (int)(blockDim.x >> 6);
    if ((threadIdx.x & 63) == 0) wave_sums[threadIdx.x >> 6] = sum;
    __syncthreads();
    float total = 0.0f;
    for (int w = 0; w < waves; w++) total = total + wave_sums[w];
    const float scale = 1.0f / __builtin_sqrtf(total / (float)n + pro.eps);
    float w[8];
    unpack_bf16x8(raw_w, w);
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
        y[j] = y[j] * scale;
        y[j + 1] = y[j + 1] * scale;
        round_pair<1>(y[j], y[j + 1]);
        y[j] = w[j] * y[j];
        y[j + 1] = w[j + 1] * y[j + 1];
        round_pair<1>(y[j], y[j + 1]);
    }
    if (writes_outputs && pro.normed_out) reinterpret_cast<uint4 *>(pro.normed_out)[g >> 3] = pack_bf16x8_exact(y);
}

// Pitch (floats) of one chain of the transposed row: 8 more than the chain's length, so that the
// lanes of a wavefront fall into different banks whether they write chains side by side or read
// along them.
__device__ __forceinline__ int chain_pitch(int n) { return (n >> 3) + 8; }

// The rotation's butterflies of distance 512 .. 2^(8 + S) on a row of 2^(9 + S) values staged in
// order in `natural`, then the scale by `inv`: work item t takes the 2^S values t, t + 512, ... (all
// of chain t % 8) and leaves them in the transposed row `chains`.  Every result is rounded to BF16.
template <int S>
__device__ __forceinline__ void late_stages_to_chains(const float *natural, float *chains, int pitch, float inv) {
    constexpr int kValues = 1 << S;
    for (int t = threadIdx.x; t < 512; t += blockDim.x) {
        float u[kValues];
#pragma unroll
        for (int j = 0; j < kValues; j++) u[j] = natural[t + (j << 9)];
#pragma unroll
        for (int s = 0; s < S; s++) {
#pragma unroll
            for (int j = 0; j < kValues; j++) {
                if (j & (1 << s)) continue;
                const float left = u[j], right = u[j + (1 << s)];
                u[j] = left + right;
                u[j + (1 << s)] = left - right;
                round_pair<1>(u[j], u[j + (1 << s)]);
            }
        }
#pragma unroll
        for (int j = 0; j < kValues; j += 2) {
            u[j] = u[j] * inv;
            u[j + 1] = u[j + 1] * inv;
            round_pair<1>(u[j], u[j + 1]);
        }
        float *out = chains + (t & 7) * pitch + (t >> 3);
#pragma unroll
        for (int j = 0; j < kValues; j++) out[j << 6] = u[j];
    }
}

enum LaneEncodeForm { kEightLanes = 0, kFirstLanes = 1, kEveryLane = 2, kBlockLanes = 3 };

// Stores of the decoded BF16 row.  kCoherent: written through to memory at device scope (sc1), for a
// launch whose other workgroups, on other XCDs with L2 caches of their own, read the row while this
// kernel is still running (they read it with device-scope loads after a flag says it is complete).
template <bool kCoherent>
__device__ __forceinline__ void store_decoded(uint4 *at, const uint4 value) {
    if (kCoherent) {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 v = {value.x, value.y, value.z, value.w};
        asm volatile("global_store_dwordx4 %0, %1, off sc1" :: "v"(at), "v"(v) : "memory");
    } else {
        *at = value;
    }
}
template <bool kCoherent>
__device__ __forceinline__ void store_decoded(uint16_t *at, const uint16_t value) {
    if (kCoherent) asm volatile("global_store_short %0, %1, off sc1" :: "v"(at), "v"((uint32_t)value) : "memory");
    else *at = value;
}

// The work of workgroup `block_index` of a launch of rows * slices workgroups of n / 8 lanes.
template <int kPrologue, int kForm, bool kCoherent = false>
__device__ __forceinline__ void
row_lanes_encode(const void *__restrict__ x_any, int x_is_f32, int64_t rows, int n, const float *__restrict__ betas,
                 int beta_count, float sqrt_n, uint32_t *__restrict__ codes, uint8_t *__restrict__ beta_ids,
                 float *__restrict__ norms, uint4 *__restrict__ decoded, int slices, int rotate,
                 const InputPrologue &pro, int block_index) {
    // 16-byte aligned whatever static LDS the kernel around this code declares: the chains are read 128 bits
    // at a time, and such reads from an address that is not a multiple of 16 take eight times as long
    extern __shared__ __align__(16) float lds[];
    const int pitch = chain_pitch(n);
    float *chains = lds;                                  // 8 * pitch floats: the row, transposed
    float *natural = chains + 8 * pitch;                  // n floats: the row in order (rows above 512 values, rotated)
    // behind them (static LDS of odd size would be laid out in front of the dynamic part and leave the
    // chains, which are read 128 bits at a time, misaligned): the row norm and a pass's beta choices
    float *row_norm_shared = natural + n;
    uint8_t *chosen = reinterpret_cast<uint8_t *>(natural + n + 4);       // 32 entries
    __shared__ float wave_sums[16];
    const int tid = threadIdx.x, lane = tid & 63;
    const int slice = block_index % slices;
    const int64_t row = block_index / slices;
    const int log_n = 31 - __builtin_clz(n);
    // How the slice's (block, beta) pairs meet the lanes (kForm, one instantiation each):
    //   kEightLanes  eight lanes per pair, lane c the block's coordinate c, beta (lane / 8) % 4: a quarter
    //                of the instructions per lane, the shortest path for the few rows of a decode step
    //                (rows of up to 4096 values; with the sixteen wavefronts of an 8192-value row that
    //                would be four encoding wavefronts per SIMD taking turns);
    //   kFirstLanes  one lane per pair on the first four wavefronts, one per SIMD (256 pairs a slice):
    //                an 8192-value row of a decode step;
    //   kEveryLane   one lane per pair on every lane, blockDim pairs at a time (four slices a row, fewer
    //                and several turns when that would be more than two workgroups of an 8192-value row
    //                per compute unit): for prefills of some tens of rows;
    //   kBlockLanes  one lane per block, its betas in turn, only the winner turned into a code word and
    //                the coset reduction skipped where every block of the wavefront lies inside the
    //                Voronoi cell (quantize_block_betas_in_turn): the fewest instructions per block, for
    //                hundreds of rows and more, one workgroup a row.
    constexpr bool eight_lanes = kForm == kEightLanes;
    const int c = lane & 7, bi = eight_lanes ? (lane >> 3) & 3 : tid & 3;
    const bool live = bi < beta_count;
    // requested first, used last; a launch that only runs the element-wise stage has no table
    const float beta = codes != nullptr ? betas[live ? bi : 0] : 1.0f;
    NQ_STAMP(0);

    float v[8];
    if (kForm == kBlockLanes && kPrologue == 0 && x_is_f32) {      // plain float32 rows (never rotated here)
        const float4 *at = reinterpret_cast<const float4 *>(x_any) + ((row * n) >> 2) + 2 * tid;
        const float4 lo = at[0], hi = at[1];
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
    } else {
        lane_prologue<kPrologue>(reinterpret_cast<const uint16_t *>(x_any), pro, row, n, slice == 0, wave_sums, v);
    }
    if (codes == nullptr) return;                         // element-wise stage only
    NQ_STAMP(1);

    const bool late_stages = rotate && log_n > 9;
    if (rotate) hadamard_chunk<1>(v, lane, log_n - 3 < 6 ? log_n - 3 : 6, log_n <= 9, 1.0f / __builtin_sqrtf((float)n));
    NQ_STAMP(8);
    if (late_stages) {
        *reinterpret_cast<float4 *>(natural + 8 * tid) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(natural + 8 * tid + 4) = make_float4(v[4], v[5], v[6], v[7]);
        __syncthreads();
        NQ_STAMP(9);
        const float inv = 1.0f / __builtin_sqrtf((float)n);
        switch (log_n - 9) {
            case 1: late_stages_to_chains<1>(natural, chains, pitch, inv); break;
            case 2: late_stages_to_chains<2>(natural, chains, pitch, inv); break;
            case 3: late_stages_to_chains<3>(natural, chains, pitch, inv); break;
            default: late_stages_to_chains<4>(natural, chains, pitch, inv); break;
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) chains[j * pitch + tid] = v[j];
    }
    __syncthreads();
    NQ_STAMP(2);

    // row norm in the reference's order (quantizer.py:257): chain k sums the squares of elements
    // k, k + 8, ... with fused multiply-adds; chains added 0..7; sqrt.  The first four wavefronts (one
    // per SIMD: the chain is a latency, and wavefronts that shared a SIMD would take turns) run it,
    // lanes 8 .. 63 running along (on chain lane % 8) so that the wavefront stays uniform; the others
    // get the result through LDS.
    float norm = 0.0f;
    if (tid < 256) {
        const float4 *chain = reinterpret_cast<const float4 *>(chains + (lane & 7) * pitch);
        const int quads = n >> 5;                          // 128-bit loads per chain, a multiple of 16
        float acc = 0.0f;
        // Batches of 32 chain steps, double-buffered by hand: the next batch is requested from LDS
        // before the chain runs over the current one.  The address of a request waits for the chain
        // (adding zero unless the sum is NaN), so that it reuses the registers the chain has just
        // released and the loop carries no copies.
        float4 a[8], b[8];
#pragma unroll
        for (int k = 0; k < 8; k++) a[k] = chain[k];
        int at = 0;
        for (; at + 16 < quads; at += 16) {
#pragma unroll
            for (int k = 0; k < 8; k++) b[k] = chain[at + 8 + k];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                acc = __builtin_fmaf(a[k].x, a[k].x, acc);
                acc = __builtin_fmaf(a[k].y, a[k].y, acc);
                acc = __builtin_fmaf(a[k].z, a[k].z, acc);
                acc = __builtin_fmaf(a[k].w, a[k].w, acc);
            }
            __builtin_amdgcn_sched_barrier(0);
            const float4 *next = chain + at + 16 + (acc != acc ? 1 : 0);
#pragma unroll
            for (int k = 0; k < 8; k++) a[k] = next[k];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k = 0; k < 8; k++) {
                acc = __builtin_fmaf(b[k].x, b[k].x, acc);
                acc = __builtin_fmaf(b[k].y, b[k].y, acc);
                acc = __builtin_fmaf(b[k].z, b[k].z, acc);
                acc = __builtin_fmaf(b[k].w, b[k].w, acc);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int k = 0; k < 8; k++) b[k] = chain[at + 8 + k];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            acc = __builtin_fmaf(a[k].x, a[k].x, acc);
            acc = __builtin_fmaf(a[k].y, a[k].y, acc);
            acc = __builtin_fmaf(a[k].z, a[k].z, acc);
            acc = __builtin_fmaf(a[k].w, a[k].w, acc);
        }
#pragma unroll
        for (int k = 0; k < 8; k++) {
            acc = __builtin_fmaf(b[k].x, b[k].x, acc);
            acc = __builtin_fmaf(b[k].y, b[k].y, acc);
            acc = __builtin_fmaf(b[k].z, b[k].z, acc);
            acc = __builtin_fmaf(b[k].w, b[k].w, acc);
        }
        NQ_STAMP(10);
        float total = 0.0f;
        const int bits = __builtin_bit_cast(int, acc);
#pragma unroll
        for (int k = 0; k < 8; k++) total = total + __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, k));
        norm = __builtin_sqrtf(total);
        if (tid == 0) *row_norm_shared = norm;
    }
    if (kForm == kFirstLanes && tid >= 256) return;
    if (kForm != kFirstLanes && blockDim.x > 256) {
        __syncthreads();
        norm = *row_norm_shared;
    }
    // math.sqrt(n) / norm is evaluated as (1 / norm) * float32(sqrt(n))
    const float scale = norm > 0.0f ? (1.0f / norm) * sqrt_n : 0.0f;
    if (slice == 0 && tid == 0) norms[row] = norm;
    NQ_STAMP(3);

    if (!eight_lanes) {
        // one lane per (block, beta) pair of the slice, blockDim pairs at a time
        struct LaneSink {
            uint32_t *codes; uint8_t *beta_ids; uint4 *decoded; int64_t first_block; float back;
            __device__ __forceinline__ bool wants(int) const { return true; }
            __device__ __forceinline__ void code(int, int b, uint32_t word, const float (&recon)[8], float beta) const {
                codes[first_block + b] = word;
                if (decoded) {
                    uint32_t h[8];
#pragma unroll
                    for (int j = 0; j < 8; j++) h[j] = f32_to_bf16((recon[j] * beta) * back);
                    store_decoded<kCoherent>(decoded + first_block + b, make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16),
                                                                                   h[4] | (h[5] << 16), h[6] | (h[7] << 16)));
                }
            }
            __device__ __forceinline__ void beta_byte(int, int b, uint32_t byte) const {
                beta_ids[(first_block + b) >> 2] = (uint8_t)byte;
            }
            __device__ __forceinline__ uint32_t counter(int, int) const { return 0; }
        };
        const LaneSink sink{codes, beta_ids, decoded, row * (n >> 3), norm / sqrt_n};
        if (kForm == kBlockLanes) {
            const int blocks_per_slice = (n >> 3) / slices;
            for (int at = tid; at < blocks_per_slice; at += (int)blockDim.x) {
                const int b = slice * blocks_per_slice + at;
                float raw[8];
#pragma unroll
                for (int j = 0; j < 8; j++) raw[j] = chains[j * pitch + b];
                quantize_block_betas_in_turn(raw, scale, betas, beta_count, 14.0f, 1.0f / 14.0f, 0, b, sink);
            }
            NQ_STAMP(4);
            return;
        }
        // (kFirstLanes: the 256 lanes that are left take the slice 256 pairs at a time, once for slices of
        // 512 values)
        const int pairs_per_slice = (n >> 1) / slices, pairs_per_pass = kForm == kFirstLanes ? 256 : (int)blockDim.x;
        for (int at = tid; at < pairs_per_slice; at += pairs_per_pass) {
            const int p = slice * pairs_per_slice + at, b = p >> 2;
            float raw[8];
#pragma unroll
            for (int j = 0; j < 8; j++) raw[j] = chains[j * pitch + b];
            quantize_pair_lane<false, true>(raw, scale, beta, live, bi, 0, b, p, 14.0f, 1.0f / 14.0f, 0u, sink);
        }
        NQ_STAMP(4);
        return;
    }

    // Encode: eight lanes per (block, beta) pair, lane c the block's coordinate c; a wavefront holds
    // two blocks with their four betas each, the workgroup blockDim / 32 blocks per pass, and the
    // slice's blocks take blocks_per_slice / (blockDim / 32) passes (one when a row has 32 slices).
    const int blocks_per_row = n >> 3;
    const int blocks_per_slice = blocks_per_row / slices, blocks_per_pass = (int)(blockDim.x >> 5);
    const int64_t first_block = row * blocks_per_row;
    const float back = norm / sqrt_n;
    for (int first = 0; first < blocks_per_slice; first += blocks_per_pass) {
        const int in_pass = 2 * (tid >> 6) + (lane >> 5);
        const int b = slice * blocks_per_slice + first + in_pass;
        const float raw = chains[c * pitch + b];
        const PairOnEightLanes pair = quantize_pair_on_eight_lanes<true>(raw, scale, beta, live, bi, lane);
        if (pair.wins) {
            if (c == 0) codes[first_block + b] = pair.word;
            if (decoded)
                store_decoded<kCoherent>(reinterpret_cast<uint16_t *>(decoded) + (first_block + b) * 8 + c,
                                         f32_to_bf16((pair.recon * beta) * back));
        }
        if ((lane & 31) == 7) chosen[in_pass] = (uint8_t)pair.best;
        __syncthreads();
        // four consecutive blocks share one beta byte
        if (tid < (blocks_per_pass >> 2)) {
            const uint32_t byte = chosen[4 * tid] | (chosen[4 * tid + 1] << 2) | (chosen[4 * tid + 2] << 4) |
                                  (chosen[4 * tid + 3] << 6);
            beta_ids[(first_block + slice * blocks_per_slice + first + 4 * tid) >> 2] = (uint8_t)byte;
        }
        if (first + blocks_per_pass < blocks_per_slice) __syncthreads();      // `chosen` is written again
    }
    NQ_STAMP(4);
}

template <int kPrologue, int kForm>
__global__ void __launch_bounds__(1024)
quantize_row_lanes_kernel(const void *__restrict__ x_any, int x_is_f32, int64_t rows, int n, const float *__restrict__ betas,
                          int beta_count, float sqrt_n, uint32_t *__restrict__ codes, uint8_t *__restrict__ beta_ids,
                          float *__restrict__ norms, uint4 *__restrict__ decoded, int slices, int rotate,
                          InputPrologue pro) {
    row_lanes_encode<kPrologue, kForm>(x_any, x_is_f32, rows, n, betas, beta_count, sqrt_n, codes, beta_ids, norms, decoded,
                                       slices, rotate, pro, (int)blockIdx.x);
}

}  // namespace nq
