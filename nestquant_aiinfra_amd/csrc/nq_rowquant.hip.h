// Row quantiser building blocks shared by the stand-alone encoder kernel and the KV page
// writer: rows are staged in LDS as float32, then
//   staged_row_norms       L2 norms in the reference's order (nestquant/core/quantizer.py:257):
//                          eight interleaved fused-multiply-add chains (element i feeds chain
//                          i % 8), chains added 0..7, sqrt; eight lanes per row run the chains;
//   quantize_staged_pairs  one lane per (block, beta) pair: a quad of lanes evaluates the four
//                          betas of one block (quantizer.py:273-289), the per-block argmin (first
//                          minimum) is a two-step quad exchange, the winning lane hands the
//                          32-bit code word to the sink, and the 2-bit ids of four neighbouring
//                          blocks are merged into one byte with two more exchanges.
#pragma once

#include "nq_e8.hip.h"

// Phase stamps (a measuring build only, -DNQ_PHASE_STAMPS, and only in a translation unit that
// names its stamp array with NQ_PHASE_STAMP_ARRAY before this header): lane 0 of workgroup 0 writes
// the 100 MHz wall clock at the phase boundaries into that device array, which the unit's
// nq_debug_*_stamps call copies out.  Otherwise the macro is empty.
#if defined(NQ_PHASE_STAMPS) && defined(NQ_PHASE_STAMP_ARRAY)
namespace nq { __device__ unsigned long long NQ_PHASE_STAMP_ARRAY[16]; }
#define NQ_STAMP(i) do { if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) nq::NQ_PHASE_STAMP_ARRAY[i] = wall_clock64(); } while (0)
#else
#define NQ_STAMP(i) do { } while (0)
#endif

namespace nq {

// exchange with the lane whose id differs in bit 0 / bit 1 (inside a quad)
__device__ __forceinline__ uint32_t quad_xor1(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
}
__device__ __forceinline__ uint32_t quad_xor2(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
}


// Round a float32 to the value the given storage dtype would hold (tags as in nqhip.h:
// 0 = float32, 1 = bfloat16, 2 = float16), keeping it as float32.
__device__ __forceinline__ float round_to_dtype(float x, int dtype) {
    if (dtype == 1) return bf16_to_f32(f32_to_bf16(x));
    if (dtype == 2) return (float)(_Float16)x;
    return x;
}

// Both values rounded to the storage dtype kDtype (tags as above), kept as float32.
template <int kDtype>
__device__ __forceinline__ void round_pair(float &a, float &b) {
    if (kDtype == 1) {
        const uint32_t packed = __builtin_bit_cast(uint32_t, pack_bf16x2(a, b));
        a = __uint_as_float(packed << 16);
        b = __uint_as_float(packed & 0xffff0000u);
    } else if (kDtype == 2) {
        a = (float)(_Float16)a;
        b = (float)(_Float16)b;
    }
}

// S butterfly stages (pair distances 2^log_w .. 2^(log_w + S - 1)) on 2^S values held in
// registers: one LDS round trip per pass instead of one per stage.  `total` counts all staged
// values; groups never straddle rows because n is a power of two.  With kScale the results are multiplied by `inv` and rounded once more on the way out.
template <int S, int kDtype, bool kScale>
__device__ __forceinline__ void hadamard_pass(float *rows, int total, int log_w, float inv) {
    constexpr int kValues = 1 << S;
    const int groups = total >> S;
    for (int t = threadIdx.x; t < groups; t += blockDim.x) {
        const int base = ((t >> log_w) << (log_w + S)) + (t & ((1 << log_w) - 1));
        float v[kValues];
#pragma unroll
        for (int j = 0; j < kValues; j++) v[j] = rows[base + (j << log_w)];
#pragma unroll
        for (int s = 0; s < S; s++) {
#pragma unroll
            for (int j = 0; j < kValues; j++) {
                if (j & (1 << s)) continue;
                const float left = v[j], right = v[j + (1 << s)];
                v[j] = left + right;
                v[j + (1 << s)] = left - right;
                round_pair<kDtype>(v[j], v[j + (1 << s)]);
            }
        }
        if (kScale) {
#pragma unroll
            for (int j = 0; j < kValues; j += 2) {
                v[j] = v[j] * inv;
                v[j + 1] = v[j + 1] * inv;
                round_pair<kDtype>(v[j], v[j + 1]);
            }
        }
#pragma unroll
        for (int j = 0; j < kValues; j++) rows[base + (j << log_w)] = v[j];
    }
    __syncthreads();
}

// The value the lane whose id differs by kXor holds (all lanes of the exchange active).
template <int kXor>
__device__ __forceinline__ float lane_xor(float v) {
    const int x = __builtin_bit_cast(int, v);
    if (kXor == 1) return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(x, 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    if (kXor == 2) return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(x, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    if (kXor == 4) {
        int r = __builtin_amdgcn_update_dpp(0, x, 0x104, 0xF, 0x5, false);       // row_shl:4 into lanes 0-3, 8-11
        r = __builtin_amdgcn_update_dpp(r, x, 0x114, 0xF, 0xA, false);           // row_shr:4 into lanes 4-7, 12-15
        return __builtin_bit_cast(float, r);
    }
    if (kXor == 8) return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(x, 0x128, 0xF, 0xF, true));  // row_ror:8
    return __shfl_xor(v, kXor, 64);
}

// One butterfly stage between lanes: the lane with the lower id holds the left operands.
template <int kXor, int kDtype>
__device__ __forceinline__ void lane_stage(float (&v)[8], int lane) {
    const bool upper = (lane & kXor) != 0;
    if (kXor == 16 || kXor == 32) {
        // v_permlane{16,32}_swap exchanges the odd rows (of 16 / 32 lanes) of its first operand with
        // the even rows of its second: given the value twice, the first result holds the left
        // operand of the lane's butterfly and the second the right one, in both partner lanes
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int bits = __builtin_bit_cast(int, v[j]);
            float left, right;
            if (kXor == 16) {
                const auto pair = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
                left = __builtin_bit_cast(float, (int)pair[0]);
                right = __builtin_bit_cast(float, (int)pair[1]);
            } else {
                const auto pair = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
                left = __builtin_bit_cast(float, (int)pair[0]);
                right = __builtin_bit_cast(float, (int)pair[1]);
            }
            v[j] = upper ? left - right : left + right;
        }
#pragma unroll
        for (int j = 0; j < 8; j += 2) round_pair<kDtype>(v[j], v[j + 1]);
        return;
    }
    float other[8];
#pragma unroll
    for (int j = 0; j < 8; j++) other[j] = lane_xor<kXor>(v[j]);
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = other[j] + (upper ? -v[j] : v[j]);       // left + right | left - right
#pragma unroll
    for (int j = 0; j < 8; j += 2) round_pair<kDtype>(v[j], v[j + 1]);
}

// The butterflies of distance 1 .. 2^(2 + lane_stages) on the eight neighbouring values every lane of
// a wavefront holds (value j of lane l is element 8 l + j of the wavefront's 512): distances 1, 2, 4
// in registers, 8 .. 256 between lanes.  With scale_here the results are multiplied by `inv` and
// rounded once more.
template <int kDtype>
__device__ __forceinline__ void hadamard_chunk(float (&v)[8], int lane, int lane_stages, bool scale_here, float inv) {
#pragma unroll
    for (int s = 0; s < 3; s++) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if (j & (1 << s)) continue;
            const float left = v[j], right = v[j + (1 << s)];
            v[j] = left + right;
            v[j + (1 << s)] = left - right;
            round_pair<kDtype>(v[j], v[j + (1 << s)]);
        }
    }
    if (lane_stages > 0) lane_stage<1, kDtype>(v, lane);
    if (lane_stages > 1) lane_stage<2, kDtype>(v, lane);
    if (lane_stages > 2) lane_stage<4, kDtype>(v, lane);
    if (lane_stages > 3) lane_stage<8, kDtype>(v, lane);
    if (lane_stages > 4) lane_stage<16, kDtype>(v, lane);
    if (lane_stages > 5) lane_stage<32, kDtype>(v, lane);
    if (scale_here) {
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            v[j] = v[j] * inv;
            v[j + 1] = v[j + 1] * inv;
            round_pair<kDtype>(v[j], v[j + 1]);
        }
    }
}

// Normalized Sylvester-Hadamard transform of rows staged in LDS (nestquant/core/rotation.py:12-27):
// butterflies of growing width, each sum and difference rounded to `stage_dtype` (the dtype
// the reference's tensor ops would run in), then one multiplication by float32(1 / sqrt(n))
// -- the form a tensor / python-scalar division takes on the GPU.  Ends with a barrier.
//
// Every lane takes eight neighbouring values: distances 1, 2, 4 are butterflies in registers,
// distances 8 .. 256 exchanges between the lanes of a wavefront, and only the distances from
// 512 up (rows of 1024 values and more) make further trips through LDS.
template <int kDtype>
__device__ __forceinline__ void staged_hadamard_as(float *rows, int row_count, int n) {
    const int log_n = 31 - __builtin_clz(n);
    const int total = row_count * n;
    const float inv = 1.0f / __builtin_sqrtf((float)n);
    if (n < 8 || (blockDim.x & 63)) {
        // short rows or ragged wavefronts: every stage through LDS
        int log_w = 0;
        for (; log_n - log_w >= 3; log_w += 3) hadamard_pass<3, kDtype, false>(rows, total, log_w, inv);
        if (log_n - log_w == 2) hadamard_pass<2, kDtype, false>(rows, total, log_w, inv);
        if (log_n - log_w == 1) hadamard_pass<1, kDtype, false>(rows, total, log_w, inv);
        for (int i = 2 * threadIdx.x; i < total; i += 2 * blockDim.x) {
            float a = rows[i] * inv, b = rows[i + 1] * inv;
            round_pair<kDtype>(a, b);
            rows[i] = a;
            rows[i + 1] = b;
        }
        __syncthreads();
        return;
    }
    const int lane = threadIdx.x & 63;
    const int lane_stages = log_n - 3 < 6 ? log_n - 3 : 6;
    const bool scale_here = log_n <= 9;
    for (int chunk = threadIdx.x; chunk < (total >> 3); chunk += blockDim.x) {
        float4 *slot = reinterpret_cast<float4 *>(rows + 8 * chunk);
        const float4 lo = slot[0], hi = slot[1];
        float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        // a row's chunks sit in neighbouring lanes (n / 8 of them, a power of two), so the
        // stage count is the same for the whole wavefront
        hadamard_chunk<kDtype>(v, lane, lane_stages, scale_here, inv);
        slot[0] = make_float4(v[0], v[1], v[2], v[3]);
        slot[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
    NQ_STAMP(8);
    __syncthreads();
    NQ_STAMP(9);
    int log_w = 9;
    for (; log_n - log_w > 4; log_w += 3) hadamard_pass<3, kDtype, false>(rows, total, log_w, inv);
    switch (log_n - log_w) {
        case 4: hadamard_pass<4, kDtype, true>(rows, total, log_w, inv); break;
        case 3: hadamard_pass<3, kDtype, true>(rows, total, log_w, inv); break;
        case 2: hadamard_pass<2, kDtype, true>(rows, total, log_w, inv); break;
        case 1: hadamard_pass<1, kDtype, true>(rows, total, log_w, inv); break;
        default: break;
    }
}

__device__ __forceinline__ void staged_hadamard(float *rows, int row_count, int n, int stage_dtype) {
    if (stage_dtype == 1) staged_hadamard_as<1>(rows, row_count, n);
    else if (stage_dtype == 2) staged_hadamard_as<2>(rows, row_count, n);
    else staged_hadamard_as<0>(rows, row_count, n);
}

// rows: [row_count][n] float32 in LDS, n a multiple of 32.  Writes row_scale[r] =
// (1 / norm) * sqrt(n) (0 for a zero row) and row_norm[r]; ends with a barrier.
__device__ __forceinline__ void staged_row_norms(const float *rows, int row_count, int n, float sqrt_n,
                                                 float *row_scale, float *row_norm) {
    const int tid = threadIdx.x;
    for (int base = 0; base < 8 * row_count; base += blockDim.x) {
        const int t = base + tid;
        if (t < 8 * row_count) {
            const int r = t >> 3, lane = t & 7;
            const float *row = rows + (size_t)r * n + lane;
            float acc = 0.0f;
            // n is a multiple of 32.  Batches of 32 chain steps, double-buffered by hand: the
            // next batch is requested from LDS before the chain runs over the current one, so
            // that the LDS latency stays off the serial path (a request past the end is clamped
            // to the last batch and not used).
            const int groups = n >> 5, batches = groups >> 3;
            if (batches > 0) {
                float a[32], b[32];
#pragma unroll
                for (int k = 0; k < 32; k++) a[k] = row[8 * k];
                int batch = 0;
                for (; batch + 2 <= batches; batch += 2) {
                    const float *next = row + 256 * (batch + 1);
#pragma unroll
                    for (int k = 0; k < 32; k++) b[k] = next[8 * k];
                    __builtin_amdgcn_sched_barrier(0);      // keep the requests ahead of the chain
#pragma unroll
                    for (int k = 0; k < 32; k++) acc = __builtin_fmaf(a[k], a[k], acc);
                    __builtin_amdgcn_sched_barrier(0);
                    const int after = batch + 2 < batches ? batch + 2 : batches - 1;
                    // the address waits for the chain (adding zero unless the sum is NaN): the request
                    // then reuses the registers the chain has just released, with no copies in the loop
                    next = row + 256 * after + (acc != acc ? 1 : 0);
#pragma unroll
                    for (int k = 0; k < 32; k++) a[k] = next[8 * k];
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int k = 0; k < 32; k++) acc = __builtin_fmaf(b[k], b[k], acc);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (batch < batches) {
#pragma unroll
                    for (int k = 0; k < 32; k++) acc = __builtin_fmaf(a[k], a[k], acc);
                }
            }
#pragma unroll 1
            for (int g = batches << 3; g < groups; g++) {
                const float v0 = row[32 * g], v1 = row[32 * g + 8], v2 = row[32 * g + 16], v3 = row[32 * g + 24];
                acc = __builtin_fmaf(v0, v0, acc);
                acc = __builtin_fmaf(v1, v1, acc);
                acc = __builtin_fmaf(v2, v2, acc);
                acc = __builtin_fmaf(v3, v3, acc);
            }
            NQ_STAMP(10);
            float total = 0.0f;
#pragma unroll
            for (int k = 0; k < 8; k++) total = total + __shfl(acc, (tid & 56) + k, 64);
            const float norm = __builtin_sqrtf(total);
            if (lane == 0) {
                // math.sqrt(n) / norm is evaluated as (1 / norm) * float32(sqrt(n))
                row_scale[r] = norm > 0.0f ? (1.0f / norm) * sqrt_n : 0.0f;
                row_norm[r] = norm;
            }
        }
    }
    NQ_STAMP(11);
    __syncthreads();
}

// One lane's share of a block: its values `raw` (to be scaled by `scale`) against the beta of index
// bi (quantizer.py:273-289); the quad of lanes bi = 0..3 then settles the first minimum by two
// exchanges, the winner hands the code word to the sink, and sixteen lanes merge the beta byte of
// four neighbouring blocks.  p = (row * blocks_per_row + block) * 4 + bi.  With kFastDivide the
// division by beta goes through its reciprocal where that gives the IEEE quotient (a zero quotient
// may then carry the other sign; the lattice search treats both alike).
template <bool kDithered, bool kFastDivide, class Sink>
__device__ __forceinline__ void quantize_pair_lane(const float (&raw)[8], float scale, float beta, bool live, int bi,
                                                   int r, int b, int p, float q, float inv_q,
                                                   uint32_t seed_plus_offset, const Sink &sink) {
    float y[8], z[8], code[8], p8[8], recon[8], dither[8];
    if (kDithered) dither_block(seed_plus_offset + sink.counter(r, b), dither);
#pragma unroll
    for (int j = 0; j < 8; j++) y[j] = raw[j] * scale;
    // the same decision for the whole wavefront; the quotients are the IEEE ones either way
    const bool by_reciprocal = kFastDivide && beta >= 0x1p-40f && beta <= 0x1p40f &&
                               __builtin_amdgcn_ballot_w64(has_tiny_nonzero(y)) == 0;
    if (by_reciprocal) {
        const float rcp = 1.0f / beta;
#pragma unroll
        for (int j = 0; j < 8; j++) z[j] = divide_by_reciprocal(y[j], beta, rcp);
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) z[j] = y[j] / beta;     // IEEE division
    }
    if (kDithered) {
#pragma unroll
        for (int j = 0; j < 8; j++) z[j] = z[j] + dither[j];
    }
    NQ_STAMP(5);
    encode_block(z, q, inv_q, code);
    NQ_STAMP(6);
    e8_coset_point(code, p8);
    if (kDithered) {
#pragma unroll
        for (int j = 0; j < 8; j++) p8[j] = p8[j] - dither[j];
    }
    reduce_coset_point(p8, q, recon);
    float err = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float d = recon[j] * beta - y[j];
        err = err + d * d;
    }
    if (!live) err = __builtin_inff();
    NQ_STAMP(7);

    // first minimum over the quad: order by (err, beta index)
    uint32_t best_err = __float_as_uint(err), best = (uint32_t)bi;
    {
        const uint32_t oe = quad_xor1(best_err), oi = quad_xor1(best);
        const float fe = __uint_as_float(oe), me = __uint_as_float(best_err);
        const bool take = fe < me || (fe == me && oi < best);
        best_err = take ? oe : best_err;
        best = take ? oi : best;
    }
    {
        const uint32_t oe = quad_xor2(best_err), oi = quad_xor2(best);
        const float fe = __uint_as_float(oe), me = __uint_as_float(best_err);
        const bool take = fe < me || (fe == me && oi < best);
        best = take ? oi : best;
    }
    const bool wanted = sink.wants(r);
    if (best == (uint32_t)bi && wanted) sink.code(r, b, pack_codeword(code), recon, beta);

    // four consecutive blocks (16 lanes) share one beta byte
    uint32_t byte = best << (2 * (b & 3));
    byte |= (uint32_t)__shfl_xor((int)byte, 4, 64);
    byte |= (uint32_t)__shfl_xor((int)byte, 8, 64);
    if ((p & 15) == 0 && wanted) sink.beta_byte(r, b, byte);
}

// ---------------------------------------------------------------------------------------
// One (block, beta) pair on eight neighbouring lanes, lane c (= lane id % 8) holding coordinate c.
// For a few rows the encoder is a latency problem: with one lane per pair a wavefront walks about
// 850 instructions that depend on each other; spread over its coordinates a pair takes about 250
// per lane, and the eight-term sums whose order the reference fixes (squares added j = 0..7) become
// scans along the eight lanes.  Every float32 operation is the one quantize_pair_lane performs, in
// the same order, so codes, beta ids and decoded values are the same bits.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float dpp_from_lane_below(float v) {       // lane i <- lane i - 1 (row_shr:1)
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x111, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_from_lane_above(float v) {       // lane i <- lane i + 1 (row_shl:1)
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x101, 0xF, 0xF, true));
}
// ((v0 + v1) + v2) + ... + v7 of the eight lanes of a group, valid in its last lane (c == 7): after
// step k lane i holds the left-to-right sum of lanes i - k .. i, so the window of lane 7 never
// leaves the group.
__device__ __forceinline__ float ordered_sum8_in_last(float v) {
    float s = v;
#pragma unroll
    for (int k = 1; k < 8; k++) s = dpp_from_lane_below(s) + v;
    return s;
}
// the value of the group's last lane in all eight: the last lane of each quad to its quad, then the
// upper quad mirrored into the lower one
__device__ __forceinline__ float from_last8(float v) {
    const int quad = __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xFF, 0xF, 0xF, true);       // quad_perm [3,3,3,3]
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(quad, quad, 0x141, 0xF, 0x5, false)); // half mirror into lanes 0-3
}
__device__ __forceinline__ float max8(float v) {
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true)));
    return v;
}
__device__ __forceinline__ uint32_t or8(uint32_t v) {
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true);
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x141, 0xF, 0xF, true);
    return v;
}
// whether this lane is the first of its group of eight whose flag is set
__device__ __forceinline__ bool first_set8(bool flag, int lane) {
    const uint64_t all = __builtin_amdgcn_ballot_w64(flag);
    const uint32_t group = (uint32_t)(all >> (lane & 56)) & 0xffu;
    return flag && (group & ((1u << (lane & 7)) - 1u)) == 0u;
}

// e8_nearest (nq_e8.hip.h) with x_c in lane c: returns coordinate c of the nearest point.
__device__ __forceinline__ float e8_nearest_on_eight_lanes(float x, int lane) {
    const float a = __builtin_rintf(x);
    const float ea = x - a;                                    // exact
    const float xm = x - 0.5f;
    const float b = __builtin_rintf(xm);
    const float eb = xm - b;
    const float sum_a = from_last8(ordered_sum8_in_last(a)), sum_b = from_last8(ordered_sum8_in_last(b));
    const float max_a = max8(fabsf(ea)), max_b = max8(fabsf(eb));
    const float moved_a = max_a - 1.0f;
    const float alt_a = moved_a * moved_a;
    // the first coordinate with the largest |residual| moves when the coordinate sum is odd
    const bool hit_a = first_set8(fabsf(ea) == max_a, lane) && is_odd(sum_a);
    const bool hit_b = first_set8(fabsf(eb) == max_b, lane) && is_odd(sum_b);
    const float sq = ea * ea;
    const float term_a = hit_a ? alt_a : sq;
    const float point_a = hit_a ? a + __builtin_copysignf(1.0f, ea) : a;
    const float half_point = b + 0.5f;
    const float point_b = hit_b ? half_point + __builtin_copysignf(1.0f, eb) : half_point;
    const float t = x - point_b;
    const float term_b = t * t;
    const float dist_a = ordered_sum8_in_last(term_a), dist_b = ordered_sum8_in_last(term_b);
    const bool pick_a = from_last8(dist_a < dist_b ? 1.0f : 0.0f) != 0.0f;       // ties go to the half-integer coset
    return pick_a ? point_a : point_b;
}

struct PairOnEightLanes {
    uint32_t word;      // the packed code word, in all eight lanes
    uint32_t best;      // the block's winning beta index, in the last lane of each of the four groups
    float recon;        // coordinate c of the pair's decoded lattice point
    bool wins;          // this pair's beta is the block's choice, in all eight lanes
};

// quantize_pair_lane for the pair whose coordinate c this lane holds (`raw`), q = 14.  The four
// betas of a block sit in four neighbouring groups of eight lanes (beta index bi = (lane / 8) % 4).
template <bool kFastDivide>
__device__ __forceinline__ PairOnEightLanes quantize_pair_on_eight_lanes(float raw, float scale, float beta, bool live,
                                                                         int bi, int lane) {
    const int c = lane & 7;
    const float y = raw * scale;
    const uint32_t key = (__float_as_uint(y) << 1) - 1u;                         // as has_tiny_nonzero
    const bool tiny = key < ((66u << 24) - 1u);
    const bool by_reciprocal = kFastDivide && beta >= 0x1p-40f && beta <= 0x1p40f && __builtin_amdgcn_ballot_w64(tiny) == 0;
    float z;
    if (by_reciprocal) z = divide_by_reciprocal(y, beta, 1.0f / beta);
    else z = y / beta;                                                           // IEEE division
    // encode_block: nearest point, generator coordinates (the recurrence of e8_coords, one step per
    // coordinate from c = 5 down), residues modulo q
    const float point = e8_nearest_on_eight_lanes(z, lane);
    const float last = from_last8(point);
    float coord = c == 7 ? 2.0f * point : point - last;                          // c[7], c[6]
#pragma unroll
    for (int step = 5; step >= 0; step--) {
        const float candidate = (point + dpp_from_lane_above(coord)) - last;
        coord = c == step ? (step == 0 ? 0.5f * candidate : candidate) : coord;
    }
    const float code = mod_q(coord, 14.0f, 1.0f / 14.0f);
    // e8_coset_point
    const float h = 0.5f * from_last8(code);
    const float next = dpp_from_lane_above(code);
    const float p8 = c == 0 ? (2.0f * code - next) + h : (c <= 5 ? (code - next) + h : (c == 6 ? code + h : h));
    // reduce_coset_point
    const float k = e8_nearest_on_eight_lanes(div_by_14(p8), lane);
    const float recon = p8 - 14.0f * k;                                          // exact
    const float d = recon * beta - y;
    float err = ordered_sum8_in_last(d * d);
    if (!live) err = __builtin_inff();
    // first minimum over the four betas: order by (err, beta index); partners 8 and 16 lanes away
    uint32_t best_err = __float_as_uint(err), best = (uint32_t)bi;
    {
        const uint32_t oe = (uint32_t)__builtin_amdgcn_mov_dpp((int)best_err, 0x128, 0xF, 0xF, true);   // row_ror:8
        const uint32_t oi = (uint32_t)__builtin_amdgcn_mov_dpp((int)best, 0x128, 0xF, 0xF, true);
        const float fe = __uint_as_float(oe), me = __uint_as_float(best_err);
        const bool take = fe < me || (fe == me && oi < best);
        best_err = take ? oe : best_err;
        best = take ? oi : best;
    }
    {
        const auto e2 = __builtin_amdgcn_permlane16_swap(best_err, best_err, false, false);
        const auto i2 = __builtin_amdgcn_permlane16_swap(best, best, false, false);
        const bool upper = (lane & 16) != 0;
        const uint32_t oe = upper ? (uint32_t)e2[0] : (uint32_t)e2[1], oi = upper ? (uint32_t)i2[0] : (uint32_t)i2[1];
        const float fe = __uint_as_float(oe), me = __uint_as_float(best_err);
        const bool take = fe < me || (fe == me && oi < best);
        best = take ? oi : best;
    }
    PairOnEightLanes out;
    out.best = best;
    out.wins = from_last8(best == (uint32_t)bi ? 1.0f : 0.0f) != 0.0f;
    out.word = or8(((uint32_t)code) << (4 * c));
    out.recon = recon;
    return out;
}

// Pairs [pair_begin, pair_end) of the staged rows (pair = (row * n / 8 + block) * 4 + beta
// index; both bounds multiples of 16).  betas_of(row) returns that row's beta table.
// Sink: wants(row), code(row, block, word, recon, beta), beta_byte(row, block, byte),
// counter(row, block) (dither counter of the block's first element, dithered rows only).
template <bool kDithered, class BetasOf, class Sink>
__device__ __forceinline__ void quantize_staged_pairs(const float *rows, const float *row_scale, int n, float q,
                                                      float inv_q, BetasOf betas_of, int beta_count,
                                                      uint32_t seed_plus_offset, int pair_begin, int pair_end,
                                                      const Sink &sink) {
    const int blocks_per_row = n >> 3;
    for (int p = pair_begin + (int)threadIdx.x; p < pair_end; p += blockDim.x) {
        const int blk = p >> 2, bi = p & 3;
        const int r = blk / blocks_per_row, b = blk - r * blocks_per_row;
        const float scale = row_scale[r];
        const float4 lo = *reinterpret_cast<const float4 *>(rows + (size_t)r * n + 8 * b);
        const float4 hi = *reinterpret_cast<const float4 *>(rows + (size_t)r * n + 8 * b + 4);
        const float raw[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        const bool live = bi < beta_count;
        quantize_pair_lane<kDithered, false>(raw, scale, betas_of(r)[live ? bi : 0], live, bi, r, b, p, q, inv_q,
                                             seed_plus_offset, sink);
    }
}

// Blocks [block_begin, block_end) of the staged rows, one lane per block with the betas
// taken in turn: the form for many rows, where the vector units are the limit rather than
// the latency of one row.  Same results as quantize_staged_pairs (undithered rows).
//
// A lattice point x = Q_E8(y / beta) with |x|^2 <= q^2 / 2 - 2 lies strictly inside the
// Voronoi cell of q E8 (packing radius q / sqrt 2, margin far above the rounding of p / q), so
// the nested decode of its code returns x itself: when that holds for every lane of the
// wavefront the coset reduction (a second lattice search) is skipped.  The first minimum over
// the betas is a strict comparison in ascending order, and only the winner is turned into a
// code word.
// One block, its betas in turn (see quantize_staged_blocks): raw holds the block's eight staged
// values, `betas` the row's table.  Every lane of the wavefront must call it together.
template <class Sink>
__device__ __forceinline__ void quantize_block_betas_in_turn(const float (&raw)[8], float scale, const float *betas,
                                                             int beta_count, float q, float inv_q, int r, int b,
                                                             const Sink &sink) {
    const float inside_limit = 0.5f * q * q - 2.0f;
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; j++) y[j] = raw[j] * scale;
    // the same for the whole wavefront, so that the betas stay a uniform loop
    const bool fast_division = __builtin_amdgcn_ballot_w64(has_tiny_nonzero(y)) == 0;
    float best_err = __builtin_inff(), best_beta = betas[0], best_point[8], best_recon[8];
    uint32_t best = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) best_point[j] = best_recon[j] = 0.0f;
#pragma unroll 1
    for (int bi = 0; bi < beta_count; bi++) {
        const float beta = betas[bi];
        float z[8], point[8], recon[8];
        if (fast_division && beta >= 0x1p-40f && beta <= 0x1p40f) {
            const float rcp = 1.0f / beta;
#pragma unroll
            for (int j = 0; j < 8; j++) z[j] = divide_by_reciprocal(y[j], beta, rcp);
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) z[j] = y[j] / beta;         // IEEE division
        }
        e8_nearest(z, point);
        float energy = 0.0f;                                       // small half-integers: exact
#pragma unroll
        for (int j = 0; j < 8; j++) energy = __builtin_fmaf(point[j], point[j], energy);
        if (__builtin_amdgcn_ballot_w64(!(energy <= inside_limit)) == 0) {
#pragma unroll
            for (int j = 0; j < 8; j++) recon[j] = point[j] + 0.0f;  // the decode never returns -0
        } else {
            float c[8], code[8], p8[8];
            e8_coords(point, c);
#pragma unroll
            for (int j = 0; j < 8; j++) code[j] = mod_q(c[j], q, inv_q);
            e8_coset_point(code, p8);
            reduce_coset_point(p8, q, recon);
        }
        float err = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float d = recon[j] * beta - y[j];
            err = err + d * d;
        }
        const bool take = err < best_err;                          // first minimum
        best_err = take ? err : best_err;
        best = take ? (uint32_t)bi : best;
        best_beta = take ? beta : best_beta;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            best_point[j] = take ? point[j] : best_point[j];
            best_recon[j] = take ? recon[j] : best_recon[j];
        }
    }
    const bool wanted = sink.wants(r);
    if (wanted) {
        float c[8], code[8];
        e8_coords(best_point, c);
#pragma unroll
        for (int j = 0; j < 8; j++) code[j] = mod_q(c[j], q, inv_q);
        sink.code(r, b, pack_codeword(code), best_recon, best_beta);
    }
    // four consecutive blocks (a quad of lanes) share one beta byte
    uint32_t byte = best << (2 * (b & 3));
    byte |= quad_xor1(byte);
    byte |= quad_xor2(byte);
    if ((b & 3) == 0 && wanted) sink.beta_byte(r, b, byte);
}

template <class BetasOf, class Sink>
__device__ __forceinline__ void quantize_staged_blocks(const float *rows, const float *row_scale, int n, float q,
                                                       float inv_q, BetasOf betas_of, int beta_count,
                                                       int block_begin, int block_end, const Sink &sink) {
    const int blocks_per_row = n >> 3;
    for (int blk = block_begin + (int)threadIdx.x; blk < block_end; blk += blockDim.x) {
        const int r = blk / blocks_per_row, b = blk - r * blocks_per_row;
        const float4 lo = *reinterpret_cast<const float4 *>(rows + (size_t)r * n + 8 * b);
        const float4 hi = *reinterpret_cast<const float4 *>(rows + (size_t)r * n + 8 * b + 4);
        const float raw[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        quantize_block_betas_in_turn(raw, row_scale[r], betas_of(r), beta_count, q, inv_q, r, b, sink);
    }
}

}  // namespace nq
