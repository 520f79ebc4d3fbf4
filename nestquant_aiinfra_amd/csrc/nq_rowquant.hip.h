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

// S butterfly stages (pair distances 2^log_w .. 2^(log_w + S - 1)) on 2^S values held in
// registers: one LDS round trip per pass instead of one per stage.  `total` counts all staged
// values; groups never straddle rows because n is a power of two.
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

template <int S, int kDtype>
__device__ __forceinline__ void hadamard_pass(float *rows, int total, int log_w) {
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
#pragma unroll
        for (int j = 0; j < kValues; j++) rows[base + (j << log_w)] = v[j];
    }
    __syncthreads();
}

// Normalized Sylvester-Hadamard transform of rows staged in LDS (nestquant/core/rotation.py:12-27):
// butterflies of growing width, each sum and difference rounded to `stage_dtype` (the dtype
// the reference's tensor ops would run in), then one multiplication by float32(1 / sqrt(n))
// -- the form a tensor / python-scalar division takes on the GPU.  Ends with a barrier.
template <int kDtype>
__device__ __forceinline__ void staged_hadamard_as(float *rows, int row_count, int n) {
    const int log_n = 31 - __builtin_clz(n);
    const int total = row_count * n;
    int log_w = 0;
    for (; log_n - log_w >= 3; log_w += 3) hadamard_pass<3, kDtype>(rows, total, log_w);
    if (log_n - log_w == 2) hadamard_pass<2, kDtype>(rows, total, log_w);
    if (log_n - log_w == 1) hadamard_pass<1, kDtype>(rows, total, log_w);
    const float inv = 1.0f / __builtin_sqrtf((float)n);
    for (int i = 2 * threadIdx.x; i < total; i += 2 * blockDim.x) {
        float a = rows[i] * inv, b = rows[i + 1] * inv;
        round_pair<kDtype>(a, b);
        rows[i] = a;
        rows[i + 1] = b;
    }
    __syncthreads();
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
            // n is a multiple of 32: four chain steps per trip, many trips in flight
#pragma unroll 8
            for (int i = 0; i < (n >> 3); i += 4) {
                const float v0 = row[8 * i], v1 = row[8 * i + 8], v2 = row[8 * i + 16], v3 = row[8 * i + 24];
                acc = __builtin_fmaf(v0, v0, acc);
                acc = __builtin_fmaf(v1, v1, acc);
                acc = __builtin_fmaf(v2, v2, acc);
                acc = __builtin_fmaf(v3, v3, acc);
            }
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
    __syncthreads();
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
        const float beta = betas_of(r)[live ? bi : 0];
        float y[8], z[8], code[8], p8[8], recon[8], dither[8];
        if (kDithered) dither_block(seed_plus_offset + sink.counter(r, b), dither);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            y[j] = raw[j] * scale;
            z[j] = y[j] / beta;                 // IEEE division
            if (kDithered) z[j] = z[j] + dither[j];
        }
        encode_block(z, q, inv_q, code);
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
}

}  // namespace nq
