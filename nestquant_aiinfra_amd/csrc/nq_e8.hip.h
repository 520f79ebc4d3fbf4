// Device-side E8 codec primitives shared by every kernel of the packed W4A4KV4 path.
//
// One lane owns one 8-dimensional block: all eight coordinates live in registers, so
// the nearest-point search needs no cross-lane traffic and its eight-term sums are
// naturally sequential.  The float32 operation order below is the contract: it
// reproduces the reference's CPU arithmetic (torch on the host) so that codes, beta
// ids and every decode of an undithered code agree bit for bit:
//   * squares are rounded, then added j = 0..7 in order (the translation unit is built
//     with -ffp-contract=off, so `a + b * b` never fuses);
//   * divisions are IEEE (correctly rounded), never reciprocal multiplies;
//   * v_rndne rounds half to even; the first index wins argmax / argmin ties;
//   * the half-coset residual is (x - 0.5) - rint(x - 0.5);
//   * equal coset distances select the half-integer coset.
// Reference semantics: nestquant/core/lattice.py:18-81, nestquant/core/codec.py:30-224.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nq {

__device__ __forceinline__ float max_abs8(const float (&e)[8]) {
    return fmaxf(fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3]))),
                 fmaxf(fmaxf(fabsf(e[4]), fabsf(e[5])), fmaxf(fabsf(e[6]), fabsf(e[7]))));
}

// remainder(sum, 2) != 0 for an integer-valued float, without an integer conversion
// (also right for sums too large to convert)
__device__ __forceinline__ bool is_odd(float sum) { return __builtin_amdgcn_fractf(sum * 0.5f) != 0.0f; }

// lattice.py:37-81, tie_break "upstream_half".  Returns the nearest E8 point of x: the
// better of the nearest points of the two cosets D8 and D8 + 1/2 (lattice.py:18-34 gives
// the D8 search: round every coordinate, and if the coordinate sum is odd move the first
// coordinate with the largest |residual| to its second-nearest integer).
//
// Integer coset: the squared distance only needs the residuals x - rint(x) (exact); the
// moved coordinate contributes (|residual| - 1)^2 = (max - 1)^2, one value per block.
// Half coset: the reference measures x - (D8(x - 1/2) + 1/2), recomputed from x because
// x - 1/2 may round; the same is done here.
__device__ __forceinline__ void e8_nearest(const float (&x)[8], float (&out)[8]) {
    float a[8], ea[8], sum_a = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        a[j] = __builtin_rintf(x[j]);
        ea[j] = x[j] - a[j];                       // exact
        sum_a = sum_a + a[j];
    }
    const float max_a = max_abs8(ea);
    const float moved_a = max_a - 1.0f;
    const float alt_a = moved_a * moved_a;
    bool done_a = !is_odd(sum_a);                  // an even sum needs no correction
    float dist_a = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const bool top = fabsf(ea[j]) == max_a;
        const bool hit = top && !done_a;           // first coordinate with the largest |residual|
        done_a = done_a || top;
        const float sq = ea[j] * ea[j];
        dist_a = dist_a + (hit ? alt_a : sq);
        // residual >= 0 moves up (a residual is never -0)
        a[j] = hit ? a[j] + __builtin_copysignf(1.0f, ea[j]) : a[j];
    }

    float b[8], eb[8], sum_b = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float xm = x[j] - 0.5f;
        b[j] = __builtin_rintf(xm);
        eb[j] = xm - b[j];
        sum_b = sum_b + b[j];
    }
    const float max_b = max_abs8(eb);
    bool done_b = !is_odd(sum_b);
    float dist_b = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const bool top = fabsf(eb[j]) == max_b;
        const bool hit = top && !done_b;
        done_b = done_b || top;
        const float half_point = b[j] + 0.5f;
        b[j] = hit ? half_point + __builtin_copysignf(1.0f, eb[j]) : half_point;
        const float t = x[j] - b[j];
        dist_b = dist_b + t * t;
    }
    const bool pick_a = dist_a < dist_b;           // ties go to the half-integer coset
#pragma unroll
    for (int j = 0; j < 8; j++) out[j] = pick_a ? a[j] : b[j];
}

// Integer generator coordinates of a lattice point (closed form of codec.py:89-96,
// as in nestquant/runtime/nqkv_page.py:141-148); every step is exact in float32.
__device__ __forceinline__ void e8_coords(const float (&l)[8], float (&c)[8]) {
    c[7] = 2.0f * l[7];
    c[6] = l[6] - l[7];
#pragma unroll
    for (int j = 5; j >= 1; j--) c[j] = (l[j] + c[j + 1]) - l[7];
    c[0] = 0.5f * ((l[0] + c[1]) - l[7]);
}

// codec.py:30-42: coset point G * c of an integer code (exact).
__device__ __forceinline__ void e8_coset_point(const float (&c)[8], float (&p)[8]) {
    const float h = 0.5f * c[7];
    p[0] = (2.0f * c[0] - c[1]) + h;
#pragma unroll
    for (int j = 1; j < 6; j++) p[j] = (c[j] - c[j + 1]) + h;
    p[6] = c[6] + h;
    p[7] = h;
}

// Non-negative residue of an integer-valued float modulo q (torch.remainder, codec.py:97).
__device__ __forceinline__ float mod_q(float c, float q, float inv_q) {
    float r = c - q * __builtin_rintf(c * inv_q);   // in [-q/2 - 1, q/2 + 1], exact
    r = (r < 0.0f) ? r + q : r;
    r = (r >= q) ? r - q : r;
    return r;
}

// Eight 4-bit codes of one block, little-endian nibbles (packing.py:191-208).
__device__ __forceinline__ void unpack_codeword(uint32_t word, float (&c)[8]) {
#pragma unroll
    for (int j = 0; j < 8; j++) c[j] = (float)((word >> (4 * j)) & 15u);
}

__device__ __forceinline__ uint32_t pack_codeword(const float (&c)[8]) {
    uint32_t word = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) word |= ((uint32_t)c[j]) << (4 * j);
    return word;
}

// codec.py:53-102 `encode_nested` for one block: codes in [0, q) as floats.
__device__ __forceinline__ void encode_block(const float (&x)[8], float q, float inv_q, float (&code)[8]) {
    float lattice[8], c[8];
    e8_nearest(x, lattice);
    e8_coords(lattice, c);
#pragma unroll
    for (int j = 0; j < 8; j++) code[j] = mod_q(c[j], q, inv_q);
}

// Correctly rounded p / 14 in three operations: q0 = RN(p * RN(1/14)), the exact remainder
// r = fma(-14, q0, p), and q1 = fma(r, RN(1/14), q0).  Checked against IEEE division for
// every finite float32 with 1e-30 <= |p| <= 1e30 (only the sign of a zero result differs).
__device__ __forceinline__ float div_by_14(float p) {
    const float c = 1.0f / 14.0f;
    const float q0 = p * c;
    const float r = __builtin_fmaf(-14.0f, q0, p);
    return __builtin_fmaf(r, c, q0);
}

// Correctly rounded a / b from the correctly rounded reciprocal `rcp` = 1 / b: a first quotient,
// then two rounds of exact remainder (one fused multiply-add) and correction.  The first round
// leaves a faithful quotient, and a faithful quotient corrected with a correctly rounded
// reciprocal is the correctly rounded one (Markstein).  Needs the remainders to be exact:
// callers keep |a| >= 2^-61 (or a == 0) and 2^-40 <= b <= 2^40.  Only the sign of a zero
// quotient can differ from the IEEE division.
__device__ __forceinline__ float divide_by_reciprocal(float a, float b, float rcp) {
    float quotient = a * rcp;
    float remainder = __builtin_fmaf(-b, quotient, a);
    quotient = __builtin_fmaf(remainder, rcp, quotient);
    remainder = __builtin_fmaf(-b, quotient, a);
    return __builtin_fmaf(remainder, rcp, quotient);
}

// True when some value is nonzero and below 2^-61 in magnitude.
__device__ __forceinline__ bool has_tiny_nonzero(const float (&v)[8]) {
    uint32_t least = 0xffffffffu;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t key = (__float_as_uint(v[j]) << 1) - 1u;      // zero wraps to the largest key
        least = key < least ? key : least;
    }
    return least < ((66u << 24) - 1u);                                // exponent field below 66
}

// codec.py:105-142 `decode_nested` for one block given its coset point (already minus
// the dither when there is one): the minimum-energy representative p - q * Q(p / q).
__device__ __forceinline__ void reduce_coset_point(const float (&p)[8], float q, float (&out)[8]) {
    float z[8], k[8];
#pragma unroll
    for (int j = 0; j < 8; j++) z[j] = (q == 14.0f) ? div_by_14(p[j]) : p[j] / q;   // IEEE division
    e8_nearest(z, k);
#pragma unroll
    for (int j = 0; j < 8; j++) out[j] = p[j] - q * k[j]; // exact
}

// ---------------------------------------------------------------------------------------
// Hinted decode of an undithered block.
//
// decode_codeword<false> spends most of its instructions on decisions that the code word fixes:
// which coset of E8 the point Q_E8(p / 14) lies in and which coordinate the parity correction of
// that coset's D8 search moves.  A writer that has just made the code word can store both in four
// bits (bit 0: the half-integer coset; bits 1..3: the coordinate), and a reader then needs neither
// the other coset's search, nor the scans for the largest residual, nor the two distance sums.
// Whether a correction happens at all is the parity of the rounded coordinates, and its direction
// the sign of the chosen coordinate's residual, both cheap to recompute.  The quotient p / 14 stays
// the correctly rounded one and the coset's offset is subtracted from it as the search does: a
// single multiply-add p * RN(1/14) - 1/2 would round the exact tie p = 14 the other way (checked on
// the CPU over every coordinate a coset point can have).  Same values as
// decode_codeword<false>(word, 14, 0, out), bit for bit, for every code word (nq_nqkv_verify_hints).
__device__ __forceinline__ uint32_t e8_nearest_hint(const float (&x)[8]) {
    // e8_nearest(x) once more, keeping the decisions instead of the point
    float ea[8], sum_a = 0.0f, eb[8], sum_b = 0.0f, a[8], b[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        a[j] = __builtin_rintf(x[j]);
        ea[j] = x[j] - a[j];
        sum_a = sum_a + a[j];
        const float xm = x[j] - 0.5f;
        b[j] = __builtin_rintf(xm);
        eb[j] = xm - b[j];
        sum_b = sum_b + b[j];
    }
    const float max_a = max_abs8(ea), max_b = max_abs8(eb);
    const float moved_a = max_a - 1.0f, alt_a = moved_a * moved_a;
    bool done_a = !is_odd(sum_a), done_b = !is_odd(sum_b);
    float dist_a = 0.0f, dist_b = 0.0f;
    uint32_t index_a = 0u, index_b = 0u;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const bool top_a = fabsf(ea[j]) == max_a, hit_a = top_a && !done_a;
        done_a = done_a || top_a;
        dist_a = dist_a + (hit_a ? alt_a : ea[j] * ea[j]);
        index_a = hit_a ? (uint32_t)j : index_a;
        const bool top_b = fabsf(eb[j]) == max_b, hit_b = top_b && !done_b;
        done_b = done_b || top_b;
        const float half_point = b[j] + 0.5f;
        const float point = hit_b ? half_point + __builtin_copysignf(1.0f, eb[j]) : half_point;
        const float t = x[j] - point;
        dist_b = dist_b + t * t;
        index_b = hit_b ? (uint32_t)j : index_b;
    }
    const bool pick_a = dist_a < dist_b;
    return pick_a ? index_a << 1 : (index_b << 1) | 1u;
}

// The hint of a stored block: the decisions decode_codeword<false>(word, 14, 0, .) takes.
__device__ __forceinline__ uint32_t hint_of_codeword(uint32_t word) {
    float c[8], p[8], z[8];
    unpack_codeword(word, c);
    e8_coset_point(c, p);
#pragma unroll
    for (int j = 0; j < 8; j++) z[j] = div_by_14(p[j]);
    return e8_nearest_hint(z);
}

__device__ __forceinline__ void decode_codeword_hinted(uint32_t word, uint32_t hint, float (&out)[8]) {
    float c[8], p[8], xm[8], r[8];
    unpack_codeword(word, c);
    e8_coset_point(c, p);
    const bool half_coset = (hint & 1u) != 0u;
    const float minus_half = half_coset ? -0.5f : 0.0f;
    const float minus_origin = half_coset ? -7.0f : 0.0f;          // 14 times the coset's offset
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        xm[j] = div_by_14(p[j]) + minus_half;
        r[j] = __builtin_rintf(xm[j]);
        sum = sum + r[j];
    }
    // the residual of the hinted coordinate, picked out of the eight by the index's bits
    const bool bit0 = (hint & 2u) != 0u, bit1 = (hint & 4u) != 0u, bit2 = (hint & 8u) != 0u;
    float e[8];
#pragma unroll
    for (int j = 0; j < 8; j++) e[j] = xm[j] - r[j];
    const float e01 = bit0 ? e[1] : e[0], e23 = bit0 ? e[3] : e[2], e45 = bit0 ? e[5] : e[4], e67 = bit0 ? e[7] : e[6];
    const float e03 = bit1 ? e23 : e01, e47 = bit1 ? e67 : e45;
    const float chosen = bit2 ? e47 : e03;
    // 14 times the step of the corrected coordinate, zero when the sum is even
    const float step = is_odd(sum) ? __builtin_copysignf(14.0f, chosen) : 0.0f;
    const uint32_t index = (hint >> 1) & 7u;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float plain = __builtin_fmaf(-14.0f, r[j], p[j] + minus_origin);      // exact: small half-integers
        out[j] = index == (uint32_t)j ? plain - step : plain;
    }
}

// x * c + a modulo 2^32.  On gfx950 the 32-bit multiply issues at the rate of the other
// three-operand integer instructions (measured: v_mul_lo_u32 2.0 ns per wavefront instruction and
// SIMD, v_dot2_u32_u16 1.9, v_lshl_add_u32 1.8, v_add_u32 1.1), so one multiply and one add beat
// the two 16-bit dot products and the shift-add a quarter-rate multiplier would call for.
__device__ __forceinline__ uint32_t mul_add_u32(uint32_t x, uint32_t c, uint32_t a) {
    return x * c + a;
}

// codec.py:213-222 / nestquant/runtime/nqrt4_device.cuh:7-17: lcg31_mix_v1.  Only the
// low 31 bits of every stage matter, so masks are folded into bit-field extracts; bit 31 of
// the value returned here is not meaningful.
__device__ __forceinline__ uint32_t lcg31_mix_bits(uint32_t counter_plus_seed) {
    uint32_t v = counter_plus_seed;
    v ^= (v >> 16) & 0x7fffu;                 // bits 16..30 of the masked value
    v = mul_add_u32(v, 1103515245u, 12345u);
    v ^= (v >> 13) & 0x3ffffu;                // bits 13..30
    v = mul_add_u32(v, 134775813u, 1u);
    v ^= (v >> 16) & 0x7fffu;
    return v;
}

__device__ __forceinline__ uint32_t lcg31_mix(uint32_t counter_plus_seed) {
    return lcg31_mix_bits(counter_plus_seed) & 0x7fffffffu;
}

// codec.py:222-224: u = float32(v) * 2^-30 in [0, 2], then d = u - Q_E8(u).
__device__ __forceinline__ void dither_block(uint32_t first_counter_plus_seed, float (&d)[8]) {
    float u[8], n[8];
#pragma unroll
    for (int j = 0; j < 8; j++)
        u[j] = (float)lcg31_mix(first_counter_plus_seed + (uint32_t)j) * (2.0f / 2147483648.0f);
    e8_nearest(u, n);
#pragma unroll
    for (int j = 0; j < 8; j++) d[j] = u[j] - n[j];
}

// Decode one packed block to lattice units (no beta / norm scale yet).
// counter_plus_seed is the low 32 bits of (global_block * 8 + seed); dithered == false
// skips the dither (activations and KV pages).
template <bool kDithered>
__device__ __forceinline__ void decode_codeword(uint32_t word, float q, uint32_t counter_plus_seed,
                                                float (&out)[8]) {
    float c[8], p[8];
    unpack_codeword(word, c);
    e8_coset_point(c, p);
    if (kDithered) {
        float d[8];
        dither_block(counter_plus_seed, d);
#pragma unroll
        for (int j = 0; j < 8; j++) p[j] = p[j] - d[j];
    }
    reduce_coset_point(p, q, out);
}

// ---------------------------------------------------------------------------------------
// Resolved weight blocks.
//
// A dithered block decodes to  w = (p - d) - 14 k  with p = G c the coset point of its code,
// d = u - n the dither (u the hashed uniforms, n = Q_E8(u)) and k = Q_E8((p - d) / 14).  Both
// lattice searches depend only on the stored code, the seed and the block index, so they can
// be done once when a weight is prepared: s = p + n - 14 k is a point of E8 and  w = s - u.
// resolve_codeword() runs the exact decode and stores s in 43 bits: the eight floors
// f_j = floor(s_j) + 15 as 5-bit fields (w and u bound s_j to [-14, 16]), one bit saying that
// the point lies in the half-integer coset, and the block's 2-bit beta id:
//   32-bit word  beta id in bits 0..1, f_0..f_5 at bits 2 + 5 j
//   16-bit word  f_6 at bits 0..4, f_7 at bits 5..9, half-coset flag in bit 10
// decode_resolved() then needs the hash and a handful of instructions per weight, no search and
// no division.  It builds the float 2^23 + (f_j 2^17 + 2^18 - 1 - U_j) in its mantissa, U_j being
// the top 18 bits of the 31-bit hash value (u_j 2^17, truncated), and subtracts the constant
// that leaves (s_j - u_j) 2^17: the lattice points are the exact ones, the dither is taken to
// 2^-17 of a lattice unit (the reference rounds it to 24 significant bits), far below the BF16
// rounding that follows.
constexpr float kResolvedUnit = 1.0f / 131072.0f;   // 2^-17

__device__ __forceinline__ bool resolve_codeword(uint32_t word, uint32_t counter_plus_seed, uint32_t beta_id,
                                                 uint32_t &lo, uint32_t &hi) {
    float c[8], p[8], u[8], n[8], t[8], k[8];
    unpack_codeword(word, c);
    e8_coset_point(c, p);
#pragma unroll
    for (int j = 0; j < 8; j++)
        u[j] = (float)lcg31_mix(counter_plus_seed + (uint32_t)j) * (2.0f / 2147483648.0f);
    e8_nearest(u, n);
#pragma unroll
    for (int j = 0; j < 8; j++) t[j] = div_by_14(p[j] - (u[j] - n[j]));
    e8_nearest(t, k);
    bool in_range = true;
    uint32_t field[8];
    float first_floor = 0.0f, first = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float s = (p[j] + n[j]) - 14.0f * k[j];     // half-integers of small magnitude: exact
        const float biased = __builtin_floorf(s) + 15.0f;
        in_range = in_range && biased >= 0.0f && biased <= 31.0f;
        field[j] = (uint32_t)(int)biased & 31u;
        if (j == 0) { first = s; first_floor = __builtin_floorf(s); }
    }
    lo = beta_id | (field[0] << 2) | (field[1] << 7) | (field[2] << 12) | (field[3] << 17) | (field[4] << 22) |
         (field[5] << 27);
    hi = field[6] | (field[7] << 5) | (first != first_floor ? 1024u : 0u);
    return in_range;
}

// x * c + a, low 32 bits, as one instruction (c and a are the same for every lane).
__device__ __forceinline__ uint32_t mad_u32(uint32_t x, uint32_t c, uint64_t a) {
    uint64_t r;
    asm("v_mad_u64_u32 %0, vcc, %1, %2, %3" : "=v"(r) : "v"(x), "s"(c), "v"(a) : "vcc");
    return (uint32_t)r;
}

__device__ __forceinline__ uint32_t resolved_beta_id(uint32_t lo) { return lo & 3u; }

// The four products beta_i * (row scale * kResolvedUnit) a lane keeps for its row, and the block's
// scale out of them: two compares and three selects on the id's bits.  (The empty asm keeps the four
// in registers: a select between two loads would become one load through a selected address, and the
// table would move to LDS.)
struct ResolvedScales {
    float s0, s1, s2, s3;
};
__device__ __forceinline__ ResolvedScales resolved_scales(const float (&beta)[4], float row_scale) {
    return ResolvedScales{beta[0] * row_scale, beta[1] * row_scale, beta[2] * row_scale, beta[3] * row_scale};
}
__device__ __forceinline__ float resolved_scale(const ResolvedScales &scales, uint32_t lo) {
    float s0 = scales.s0, s1 = scales.s1, s2 = scales.s2, s3 = scales.s3;
    asm("" : "+v"(s0), "+v"(s1), "+v"(s2), "+v"(s3));    // values in registers, whatever memory they came from
    const bool odd = (lo & 1u) != 0u;
    const float low = odd ? s1 : s0;
    const float high = odd ? s3 : s2;
    return (lo & 2u) ? high : low;
}

// out[j] = (s_j - u_j) * 2^17 * scale  (pass scale = weight scale * kResolvedUnit).
// The hash is evaluated on values shifted left by one bit, so that "modulo 2^31" is the
// register's own wrap-around: stage 1 is t (2 A) + 2 C, the second shift-xor masks bit 0, stage 2
// multiplies by -B and adds -3, which leaves the complement of (v B + 1) << 1, whose top 18 bits
// are 2^18 - 1 - U.  The last shift-xor of lcg31_mix_v1 only touches bits 0..14 of the value: two
// of the 18 bits used here (13 and 14), which then carry an unmixed but equally uniform bit.
// The counters of a block are seed + 8 block + j, so a block's eight counters lie in at most two
// aligned groups of eight counters [8 g, 8 g + 8), and which of its weights fall into the second one
// depends on seed & 7 alone, the same for every block of a tensor.  Inside an aligned group the
// counters differ in their low three bits only and share bits 16..30 (a group never straddles a
// multiple of 2^16 or of 2^31), so the first shift-xor of a whole group is one value
// T = x ^ (x >> 16), x = 8 g, and counter 8 g + i enters the hash as T ^ i.  A run of consecutive
// blocks therefore costs one T per aligned group it touches and one xor with a constant per weight,
// with no special case; seed & 7 is uniform, so the eight patterns are the arms of a scalar switch
// (resolved_dither_bits_run, for lanes that own two or more neighbouring blocks).

// From t_j = counter_j ^ (counter_j >> 16) to the float pattern's dither part: 2^18 - 1 - U_j in
// bits 0..17 under the exponent of 2^23 (the funnel shift that takes the hash's top 18 bits brings
// the exponent in from its other operand).  Five instructions per weight.
__device__ __forceinline__ void resolved_hash_bits(const uint32_t (&t)[8], uint32_t (&bits)[8]) {
    const uint64_t twice_c = 2u * 12345u;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t v1 = mad_u32(t[j], 2u * 1103515245u, twice_c);
        const uint32_t v1x = v1 ^ ((v1 >> 13) & 0x7fffeu);
        const uint32_t v2_complement = v1x * (0u - 134775813u) - 3u;
        bits[j] = __builtin_amdgcn_alignbit(0x4b000000u >> 18, v2_complement, 14);
    }
}

// t[b][j] for the kBlocks consecutive blocks whose first counter is counter_plus_seed (bit 31 of a
// value is not meaningful: the hash multiplies modulo 2^31 on values shifted left by one).
template <int kBlocks, int kShift>
__device__ __forceinline__ void resolved_hash_inputs_shifted(const uint32_t (&group)[kBlocks + 1], uint32_t (&t)[kBlocks][8]) {
#pragma unroll
    for (int b = 0; b < kBlocks; b++)
#pragma unroll
        for (int j = 0; j < 8; j++) t[b][j] = group[b + ((kShift + j) >> 3)] ^ (uint32_t)((kShift + j) & 7);
}

template <int kBlocks>
__device__ __forceinline__ void resolved_hash_inputs(uint32_t counter_plus_seed, uint32_t (&t)[kBlocks][8]) {
    const uint32_t shift = (uint32_t)__builtin_amdgcn_readfirstlane((int)(counter_plus_seed & 7u));   // seed & 7
    const uint32_t first = counter_plus_seed - shift;
    uint32_t group[kBlocks + 1];
#pragma unroll
    for (int g = 0; g <= kBlocks; g++) {
        const uint32_t x = first + 8u * (uint32_t)g;
        group[g] = x ^ ((x >> 16) & 0x7fffu);
    }
    switch (shift) {
        case 0: resolved_hash_inputs_shifted<kBlocks, 0>(group, t); break;
        case 1: resolved_hash_inputs_shifted<kBlocks, 1>(group, t); break;
        case 2: resolved_hash_inputs_shifted<kBlocks, 2>(group, t); break;
        case 3: resolved_hash_inputs_shifted<kBlocks, 3>(group, t); break;
        case 4: resolved_hash_inputs_shifted<kBlocks, 4>(group, t); break;
        case 5: resolved_hash_inputs_shifted<kBlocks, 5>(group, t); break;
        case 6: resolved_hash_inputs_shifted<kBlocks, 6>(group, t); break;
        default: resolved_hash_inputs_shifted<kBlocks, 7>(group, t); break;
    }
}

// The part of the decode that needs no memory: bits[b][j] as resolved_hash_bits leaves them, for
// kBlocks consecutive blocks of one lane from the first block's first counter.
template <int kBlocks>
__device__ __forceinline__ void resolved_dither_bits_run(uint32_t counter_plus_seed, uint32_t (&bits)[kBlocks][8]) {
    uint32_t t[kBlocks][8];
    resolved_hash_inputs<kBlocks>(counter_plus_seed, t);
#pragma unroll
    for (int b = 0; b < kBlocks; b++) resolved_hash_bits(t[b], bits[b]);
}

// One block by itself: its eight counters share bits 16..30 unless the block straddles a multiple of
// 2^16 (or of 2^31), which takes the counter-by-counter form of the first shift-xor.  (For a single
// block the test is cheaper than the switch of the run form, which ends the basic block and with it
// the overlap of this block's arithmetic with the next block's loads.)
__device__ __forceinline__ void resolved_dither_bits(uint32_t counter_plus_seed, uint32_t (&bits)[8]) {
    const uint32_t base = counter_plus_seed & 0x7fffffffu;
    const uint32_t high = base >> 16;
    uint32_t t[8];
    if (__builtin_expect((base & 0xffffu) > 0xfff8u || base > 0x7ffffff8u, 0)) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t x = (counter_plus_seed + (uint32_t)j) & 0x7fffffffu;
            t[j] = x ^ (x >> 16);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) t[j] = (base + (uint32_t)j) ^ high;
    }
    resolved_hash_bits(t, bits);
}

// The part that needs the stored block: out[j] = (s_j - u_j) * 2^17 * scale.  A weight's float
// pattern is its dither part plus f_j 2^17: a bit-field extract and a shift-add.
__device__ __forceinline__ void resolved_apply(uint32_t lo, uint32_t hi, const uint32_t (&bits)[8], float scale,
                                               float (&out)[8]) {
    // 2^23 + (2^18 - 1) + 15 * 2^17, less 2^16 in the half-integer coset
    const float origin = (hi & 1024u) ? 10551295.0f : 10616831.0f;
    // (float - origin) * scale as one fused multiply-add: one rounding instead of two (the difference
    // is exact in the first form, so only the final rounding can move, by half a unit in the last place)
    const float shift = -origin * scale;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        // spelled as instructions: left to itself the compiler turns the pair into shift, mask and add
        uint32_t field, pattern;
        if (j < 6) asm("v_bfe_u32 %0, %1, %2, 5" : "=v"(field) : "v"(lo), "n"(2 + 5 * (j < 6 ? j : 0)));
        else asm("v_bfe_u32 %0, %1, %2, 5" : "=v"(field) : "v"(hi), "n"(5 * (j < 6 ? 0 : j - 6)));
        asm("v_lshl_add_u32 %0, %1, 17, %2" : "=v"(pattern) : "v"(field), "v"(bits[j]));
        out[j] = __builtin_fmaf(__uint_as_float(pattern), scale, shift);
    }
}

__device__ __forceinline__ void decode_resolved(uint32_t lo, uint32_t hi, uint32_t counter_plus_seed, float scale,
                                                float (&out)[8]) {
    uint32_t bits[8];
    resolved_dither_bits(counter_plus_seed, bits);
    resolved_apply(lo, hi, bits, scale, out);
}

__device__ __forceinline__ float bf16_to_f32(uint16_t bits) {
    return __uint_as_float(((uint32_t)bits) << 16);
}

// float32 -> bfloat16, round to nearest even (finite inputs).
__device__ __forceinline__ uint16_t f32_to_bf16(float x) {
    uint32_t bits = __float_as_uint(x);
    bits += 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)(bits >> 16);
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ bf16x2 pack_bf16x2(float lo, float hi) {
    const floatx2 v = {lo, hi};
    return __builtin_convertvector(v, bf16x2);          // v_cvt_pk_bf16_f32, round to nearest even
}

__device__ __forceinline__ float f16_to_f32(uint16_t bits) {
    return (float)__builtin_bit_cast(_Float16, bits);
}

}  // namespace nq
