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
//
// `hint` (optional) receives six bits that let e8_nearest_hinted() rebuild the same point
// without searching: bit 0 = the integer coset won, bit 1 = a coordinate was moved,
// bits 2..4 = which one, bit 5 = it moved down (-1).
template <bool kWantHint>
__device__ __forceinline__ void e8_nearest_impl(const float (&x)[8], float (&out)[8], uint32_t *hint) {
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
    uint32_t hint_a = 0u;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const bool top = fabsf(ea[j]) == max_a;
        const bool hit = top && !done_a;           // first coordinate with the largest |residual|
        done_a = done_a || top;
        const float sq = ea[j] * ea[j];
        dist_a = dist_a + (hit ? alt_a : sq);
        // residual >= 0 moves up (a residual is never -0)
        a[j] = hit ? a[j] + __builtin_copysignf(1.0f, ea[j]) : a[j];
        if (kWantHint) hint_a = hit ? (2u | ((uint32_t)j << 2) | (ea[j] < 0.0f ? 32u : 0u)) : hint_a;
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
    uint32_t hint_b = 0u;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const bool top = fabsf(eb[j]) == max_b;
        const bool hit = top && !done_b;
        done_b = done_b || top;
        const float half_point = b[j] + 0.5f;
        b[j] = hit ? half_point + __builtin_copysignf(1.0f, eb[j]) : half_point;
        const float t = x[j] - b[j];
        dist_b = dist_b + t * t;
        if (kWantHint) hint_b = hit ? (2u | ((uint32_t)j << 2) | (eb[j] < 0.0f ? 32u : 0u)) : hint_b;
    }
    const bool pick_a = dist_a < dist_b;           // ties go to the half-integer coset
#pragma unroll
    for (int j = 0; j < 8; j++) out[j] = pick_a ? a[j] : b[j];
    if (kWantHint) *hint = pick_a ? (hint_a | 1u) : hint_b;
}

__device__ __forceinline__ void e8_nearest(const float (&x)[8], float (&out)[8]) {
    e8_nearest_impl<false>(x, out, nullptr);
}

// The point e8_nearest() returns for x, rebuilt from the six hint bits it emitted for the
// same x: round in the chosen coset, move the recorded coordinate.  Same float operations
// as the search performs on the winning coset, so the result is bit-identical.
__device__ __forceinline__ void e8_nearest_hinted(const float (&x)[8], uint32_t hint, float (&out)[8]) {
    // x - (+0) and r + (-0) leave every float, signed zeros included, unchanged
    const float shift = (hint & 1u) ? 0.0f : 0.5f;
    const float back = (hint & 1u) ? -0.0f : 0.5f;
    const float step = (hint & 2u) ? ((hint & 32u) ? -1.0f : 1.0f) : 0.0f;
    const uint32_t moved = (hint >> 2) & 7u;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float point = __builtin_rintf(x[j] - shift) + back;
        out[j] = moved == (uint32_t)j ? point + step : point;
    }
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

// codec.py:105-142 `decode_nested` for one block given its coset point (already minus
// the dither when there is one): the minimum-energy representative p - q * Q(p / q).
// kHint: 0 = search, 1 = rebuild from `hint`, 2 = search and emit `hint`.
template <int kHint = 0>
__device__ __forceinline__ void reduce_coset_point(const float (&p)[8], float q, float (&out)[8],
                                                   uint32_t *hint = nullptr) {
    float z[8], k[8];
#pragma unroll
    for (int j = 0; j < 8; j++) z[j] = (q == 14.0f) ? div_by_14(p[j]) : p[j] / q;   // IEEE division
    if (kHint == 1) e8_nearest_hinted(z, *hint, k);
    else if (kHint == 2) e8_nearest_impl<true>(z, k, hint);
    else e8_nearest(z, k);
#pragma unroll
    for (int j = 0; j < 8; j++) out[j] = p[j] - q * k[j]; // exact
}

// codec.py:213-222 / nestquant/runtime/nqrt4_device.cuh:7-17: lcg31_mix_v1.  Only the
// low 31 bits of every stage matter, so masks are folded into bit-field extracts.
__device__ __forceinline__ uint32_t lcg31_mix(uint32_t counter_plus_seed) {
    uint32_t v = counter_plus_seed;
    v ^= (v >> 16) & 0x7fffu;                 // bits 16..30 of the masked value
    v = v * 1103515245u + 12345u;
    v ^= (v >> 13) & 0x3ffffu;                // bits 13..30
    v = v * 134775813u + 1u;
    v ^= (v >> 16) & 0x7fffu;
    return v & 0x7fffffffu;
}

// codec.py:222-224: u = float32(v) * 2^-30 in [0, 2], then d = u - Q_E8(u).
template <int kHint = 0>
__device__ __forceinline__ void dither_block(uint32_t first_counter_plus_seed, float (&d)[8],
                                             uint32_t *hint = nullptr) {
    float u[8], n[8];
#pragma unroll
    for (int j = 0; j < 8; j++)
        u[j] = (float)lcg31_mix(first_counter_plus_seed + (uint32_t)j) * (2.0f / 2147483648.0f);
    if (kHint == 1) e8_nearest_hinted(u, *hint, n);
    else if (kHint == 2) e8_nearest_impl<true>(u, n, hint);
    else e8_nearest(u, n);
#pragma unroll
    for (int j = 0; j < 8; j++) d[j] = u[j] - n[j];
}

// Decode one packed block to lattice units (no beta / norm scale yet).
// counter_plus_seed is the low 32 bits of (global_block * 8 + seed); dithered == false
// skips the dither (activations and KV pages).
//
// Decode hints (dithered weights only).  Both lattice searches of a weight block depend only
// on the stored code, the seed and the block index, so their outcomes can be computed once
// when a weight is prepared and kept as 12 bits per block (bits 0..5: dither search,
// bits 6..11: coarse search; layout in e8_nearest_impl).  kHint = 1 rebuilds both points
// from `*hints` instead of searching -- the same values, about half the instructions;
// kHint = 2 searches and writes `*hints`.
template <bool kDithered, int kHint = 0>
__device__ __forceinline__ void decode_codeword(uint32_t word, float q, uint32_t counter_plus_seed,
                                                float (&out)[8], uint32_t *hints = nullptr) {
    float c[8], p[8];
    unpack_codeword(word, c);
    e8_coset_point(c, p);
    uint32_t hint_dither = 0u, hint_coarse = 0u;
    if (kHint == 1) { hint_dither = *hints & 63u; hint_coarse = (*hints >> 6) & 63u; }
    if (kDithered) {
        float d[8];
        dither_block<kHint>(counter_plus_seed, d, &hint_dither);
#pragma unroll
        for (int j = 0; j < 8; j++) p[j] = p[j] - d[j];
    }
    reduce_coset_point<kHint>(p, q, out, &hint_coarse);
    if (kHint == 2) *hints = hint_dither | (hint_coarse << 6);
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

__device__ __forceinline__ float f16_to_f32(uint16_t bits) {
    return (float)__builtin_bit_cast(_Float16, bits);
}

}  // namespace nq
