/*
 * CPU oracle for the packed W4A4KV4 path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithm of the reference's CPU
 * (torch) implementation so that the HIP kernels can be checked bit for bit
 * on integer outputs and to a stated tolerance on floating-point outputs.
 * Nothing in the shipped library links, loads or calls it: only the test
 * suite, the smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Arithmetic dialect.  The reference's goldens come from torch on the CPU,
 * whose float32 behaviour this file reproduces operation by operation:
 *   - every sum of eight squared deltas is strictly sequential, j = 0..7,
 *     squares rounded before they are added (no fused multiply-add);
 *   - `x / beta` and `p / q` are IEEE divisions, never reciprocal multiplies;
 *   - rounding is round-half-to-even; argmax / argmin keep the first index;
 *   - the half-coset residual is (x - 0.5) - rint(x - 0.5);
 *   - row norms use eight interleaved FMA accumulators, summed 0..7, sqrt;
 *   - the normalisation scale is (1 / norm) * float(sqrt(n)).
 * Build with -ffp-contract=off and without -ffast-math (see the Makefile);
 * explicit fmaf() marks the only fused operations.
 *
 * Every function cites the reference file:line it follows
 * (paths relative to the reference checkout).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define NQO_EXPORT __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* E8 nearest point: nestquant/core/lattice.py:18-81                   */
/* ------------------------------------------------------------------ */

/* lattice.py:18-34 `_nearest_even_sum_integer` */
static void d8_nearest(const float *p, float *out) {
    float residual[8];
    float sum = 0.0f;
    for (int j = 0; j < 8; j++) {
        out[j] = rintf(p[j]);                 /* torch.round: half to even */
        residual[j] = p[j] - out[j];
        sum = sum + out[j];                   /* rounded.sum(dim=-1), float32 */
    }
    const int parity = fmodf(sum, 2.0f) != 0.0f;   /* remainder(sum, 2) != 0 */
    int best = 0;
    float best_abs = fabsf(residual[0]);
    for (int j = 1; j < 8; j++) {             /* argmax keeps the first index */
        float v = fabsf(residual[j]);
        if (v > best_abs) { best_abs = v; best = j; }
    }
    if (parity)
        out[best] += (residual[best] >= 0.0f) ? 1.0f : -1.0f;
}

/* lattice.py:37-81 `nearest_e8`, tie_break="upstream_half" */
static float e8_nearest(const float *x, float *out) {
    float a[8], b[8], xm[8];
    d8_nearest(x, a);
    for (int j = 0; j < 8; j++) xm[j] = x[j] - 0.5f;
    d8_nearest(xm, b);
    for (int j = 0; j < 8; j++) b[j] = b[j] + 0.5f;
    float ea = 0.0f, eb = 0.0f;
    for (int j = 0; j < 8; j++) {
        float da = x[j] - a[j];
        float sa = da * da;
        ea = ea + sa;
        float db = x[j] - b[j];
        float sb = db * db;
        eb = eb + sb;
    }
    const float *pick = (ea < eb) ? a : b;    /* ties go to the half coset */
    for (int j = 0; j < 8; j++) out[j] = pick[j];
    return ea < eb ? ea : eb;
}

NQO_EXPORT void nqo_nearest_e8(const float *x, float *out, float *dist, size_t nvec) {
    for (size_t i = 0; i < nvec; i++) {
        float d = e8_nearest(x + 8 * i, out + 8 * i);
        if (dist) dist[i] = d;
    }
}

/* ------------------------------------------------------------------ */
/* Nested code: nestquant/core/codec.py:30-142                         */
/* ------------------------------------------------------------------ */

/* Integer generator coordinates of a lattice point.  codec.py:89-90 multiplies
 * by the inverse generator and rounds; the closed form below is the same map
 * (nestquant/runtime/nqkv_page.py:141-148) and is exact in float32. */
static void e8_coords(const float *l, long long *c) {
    float c7 = 2.0f * l[7];
    float c6 = l[6] - l[7];
    float c5 = l[5] + c6 - l[7];
    float c4 = l[4] + c5 - l[7];
    float c3 = l[3] + c4 - l[7];
    float c2 = l[2] + c3 - l[7];
    float c1 = l[1] + c2 - l[7];
    float c0 = 0.5f * (l[0] + c1 - l[7]);
    float f[8] = {c0, c1, c2, c3, c4, c5, c6, c7};
    for (int j = 0; j < 8; j++) c[j] = (long long)rintf(f[j]);
}

/* codec.py:30-42 generator applied to an integer code (exact in float32) */
static void e8_coset_point(const int *c, float *p) {
    float f[8];
    for (int j = 0; j < 8; j++) f[j] = (float)c[j];
    float h = 0.5f * f[7];
    p[0] = 2.0f * f[0] - f[1] + h;
    for (int j = 1; j < 6; j++) p[j] = f[j] - f[j + 1] + h;
    p[6] = f[6] + h;
    p[7] = h;
}

/* codec.py:53-102 `encode_nested` (codes only; the overload flag is statistics) */
static void encode_block(const float *x, const float *dither, int q, int *code) {
    float shifted[8], lattice[8];
    long long c[8];
    for (int j = 0; j < 8; j++) shifted[j] = dither ? x[j] + dither[j] : x[j];
    e8_nearest(shifted, lattice);
    e8_coords(lattice, c);
    for (int j = 0; j < 8; j++) {
        long long r = c[j] % q;               /* torch.remainder: non-negative */
        if (r < 0) r += q;
        code[j] = (int)r;
    }
}

/* codec.py:105-142 `decode_nested` */
static void decode_block(const int *code, const float *dither, int q, float *out) {
    float p[8], scaled[8], k[8];
    const float qf = (float)q;
    e8_coset_point(code, p);
    if (dither)
        for (int j = 0; j < 8; j++) p[j] = p[j] - dither[j];
    for (int j = 0; j < 8; j++) scaled[j] = p[j] / qf;   /* IEEE division */
    e8_nearest(scaled, k);
    for (int j = 0; j < 8; j++) out[j] = p[j] - qf * k[j];
}

NQO_EXPORT void nqo_encode_nested(const float *x, const float *dither, int q,
                                  int32_t *code, size_t nvec) {
    for (size_t i = 0; i < nvec; i++) {
        int c[8];
        encode_block(x + 8 * i, dither ? dither + 8 * i : NULL, q, c);
        for (int j = 0; j < 8; j++) code[8 * i + j] = c[j];
    }
}

NQO_EXPORT void nqo_decode_nested(const int32_t *code, const float *dither, int q,
                                  float *out, size_t nvec) {
    for (size_t i = 0; i < nvec; i++) {
        int c[8];
        for (int j = 0; j < 8; j++) c[j] = code[8 * i + j];
        decode_block(c, dither ? dither + 8 * i : NULL, q, out + 8 * i);
    }
}

/* ------------------------------------------------------------------ */
/* Stateless dither lcg31_mix_v1: nestquant/core/codec.py:176-224      */
/* ------------------------------------------------------------------ */

/* codec.py:213-222, all stages reduced modulo 2^31 in int64 */
static uint32_t lcg31_mix(uint64_t counter, uint64_t seed) {
    const uint64_t m = (uint64_t)1 << 31;
    uint64_t v = (counter + seed) % m;
    v ^= v >> 16;
    v = (v * 1103515245ull + 12345ull) % m;
    v ^= v >> 13;
    v = (v * 134775813ull + 1ull) % m;
    v ^= v >> 16;
    return (uint32_t)v;
}

static void dither_block(uint64_t global_block, uint64_t seed, float *d) {
    float u[8], n[8];
    for (int j = 0; j < 8; j++) {
        uint32_t v = lcg31_mix(global_block * 8 + (uint64_t)j, seed);
        /* values.to(float32) * (2.0 / 2**31): int->float is round-to-nearest-even,
         * the scale is a power of two (codec.py:222-223) */
        u[j] = (float)v * (2.0f / 2147483648.0f);
    }
    e8_nearest(u, n);
    for (int j = 0; j < 8; j++) d[j] = u[j] - n[j];
}

NQO_EXPORT void nqo_hash_lcg31(const uint64_t *counters, uint64_t seed, uint32_t *out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = lcg31_mix(counters[i], seed);
}

NQO_EXPORT void nqo_dither_stateless(uint64_t block_count, uint64_t seed,
                                     uint64_t block_offset, float *out) {
#pragma omp parallel for schedule(static)
    for (long long b = 0; b < (long long)block_count; b++)
        dither_block(block_offset + (uint64_t)b, seed, out + 8 * b);
}

/* ------------------------------------------------------------------ */
/* Row quantiser: nestquant/core/quantizer.py:214-301, 39-51           */
/* ------------------------------------------------------------------ */

/* torch.linalg.vector_norm(x, 2, dim=-1) on a contiguous float32 row, as torch's
 * CPU kernel evaluates it (quantizer.py:257): eight interleaved accumulators,
 * element i goes to lane i % 8 with a fused multiply-add, lanes added 0..7,
 * then sqrt.  A tail shorter than eight is added after the lanes, unfused. */
static float row_norm_f32(const float *x, size_t n) {
    float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    size_t full = n - (n % 8);
    for (size_t i = 0; i < full; i += 8)
        for (int k = 0; k < 8; k++) lane[k] = fmaf(x[i + k], x[i + k], lane[k]);
    float acc = 0.0f;
    for (int k = 0; k < 8; k++) acc = acc + lane[k];
    for (size_t i = full; i < n; i++) { float s = x[i] * x[i]; acc = acc + s; }
    return sqrtf(acc);
}

NQO_EXPORT void nqo_row_norms(const float *x, size_t rows, size_t n, float *norms) {
    for (size_t r = 0; r < rows; r++) norms[r] = row_norm_f32(x + r * n, n);
}

/* quantizer.py:257-261: normalise one row to L2 norm sqrt(n) */
static void normalise_row(const float *x, size_t n, float norm, float *y) {
    if (!(norm > 0.0f)) { for (size_t i = 0; i < n; i++) y[i] = 0.0f; return; }
    /* math.sqrt(n) / norms  ==  norms.reciprocal() * float32(sqrt(n)) in torch */
    const float scale = (1.0f / norm) * (float)sqrt((double)n);
    for (size_t i = 0; i < n; i++) y[i] = x[i] * scale;
}

/* quantizer.py:273-289: one block against every beta; first strict minimum wins */
static int quantize_block(const float *y, const float *dither, int q,
                          const float *betas, int nbeta, int *best_code) {
    int best = 0;
    float best_err = 0.0f;
    for (int b = 0; b < nbeta; b++) {
        float scaled[8], recon[8];
        int code[8];
        for (int j = 0; j < 8; j++) scaled[j] = y[j] / betas[b];     /* IEEE division */
        encode_block(scaled, dither, q, code);
        decode_block(code, dither, q, recon);
        float err = 0.0f;
        for (int j = 0; j < 8; j++) {
            float r = recon[j] * betas[b];
            float d = r - y[j];
            float s = d * d;
            err = err + s;
        }
        if (b == 0 || err < best_err) {
            best_err = err; best = b;
            for (int j = 0; j < 8; j++) best_code[j] = code[j];
        }
    }
    return best;
}

/* quantizer.py:214-301 `quantize_rows`.
 * x [rows, n] float32; betas already cast to float32; dither [rows, n/8, 8] or NULL.
 * codes [rows * n] one per byte in [0, q); beta_idx [rows * n/8]; norms [rows]. */
NQO_EXPORT void nqo_quantize_rows(const float *x, size_t rows, size_t n, int q,
                                  const float *betas, int nbeta, const float *dither,
                                  uint8_t *codes, uint8_t *beta_idx, float *norms) {
#pragma omp parallel
    {
        float *y = (float *)malloc(n * sizeof(float));
#pragma omp for schedule(static)
        for (long long r = 0; r < (long long)rows; r++) {
            const float *row = x + (size_t)r * n;
            float norm = row_norm_f32(row, n);
            norms[r] = norm;
            normalise_row(row, n, norm, y);
            for (size_t b = 0; b < n / 8; b++) {
                int code[8];
                const float *d = dither ? dither + ((size_t)r * n + b * 8) : NULL;
                int best = quantize_block(y + 8 * b, d, q, betas, nbeta, code);
                beta_idx[(size_t)r * (n / 8) + b] = (uint8_t)best;
                for (int j = 0; j < 8; j++) codes[(size_t)r * n + 8 * b + j] = (uint8_t)code[j];
            }
        }
        free(y);
    }
}

/* quantizer.py:39-51 `QuantizedRows.dequantize` (float32):
 * (decode(codes) * beta[beta_idx]) * (norm / float32(sqrt(n))).
 * `seed_dither` != 0 regenerates the stateless dither of global block
 * (row_offset + r) * n/8 + b  (tensor_checkpoint.py:267-272). */
NQO_EXPORT void nqo_dequantize_rows(const uint8_t *codes, const uint8_t *beta_idx,
                                    const float *norms, const float *betas, int q,
                                    size_t rows, size_t n, const float *dither,
                                    int seed_dither, uint64_t seed, float *out) {
    const float sqrt_n = (float)sqrt((double)n);
#pragma omp parallel for schedule(static)
    for (long long r = 0; r < (long long)rows; r++) {
        const float scale = norms[r] / sqrt_n;      /* tensor / python float: IEEE */
        for (size_t b = 0; b < n / 8; b++) {
            int code[8];
            float d[8], recon[8];
            const float *dp = NULL;
            size_t base = (size_t)r * n + 8 * b;
            for (int j = 0; j < 8; j++) code[j] = codes[base + j];
            if (seed_dither) { dither_block((uint64_t)r * (n / 8) + b, seed, d); dp = d; }
            else if (dither) dp = dither + base;
            decode_block(code, dp, q, recon);
            float beta = betas[beta_idx[(size_t)r * (n / 8) + b]];
            for (int j = 0; j < 8; j++) {
                float v = recon[j] * beta;
                out[base + j] = v * scale;
            }
        }
    }
}

/* ------------------------------------------------------------------ */
/* NQPK fixed-width streams: nestquant/core/packing.py:191-225         */
/* ------------------------------------------------------------------ */

/* packing.py:191-208 `_pack_unsigned`: value i sits in bits
 * [(i % per_byte) * width, +width) of byte i / per_byte; padding bits are 0. */
NQO_EXPORT void nqo_pack_unsigned(const uint8_t *values, size_t count, int width, uint8_t *out) {
    const int per_byte = 8 / width;
    size_t nbytes = (count * (size_t)width + 7) / 8;
    memset(out, 0, nbytes);
    for (size_t i = 0; i < count; i++)
        out[i / per_byte] |= (uint8_t)(values[i] << ((i % per_byte) * width));
}

/* packing.py:211-225 `_unpack_unsigned` */
NQO_EXPORT void nqo_unpack_unsigned(const uint8_t *payload, size_t count, int width, uint8_t *out) {
    const int per_byte = 8 / width;
    const uint8_t mask = (uint8_t)((1u << width) - 1u);
    for (size_t i = 0; i < count; i++)
        out[i] = (payload[i / per_byte] >> ((i % per_byte) * width)) & mask;
}

/* ------------------------------------------------------------------ */
/* Hadamard: nestquant/core/rotation.py:12-27 (float32)                */
/* ------------------------------------------------------------------ */

/* Sylvester butterflies with growing width, then one division by sqrt(n). */
NQO_EXPORT void nqo_hadamard_f32(float *x, size_t rows, size_t n) {
    const float root = (float)sqrt((double)n);
#pragma omp parallel for schedule(static)
    for (long long r = 0; r < (long long)rows; r++) {
        float *y = x + (size_t)r * n;
        for (size_t width = 1; width < n; width *= 2)
            for (size_t base = 0; base < n; base += 2 * width)
                for (size_t i = 0; i < width; i++) {
                    float l = y[base + i], rr = y[base + width + i];
                    y[base + i] = l + rr;
                    y[base + width + i] = l - rr;
                }
        for (size_t i = 0; i < n; i++) y[i] = y[i] / root;
    }
}

/* ------------------------------------------------------------------ */
/* Decode-then-matmul reference for the W4A4 product                   */
/* (nestquant/runtime/triton_w4a4_linear.py:319-480 scalar flavour:    */
/*  FP32 operands, no BF16 rounding; accumulated in double here)       */
/* ------------------------------------------------------------------ */

NQO_EXPORT void nqo_matmul_nt(const float *a, const float *w, size_t m, size_t n, size_t k,
                              float *out) {
#pragma omp parallel for schedule(static)
    for (long long j = 0; j < (long long)n; j++)
        for (size_t i = 0; i < m; i++) {
            double acc = 0.0;
            const float *ar = a + i * k, *wr = w + (size_t)j * k;
            for (size_t t = 0; t < k; t++) acc += (double)ar[t] * (double)wr[t];
            out[i * n + (size_t)j] = (float)acc;
        }
}

/* ------------------------------------------------------------------ */
/* Decode attention oracle: nestquant/runtime/nqkv_attention.py:14-86  */
/* ------------------------------------------------------------------ */

/* One (query head, sequence): softmax(q . K^T * scale) . V over `tokens`
 * dequantised float32 rows.  k, v: [tokens, kv_heads, dim]; q, out: [q_heads, dim]. */
NQO_EXPORT void nqo_attention_dense(const float *query, const float *k, const float *v,
                                    size_t tokens, int q_heads, int kv_heads, int dim,
                                    float scale, float *out) {
    const int group = q_heads / kv_heads;
    for (int h = 0; h < q_heads; h++) {
        const int g = h / group;
        double *score = (double *)malloc((tokens ? tokens : 1) * sizeof(double));
        double top = -INFINITY;
        for (size_t t = 0; t < tokens; t++) {
            double s = 0.0;
            const float *kr = k + (t * (size_t)kv_heads + (size_t)g) * (size_t)dim;
            for (int d = 0; d < dim; d++) s += (double)query[h * dim + d] * (double)kr[d];
            score[t] = s * (double)scale;
            if (score[t] > top) top = score[t];
        }
        double denom = 0.0;
        for (size_t t = 0; t < tokens; t++) { score[t] = exp(score[t] - top); denom += score[t]; }
        for (int d = 0; d < dim; d++) {
            double acc = 0.0;
            for (size_t t = 0; t < tokens; t++)
                acc += score[t] * (double)v[(t * (size_t)kv_heads + (size_t)g) * (size_t)dim + d];
            out[h * dim + d] = tokens ? (float)(acc / denom) : 0.0f;
        }
        free(score);
    }
}

/* ------------------------------------------------------------------ */
/* Exhaustive check of the GPU kernels' three-operation division by 14 */
/* ------------------------------------------------------------------ */

/* For every finite float32 p with 1e-30 <= |p| <= 1e30 (and +-0) compares
 *   q0 = p * c;  r = fma(-14, q0, p);  q1 = fma(r, c, q0),  c = float(1/14)
 * with the IEEE quotient p / 14.  Returns the number of inputs whose results
 * differ as numbers (a differing sign of zero is not counted). */
NQO_EXPORT long long nqo_count_div14_mismatches(void) {
    const float c = 1.0f / 14.0f;
    long long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (long long b = 0; b < (1LL << 32); b++) {
        uint32_t bits = (uint32_t)b;
        float p;
        memcpy(&p, &bits, 4);
        if (!isfinite(p)) continue;
        float ap = fabsf(p);
        if (ap != 0.0f && (ap < 1e-30f || ap > 1e30f)) continue;
        float q0 = p * c;
        float r = fmaf(-14.0f, q0, p);
        float q1 = fmaf(r, c, q0);
        float t = p / 14.0f;
        if (q1 != t) bad++;
    }
    return bad;
}

/* The many-row encoder divides by a beta through its correctly rounded reciprocal:
 *   q0 = a * r;  q1 = fma(fma(-b, q0, a), r, q0);  q2 = fma(fma(-b, q1, a), r, q1),  r = 1 / b
 * Compared with the IEEE quotient a / b for every float32 a with 2^-61 <= |a| < 2^40 (the
 * kernel takes the IEEE division below that magnitude) and for a = 0.  Returns the number of
 * inputs whose results differ as numbers. */
NQO_EXPORT long long nqo_count_reciprocal_division_mismatches(float b) {
    volatile float one = 1.0f;
    const float r = one / b;
    long long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (long long e = 66; e < 168; e++) {
        for (uint32_t m = 0; m < (1u << 23); m++) {
            for (int sign = 0; sign < 2; sign++) {
                uint32_t bits = ((uint32_t)sign << 31) | ((uint32_t)e << 23) | m;
                float a;
                memcpy(&a, &bits, 4);
                float q = a * r;
                q = fmaf(fmaf(-b, q, a), r, q);
                q = fmaf(fmaf(-b, q, a), r, q);
                if (q != a / b) bad++;
            }
        }
    }
    const float zero = 0.0f;
    float q = zero * r;
    q = fmaf(fmaf(-b, q, zero), r, q);
    q = fmaf(fmaf(-b, q, zero), r, q);
    if (q != 0.0f) bad++;
    return bad;
}

NQO_EXPORT int nqo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

NQO_EXPORT void nqo_set_num_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}
