/*
 * libnqhip: C ABI of the MI355X (gfx950) kernels for NestQuant's packed W4A4KV4 path.
 *
 * Conventions
 *  - Every pointer named *_dev / documented "device" is a device pointer owned by the
 *    caller; the library borrows it for the duration of the enqueued work and never
 *    allocates, frees or synchronises.  Work is enqueued on `stream` (a hipStream_t
 *    passed as void*; NULL is the default stream) and is capturable in a HIP graph.
 *  - Every function returns NQ_OK (0) or a negative NQ_ERR_* code; nq_last_error()
 *    then returns a thread-local, human-readable message.  Shapes are validated on the
 *    host before anything is launched.
 *  - Streams of 4-bit codes and 2-bit beta ids use the reference's NQPK layout:
 *    value i of a flat row-major stream sits in bits [(i % per_byte) * width, +width)
 *    of byte i / per_byte (nestquant/core/packing.py:191-208).  One 8-value block is
 *    one little-endian uint32; four consecutive blocks share one beta byte.
 *  - dtype tags: NQ_F32 = 0, NQ_BF16 = 1, NQ_F16 = 2.
 *
 * File:line citations name the reference interface each entry point replaces
 * (paths relative to the reference checkout).
 */
#ifndef NQHIP_H
#define NQHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NQ_OK 0
#define NQ_ERR_ARGUMENT (-1)   /* bad pointer, dtype tag or flag            -> ValueError / TypeError */
#define NQ_ERR_SHAPE (-2)      /* shape unsupported by the kernel family    -> ValueError            */
#define NQ_ERR_LAUNCH (-3)     /* hipGetLastError() after the launch        -> RuntimeError          */
#define NQ_ERR_WORKSPACE (-4)  /* workspace missing or too small            -> RuntimeError          */

#define NQ_F32 0
#define NQ_BF16 1
#define NQ_F16 2

/* ABI version of this header; bumped on any signature change. */
int nq_abi_version(void);

/* Message for the last non-zero return on the calling thread ("" if none). */
const char *nq_last_error(void);

/*
 * Nearest E8 lattice point of `count` float32 vectors of length 8 (ties between the
 * two cosets go to the half-integer coset).
 * Replaces: e8_nearest(x[N,8]) -> [N,8], nestquant/runtime/cuda_e8.cu:8-59 and
 * cuda_e8.py:30-43 (that one launches on the default stream; this one on `stream`).
 */
int nq_e8_nearest(const float *x_dev, float *out_dev, int64_t count, void *stream);

/*
 * Row quantiser with per-8-block multi-beta selection, packed output (NQA4 activations
 * and NQKV4 page rows): L2 row norm, normalise to norm sqrt(n), for each of `beta_count`
 * betas encode + decode + error, keep the first minimum, pack 4-bit codes and 2-bit ids.
 *   x_dev      [rows, n] row-major, dtype tag x_dtype (BF16 / F16 are promoted to F32)
 *   betas_dev  float32[beta_count], 1 <= beta_count <= 4
 *   codes_dev  uint8[rows * n / 2]; beta_ids_dev uint8[rows * n / 32]; norms_dev float32[rows]
 * With has_dither != 0 the subtractive stateless dither lcg31_mix_v1 of global block
 * block_offset + r * n/8 + b and `seed` is added before the lattice search and removed
 * after it: this is the NQRT4 weight encoder (nestquant/core/quantizer.py:214-301 with
 * generate_e8_dither_stateless, nestquant/core/codec.py:176-224).
 * decoded_bf16_dev (optional, may be NULL): BF16 [rows, n] decode of the stored codes,
 * bf16((decode * beta) * (norm / sqrt(n))), which the linear kernels accept in place of
 * decoding the packed activation again.
 * Requires n % 32 == 0, n <= 32768, 2 <= q <= 16.
 * Replaces: _quantize_rows_cuda_fused + _nqkv_encode_kernel + _pack_unsigned_cuda,
 * nestquant/runtime/nqkv_page.py:332-372, 97-185, 446-456 (called by
 * quantize_activation_cuda, triton_w4a4_linear.py:581-617, and quantize_nqkv_page_cuda,
 * nqkv_page.py:241-329); arithmetic follows nestquant/core/quantizer.py:214-301.
 */
int nq_quantize_rows(const void *x_dev, int x_dtype, int64_t rows, int64_t n, int q,
                     const float *betas_dev, int beta_count, int has_dither, int64_t seed,
                     int64_t block_offset, uint8_t *codes_dev, uint8_t *beta_ids_dev,
                     float *norms_dev, void *decoded_bf16_dev, void *stream);

/*
 * Inverse of nq_quantize_rows: out[r, :] = (decode(codes) * beta[id]) * (norm[r] / sqrt(n)).
 * With has_dither != 0 the stateless dither lcg31_mix_v1 of global block
 * block_offset + r * n/8 + b and `seed` is regenerated and subtracted (NQRT4 weights).
 * out dtype tag out_dtype.  Requires n % 32 == 0.
 * Replaces: dequantize_nqkv_page_triton / _nqkv_decode_kernel,
 * nestquant/runtime/nqkv_page.py:494-537, 22-95; the NQA4 diagnostic decode
 * nqa4_decode_m16_kernel, nestquant/runtime/nqrt4_w4a4_mma.cu:83-93; arithmetic of
 * QuantizedRows.dequantize, nestquant/core/quantizer.py:39-51.
 */
int nq_dequantize_rows(const uint8_t *codes_dev, const uint8_t *beta_ids_dev,
                       const float *norms_dev, const float *betas_dev, int64_t rows,
                       int64_t n, int q, int has_dither, int64_t seed, int64_t block_offset,
                       void *out_dev, int out_dtype, void *stream);

/*
 * Packed W4A4 linear for decode, M = 1..8 tokens: y[m, n] = sum_k bf16(a[m, k]) * bf16(w[n, k]),
 * FP32 accumulation; the weight is decoded in registers from its packed stream (dither
 * regenerated; counter = weight_offset * 8 + n * K + k).
 *   act_*            NQA4 streams of [M, K] (codes M*K/2 B, beta ids M*K/32 B, norms f32[M], betas f32[4])
 *   act_decoded_dev  optional BF16 [M, K] decode of the same activation (from nq_quantize_rows);
 *                    when NULL the packed streams are decoded once into the workspace,
 *                    when given the packed streams may be NULL
 *   w_*              NQRT4 streams of [N, K] (codes N*K/2 B, beta ids N*K/32 B, norms f32[N], betas f32[4])
 *   out_dev          [M, N] of out_dtype (NQ_F32 or NQ_BF16)
 *   split_k          1, 2, 4 or 8 slices of K reduced in ascending order (deterministic); 0 lets
 *                    the library choose
 *   workspace_dev    at least nq_w4a4_gemv_workspace_bytes() bytes, 16-byte aligned (may be
 *                    NULL when that is 0)
 * Requires q = 14, K % 32 == 0, (K / split_k) % 32 == 0, 1 <= M <= 8.
 * Replaces: run_m1 / run_m1_splitk_probe / run_small_m / run_small_m_splitk_probe of the
 * torch extension, nestquant/runtime/nqrt4_w4a4_mma_binding.cpp:3-46, kernels
 * nestquant/runtime/nqrt4_w4a4_mma.cu:901-947, 952-1001, 411-420, 229-286.
 */
int nq_w4a4_gemv(const uint8_t *act_codes_dev, const uint8_t *act_beta_ids_dev,
                 const float *act_norms_dev, const float *act_betas_dev,
                 const void *act_decoded_dev, const uint8_t *w_codes_dev,
                 const uint8_t *w_beta_ids_dev, const float *w_norms_dev,
                 const float *w_betas_dev, int m, int k, int n, int64_t weight_offset,
                 int64_t weight_seed, int split_k, void *out_dev, int out_dtype,
                 void *workspace_dev, size_t workspace_bytes, void *stream);

size_t nq_w4a4_gemv_workspace_bytes(int m, int k, int n, int split_k, int have_decoded_activation);

/*
 * Packed W4A4 linear for prefill, any M >= 1 (meant for M >= 9): same product and same
 * arguments as nq_w4a4_gemv, computed on the matrix cores (v_mfma_f32_32x32x16_bf16).  The
 * weight tile is decoded once per call into double-buffered LDS as MFMA B fragments; ragged
 * M is padded to a multiple of 32 with zero rows inside the kernel and M above 512 is
 * processed in chunks of 512 rows.  split_k in {0 (library picks), 1, 2, 4, 8, 16}.
 * Requires q = 14, K % 128 == 0, (K / split_k) % 128 == 0.
 * Replaces: run_m16 / run_large_m_staged of the torch extension
 * (nestquant/runtime/nqrt4_w4a4_mma_binding.cpp:3-46, kernels
 * nestquant/runtime/nqrt4_w4a4_mma.cu:124-171, 606-667) and the Python chunk-and-pad wrapper
 * linear_packed_w4a4_mma_chunked_staged (nestquant/runtime/cuda_w4a4_mma.py:393-484).
 */
int nq_w4a4_gemm(const uint8_t *act_codes_dev, const uint8_t *act_beta_ids_dev,
                 const float *act_norms_dev, const float *act_betas_dev,
                 const void *act_decoded_dev, const uint8_t *w_codes_dev,
                 const uint8_t *w_beta_ids_dev, const float *w_norms_dev,
                 const float *w_betas_dev, int m, int k, int n, int64_t weight_offset,
                 int64_t weight_seed, int split_k, void *out_dev, int out_dtype,
                 void *workspace_dev, size_t workspace_bytes, void *stream);

size_t nq_w4a4_gemm_workspace_bytes(int m, int k, int n, int split_k, int have_decoded_activation);

#ifdef __cplusplus
}
#endif

#endif /* NQHIP_H */
