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
 * hadamard != 0 first rotates every row with the normalized Hadamard transform (n a power
 * of two), in the arithmetic of x_dtype as nq_hadamard does with stage_dtype = x_dtype, so
 * a Linear input needs one launch for rotate + norm + encode + pack.
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
                     int64_t block_offset, int hadamard, uint8_t *codes_dev, uint8_t *beta_ids_dev,
                     float *norms_dev, void *decoded_bf16_dev, void *stream);

/*
 * One launch for everything between two Linear layers of a Llama block and the packed
 * activation the next Linear consumes: an element-wise stage on BF16 rows [rows, n], then
 * (when codes_dev is given) the rotate + norm + encode + pack of nq_quantize_rows.
 *   mode 1  h = x + residual (residual_dev may be NULL: h = x); residual_out_dev (optional)
 *           receives h; y = norm_weight * bf16(h * rsqrt(mean(h^2) + eps))  -- the residual
 *           add and LlamaRMSNorm in front of q/k/v_proj and gate/up_proj
 *   mode 2  y = bf16(silu(gate)) * x  -- the SwiGLU product in front of down_proj
 * Every tensor-level result is rounded to BF16 as the BF16 tensor operations it replaces do.
 * staged_out_dev (optional) receives y as BF16 [rows, n].  With codes_dev == NULL only the
 * element-wise stage runs (the final norm in front of the LM head).
 * Replaces (decode step): the residual adds, LlamaRMSNorm / SiLU-and-multiply tensor
 * operations of the model code and the input stage of FusedNQRTLinear.forward,
 * nestquant/models/fused_linear.py:287-306.
 */
int nq_fused_input_stage(const void *x_dev, int64_t rows, int64_t n, int mode,
                         const void *residual_dev, void *residual_out_dev,
                         const void *norm_weight_dev, float eps, const void *gate_dev,
                         void *staged_out_dev, int q, const float *betas_dev, int beta_count,
                         int hadamard, uint8_t *codes_dev, uint8_t *beta_ids_dev, float *norms_dev,
                         void *decoded_bf16_dev, void *stream);

/*
 * Normalized Sylvester-Hadamard transform of `rows` rows of power-of-two length n, with the
 * reference's butterfly order (widths 1, 2, 4, ...), every sum and difference rounded to
 * stage_dtype (NQ_F32 = no intermediate rounding) and a final multiplication by
 * float32(1 / sqrt(n)); the result is written as out_dtype.
 * Replaces: hadamard(), nestquant/core/rotation.py:12-27, as used on Linear inputs
 * (nestquant/models/fused_linear.py:287-290, in the input dtype) and on post-RoPE queries
 * and keys (nestquant/runtime/nqkv_batched_hf_backend.py:381, 549, in float32).
 */
int nq_hadamard(const void *x_dev, int x_dtype, int64_t rows, int64_t n, int stage_dtype,
                void *out_dev, int out_dtype, void *stream);

/*
 * Rotary position embedding and Hadamard rotation of BF16 head vectors x [rows, heads, head_dim]
 * in one launch (prefill queries and keys).  rope_cos_dev / rope_sin_dev (optional, both or
 * neither): BF16 [rows, head_dim]; (x * cos) + (rotate_half(x) * sin) in BF16 tensor arithmetic
 * (every product and the sum rounded to BF16), as nq_nqkv_write applies it.  hadamard != 0 then
 * applies the normalized Hadamard transform over head_dim with float32 butterflies, rounded to
 * BF16 once.  head_dim is 64 or 128.
 * Replaces: apply_rotary_pos_emb (transformers' Llama) followed by
 * hadamard(x.float()).to(bfloat16), nestquant/runtime/nqkv_batched_hf_backend.py:381, 549.
 */
int nq_rope_hadamard(const void *x_dev, int64_t rows, int heads, int head_dim, const void *rope_cos_dev,
                     const void *rope_sin_dev, int hadamard, void *out_dev, void *stream);

/*
 * nq_rope_hadamard for the queries [rows, query_heads, head_dim] and the keys [rows, key_heads,
 * head_dim] of the same rows in one launch (same tables, same arithmetic, each tensor to an output
 * of its own): a prefill applies both right after the q/k/v product.
 * Replaces: the two apply_rotary_pos_emb results and their rotations,
 * nestquant/runtime/nqkv_batched_hf_backend.py:381, 549.
 */
int nq_rope_hadamard_pair(const void *query_dev, int query_heads, void *query_out_dev, const void *key_dev,
                          int key_heads, void *key_out_dev, int64_t rows, int head_dim, const void *rope_cos_dev,
                          const void *rope_sin_dev, int hadamard, void *stream);

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
 * Resolved form of one NQRT4 weight [rows, K], made once when the weight is prepared.
 * A dithered block decodes to w = (G c - d) - 14 Q_E8((G c - d) / 14), d = u - Q_E8(u) with u
 * the hashed uniforms of the block; both lattice searches depend only on the stored code, the
 * seed and the block index.  This entry runs the exact decode and stores the lattice point
 * s = G c + Q_E8(u) - 14 Q_E8(...) of every block, so that the linear kernels compute w = s - u
 * with the hash alone (no search, no division; about a third of the vector instructions).
 *   words_dev  uint32[rows * K / 8]: the block's beta id in bits 0..1, floor(s_j) + 15 for
 *              j = 0..5 in 5-bit fields from bit 2
 *   tails_dev  uint16[rows * K / 8]: fields 6 and 7 in bits 0..9, bit 10 set when s lies in
 *              the half-integer coset
 *   out_of_range_dev  int32 counter (caller zeroes it): blocks whose s does not fit the
 *              fields; geometry bounds s_j to [-14, 16], so any count other than 0 means the
 *              streams are not a valid NQRT4 record and the resolved form must not be used
 * 6 bytes per block (6 bits per weight) against the 4.25 bits of the NQRT4 streams.
 * No counterpart in the reference (its kernels repeat both searches on every call,
 * nestquant/runtime/nqrt4_cooperative_device.cuh:150-171).
 */
int nq_w4a4_resolve_weight(const uint8_t *w_codes_dev, const uint8_t *w_beta_ids_dev, int64_t rows,
                           int64_t k, int64_t weight_offset, int64_t weight_seed,
                           uint32_t *words_dev, uint16_t *tails_dev, int32_t *out_of_range_dev,
                           void *stream);

/*
 * Packed W4A4 linear for decode, M = 1..8 tokens: y[m, n] = sum_k bf16(a[m, k]) * bf16(w[n, k]),
 * FP32 accumulation; the weight is decoded in registers from its packed stream (dither
 * regenerated; counter = weight_offset * 8 + n * K + k).
 *   act_*            NQA4 streams of [M, K] (codes M*K/2 B, beta ids M*K/32 B, norms f32[M], betas f32[4])
 *   act_decoded_dev  optional BF16 [M, K] decode of the same activation (from nq_quantize_rows);
 *                    when NULL the packed streams are decoded once into the workspace,
 *                    when given the packed streams may be NULL
 *   w_*              NQRT4 streams of [N, K] (codes N*K/2 B, beta ids N*K/32 B, norms f32[N], betas f32[4])
 *   w_resolved_words_dev, w_resolved_tails_dev
 *                    optional resolved form from nq_w4a4_resolve_weight; when given it is used
 *                    instead of w_codes_dev / w_beta_ids_dev, which may then be NULL.  Results
 *                    agree with the NQRT4 path to FP32 rounding (before the BF16 rounding of
 *                    the weight), not bit for bit
 *   out_dev          [M, N] of out_dtype (NQ_F32 or NQ_BF16)
 *   split_k          1, 2, 4 or 8 slices of K reduced in ascending order (deterministic); 0 lets
 *                    the library choose
 *   workspace_dev    at least nq_w4a4_gemv_workspace_bytes() bytes, 16-byte aligned (may be
 *                    NULL when that is 0)
 * Requires q = 14, K % 32 == 0, (K / split_k) % 32 == 0, 1 <= M <= 8.  With resolved weights
 * (16-byte aligned words, 8-byte aligned tails), K % 128 == 0 and split_k 0 or 1, M up to 16: above
 * eight rows, from two rows on, and for any row count when N fills 512 tiles of 16 channels,
 * the products run on the matrix cores (v_mfma_f32_16x16x32_bf16 fed from registers), still one
 * decode per block.
 * Replaces: run_m1 / run_m1_splitk_probe / run_small_m / run_small_m_splitk_probe of the
 * torch extension, nestquant/runtime/nqrt4_w4a4_mma_binding.cpp:3-46, kernels
 * nestquant/runtime/nqrt4_w4a4_mma.cu:901-947, 952-1001, 411-420, 229-286.
 */
int nq_w4a4_gemv(const uint8_t *act_codes_dev, const uint8_t *act_beta_ids_dev,
                 const float *act_norms_dev, const float *act_betas_dev,
                 const void *act_decoded_dev, const uint8_t *w_codes_dev,
                 const uint8_t *w_beta_ids_dev, const uint32_t *w_resolved_words_dev,
                 const uint16_t *w_resolved_tails_dev, const float *w_norms_dev,
                 const float *w_betas_dev, int m, int k, int n, int64_t weight_offset,
                 int64_t weight_seed, int split_k, void *out_dev, int out_dtype,
                 void *workspace_dev, size_t workspace_bytes, void *stream);

size_t nq_w4a4_gemv_workspace_bytes(int m, int k, int n, int split_k, int have_decoded_activation);

/*
 * nq_w4a4_gemv without a caller workspace: the decoded activation and the split-K partial sums
 * live in a 4 MiB buffer inside the library's own device image (one copy per GPU, held until the
 * process ends), so the call allocates nothing and asks for nothing that was allocated for it.
 * Same arguments, kernels and results (bit for bit) as nq_w4a4_gemv; shapes whose workspace
 * (nq_w4a4_gemv_workspace_bytes) exceeds the buffer are rejected with NQ_ERR_WORKSPACE.  The
 * first use on a device looks up the buffer's address (hipGetSymbolAddress), which a stream
 * under capture must not see: nq_w4a4_gemv_static_init() does that lookup for the current
 * device ahead of time, and a first call made inside a capture without it is rejected with
 * NQ_ERR_ARGUMENT instead of being recorded.  All calls on one GPU share the buffer: calls that
 * may overlap there (different streams, different threads) race and must be serialised by the
 * caller.  Nothing in the buffer needs clearing between calls.
 * No counterpart in the reference (its extension allocates partials with torch::empty on every
 * call, nestquant/runtime/nqrt4_w4a4_mma.cu:1213-1214); it is for callers that cannot allocate
 * device memory: code under HIP graph capture, tight serving loops, harnesses that forbid it.
 */
int nq_w4a4_gemv_static_init(void);
int nq_w4a4_gemv_static(const uint8_t *act_codes_dev, const uint8_t *act_beta_ids_dev,
                        const float *act_norms_dev, const float *act_betas_dev,
                        const void *act_decoded_dev, const uint8_t *w_codes_dev,
                        const uint8_t *w_beta_ids_dev, const uint32_t *w_resolved_words_dev,
                        const uint16_t *w_resolved_tails_dev, const float *w_norms_dev,
                        const float *w_betas_dev, int m, int k, int n, int64_t weight_offset,
                        int64_t weight_seed, int split_k, void *out_dev, int out_dtype, void *stream);

/*
 * nq_w4a4_gemv for `count` (1..4) weights that share one activation (q/k/v_proj, gate/up_proj)
 * in a single launch.  Every array argument is a host array of `count` entries; weights are
 * given in resolved form (nq_w4a4_resolve_weight) and the activation as its decoded BF16
 * [M, K] rows; out_dev[i] receives [M, n[i]] of out_dtype.  No split-K, no workspace.
 * Results equal those of `count` nq_w4a4_gemv calls with split_k = 1 bit for bit.
 * No counterpart in the reference, which launches once per projection
 * (nestquant/models/fused_linear.py:316-407).
 */
int nq_w4a4_gemv_grouped(const void *act_decoded_dev, int count, const uint32_t *const *w_resolved_words_dev,
                         const uint16_t *const *w_resolved_tails_dev, const float *const *w_norms_dev,
                         const float *const *w_betas_dev, const int *n, const int64_t *weight_offsets,
                         const int64_t *weight_seeds, void *const *out_dev, int m, int k, int out_dtype,
                         void *stream);

/*
 * Packed W4A4 linear for prefill, any M >= 1 (meant for M >= 9): same product and same
 * arguments as nq_w4a4_gemv, computed on the matrix cores (v_mfma_f32_32x32x16_bf16).  The
 * weight tile is decoded once per call into double-buffered LDS as MFMA B fragments; ragged
 * M is padded to a multiple of 32 with zero rows inside the kernel and M above 512 is
 * processed in chunks of 512 rows.  split_k in {0 (library picks), 1, 2, 4, 8, 16}.
 * From 257 rows on, with split_k = 0 and BF16 output, the weight is instead decoded once into a
 * BF16 scratch [N, K] inside the workspace (nq_w4a4_decode_weight) and multiplied by
 * nq_bf16_gemm; nq_w4a4_gemm_workspace_bytes includes that scratch.
 * Requires q = 14, K % 128 == 0, (K / split_k) % 128 == 0.
 * Replaces: run_m16 / run_large_m_staged of the torch extension
 * (nestquant/runtime/nqrt4_w4a4_mma_binding.cpp:3-46, kernels
 * nestquant/runtime/nqrt4_w4a4_mma.cu:124-171, 606-667) and the Python chunk-and-pad wrapper
 * linear_packed_w4a4_mma_chunked_staged (nestquant/runtime/cuda_w4a4_mma.py:393-484).
 */
int nq_w4a4_gemm(const uint8_t *act_codes_dev, const uint8_t *act_beta_ids_dev,
                 const float *act_norms_dev, const float *act_betas_dev,
                 const void *act_decoded_dev, const uint8_t *w_codes_dev,
                 const uint8_t *w_beta_ids_dev, const uint32_t *w_resolved_words_dev,
                 const uint16_t *w_resolved_tails_dev, const float *w_norms_dev,
                 const float *w_betas_dev, int m, int k, int n, int64_t weight_offset,
                 int64_t weight_seed, int split_k, void *out_dev, int out_dtype,
                 void *workspace_dev, size_t workspace_bytes, void *stream);

size_t nq_w4a4_gemm_workspace_bytes(int m, int k, int n, int split_k, int have_decoded_activation);

/*
 * nq_w4a4_gemm for up to four weights that share one activation (q, k and v; gate and up) of at
 * most 512 rows, in one launch: decoded BF16 activation [M, K], resolved weights, every N[i] a
 * positive multiple of 32, BF16 outputs [M, N[i]] of their own.  The K split follows the sum of the
 * N[i]; with a split the partial sums wait in the workspace (nq_w4a4_gemm_grouped_workspace_bytes
 * for M, K and the sum of N) and one more launch adds them in slab order.  Same values as one
 * nq_w4a4_gemm per weight with that split.
 * Replaces: the three (two) calls of run_large_m_staged a prefill makes for one input
 * (nestquant/models/fused_linear.py:316-407, nestquant/runtime/nqrt4_w4a4_mma.cu:606-667).
 */
int nq_w4a4_gemm_grouped(const void *act_decoded_dev, int count, const uint32_t *const *w_resolved_words_dev,
                         const uint16_t *const *w_resolved_tails_dev, const float *const *w_norms_dev,
                         const float *const *w_betas_dev, const int *n, const int64_t *weight_offsets,
                         const int64_t *weight_seeds, void *const *out_bf16_dev, int m, int k,
                         void *workspace_dev, size_t workspace_bytes, void *stream);

size_t nq_w4a4_gemm_grouped_workspace_bytes(int m, int k, int n_total);

/*
 * The BF16 weight [N, K] that nq_w4a4_gemv / nq_w4a4_gemm multiply by, written out:
 * bf16(decode * beta * (norm / sqrt(K))) per element, from the resolved form when given, else
 * from the NQRT4 streams.  For prefills long enough that decoding the weight once and running
 * a plain BF16 GEMM (a library's) beats decoding it inside the multiply; the scratch is the
 * caller's and lives only for that call.
 * Replaces: PackedNestQuantTensor.dequantize_chunked(output_dtype=bfloat16),
 * nestquant/core/tensor_checkpoint.py:285-330 (up to the scale's rounding order, which follows
 * the linear kernels here).
 */
int nq_w4a4_decode_weight(const uint8_t *w_codes_dev, const uint8_t *w_beta_ids_dev,
                          const uint32_t *w_resolved_words_dev, const uint16_t *w_resolved_tails_dev,
                          const float *w_norms_dev, const float *w_betas_dev, int64_t n, int64_t k,
                          int64_t weight_offset, int64_t weight_seed, void *out_bf16_dev, void *stream);

/*
 * Dense BF16 GEMM on the matrix cores: c[m, n] = sum_k a[m, k] b[n, k], a [M, K] and b [N, K]
 * row-major BF16 (16-byte aligned), FP32 accumulation, c [M, N] BF16.  K a multiple of 128.
 * tile = -1 lets the library choose the workgroup tile from the shape; 0..6 force
 * 256x256, 128x256, 256x128, 128x128, 64x128, 128x64, 64x64, and 7..9 the 128x128, 64x128 and
 * 64x64 tiles on the kernel that splits its wavefronts into movers and multipliers, which the
 * library takes by itself when every compute unit gets at most one tile (for measurements).
 * A product with few tiles (a few hundred rows) is split along K into 2, 4 or 8 slabs whose
 * float32 partial results meet in a second launch: split_k = 0 lets the library decide, 1 forbids
 * it, 2 / 4 / 8 force it (K a multiple of 128 split_k).  The partial results need
 * split_k * M * N * 4 bytes of workspace (16-byte aligned); without a workspace nothing is split.
 * nq_w4a4_gemm calls it on the weight it has decoded once when M is large; it is exported for
 * callers that keep a decoded weight themselves.
 * Replaces: the multiply of run_large_m_staged for long prefills,
 * nestquant/runtime/nqrt4_w4a4_mma.cu:606-667 (which decodes inside the multiply).
 */
int nq_bf16_gemm(const void *a_bf16_dev, const void *b_bf16_dev, int64_t m, int64_t n, int64_t k,
                 void *c_bf16_dev, int tile, int split_k, void *workspace_dev, size_t workspace_bytes,
                 void *stream);

/*
 * The same product with its columns going to one to three outputs of their own: b stacks the
 * weights of linears that share the activation a (q, k and v; gate and up), output i receives the
 * next widths[i] columns as a row-major [M, widths[i]] BF16 matrix (16-byte aligned; every width
 * a multiple of 256, so that no workgroup tile straddles two outputs).  One launch instead of one
 * per linear: the narrow ones (k and v: 512 columns) no longer leave most of the chip idle.  No K
 * split.  outs_bf16_dev and widths are host arrays of `count` entries.
 * Replaces: the per-projection calls of FusedNQRTLinear.forward for projections that share their
 * input (nestquant/models/fused_linear.py:49-127, SharedPackedActivationCache) in a long prefill.
 */
int nq_bf16_gemm_split(const void *a_bf16_dev, const void *b_bf16_dev, int64_t m, int64_t k,
                       void *const *outs_bf16_dev, const int64_t *widths, int count, int tile, void *stream);

/*
 * NQKV cache, device-resident state.  Per slot (int32[slots]): sequence_lengths,
 * page_counts, last_page_lens, hot_lengths; page_indices int32[slots, max_pages] maps a
 * slot's page ordinal to a physical page; hot tails BF16 [slots, page_size, kv_heads,
 * head_dim]; the page pool is six SoA streams indexed by physical page (per page and side:
 * codes page_size*kv_heads*head_dim/2 B, beta ids .../32 B, norms f32[page_size*kv_heads]),
 * rows in NHD order, row = token * kv_heads + head.  Same tensors as the reference's
 * NQKVPagePool / BatchedNQKVMetadata / NQKVHotColdCache (nestquant/runtime/nqkv_pool.py:94-110,
 * paged_nqkv_cache.py:25-95, nqkv_hot_cache.py:14-37).
 *
 * nq_nqkv_advance: for every active batch row r with slot s = slot_ids[r] (rows with a
 * slot outside [0, slots) are ignored), add counts[r] (or uniform_count when counts is NULL)
 * to sequence_lengths[s], clamped at max_tokens, and refresh the three derived tensors.
 * Called once per step, before the layers run.  Replaces the per-layer metadata kernels
 * and host-side page reservation of nestquant/runtime/nqkv_graph_writer.py:15-80, 291-332,
 * nestquant/runtime/nqkv_graph_pack.py:18-69 and nqkv_batch_manager.py:648-707.
 */
int nq_nqkv_advance(const int32_t *slot_ids_dev, const uint8_t *active_mask_dev,
                    const int32_t *counts_dev, int uniform_count, int batch, int slots,
                    int page_size, int max_tokens, int32_t *sequence_lengths_dev,
                    int32_t *page_counts_dev, int32_t *last_page_lens_dev,
                    int32_t *hot_lengths_dev, void *stream);

/*
 * The head of a step that writes prompts (or further chunks of them) in one launch.  `record` is
 * int32 [3, batch] as the host describes the step: row r writes its first record[1][r] tokens
 * (clamped to [0, width]) into slot record[0][r]; record[2][r] != 0 says the slot starts a new
 * sequence, whose four table entries restart at zero and whose cache_active flag is set.  The
 * launch leaves the row state where nq_nqkv_write and the attention entries read it
 * (step_slot_ids, step_counts int32 [batch]; step_active uint8 [batch] = the row writes something),
 * fills positions[r, c] = tokens the slot held + c (int64 [batch, width], may be NULL) and
 * last_token[r] = count - 1 (int64 [batch], 0 for a row that writes nothing; may be NULL), and
 * advances the tables as nq_nqkv_advance does.  Rows must name distinct slots.  Replaces, for a
 * prompt step, the slot reset, the row-state copies and the metadata update of
 * nestquant/runtime/nqkv_batched_hf_backend.py:147-280 and nqkv_batch_manager.py:394-422, 245-285
 * (about twenty small launches and copies through the tensor library).
 */
int nq_prompt_step_begin(const int32_t *record_dev, int batch, int width, int slots, int page_size,
                         int max_tokens, int32_t *step_slot_ids_dev, int32_t *step_counts_dev,
                         uint8_t *step_active_dev, int32_t *sequence_lengths_dev, int32_t *page_counts_dev,
                         int32_t *last_page_lens_dev, int32_t *hot_lengths_dev, uint8_t *cache_active_dev,
                         int64_t *positions_dev, int64_t *last_token_dev, void *stream);

/*
 * The head of a decode step in one launch: nq_nqkv_advance with a count of one token per row,
 * embedded[r] = embedding[tokens[r]] (BF16 rows of `hidden` values; a token outside [0, vocab)
 * embeds as zero) and the rotary embedding's rows of positions[r] (clamped to the table):
 * rotary is BF16 [2, rotary_positions, head_dim] (cos rows, then sin rows), rotary_rows BF16
 * [2, batch, head_dim].  Replaces: embed_tokens and LlamaRotaryEmbedding at the top of the model
 * forward of a decode step (nestquant/runtime/nqkv_batched_runner.py:162-169) together with the
 * step's metadata update (nqkv_graph_writer.py:15-80).
 */
int nq_decode_step_begin(const int32_t *slot_ids_dev, const uint8_t *active_mask_dev, int batch, int slots,
                         int page_size, int max_tokens, int32_t *sequence_lengths_dev, int32_t *page_counts_dev,
                         int32_t *last_page_lens_dev, int32_t *hot_lengths_dev, const int64_t *tokens_dev,
                         const void *embedding_bf16_dev, int64_t vocab, int hidden, void *embedded_bf16_dev,
                         const int64_t *positions_dev, const void *rotary_bf16_dev, int64_t rotary_positions,
                         int head_dim, void *rotary_rows_bf16_dev, void *stream);

/*
 * Paged ragged writer for one layer.  key/value: BF16 [batch, tokens, kv_heads, head_dim];
 * row r contributes its first counts[r] tokens (uniform_count when counts is NULL) at
 * positions sequence_lengths[s] - count .. sequence_lengths[s] - 1 (lengths already advanced).
 * Rows land in the slot's hot tail; every page completed by the write is encoded (the row
 * quantiser of nq_quantize_rows, bit-identical) into physical page page_indices[s, ordinal].
 * rotate_keys != 0 first applies the normalized Hadamard transform over head_dim to the new
 * key rows (float32 butterflies, result rounded to BF16), i.e. the caller passes post-RoPE
 * keys and need not launch nq_hadamard.
 * rope_cos_dev / rope_sin_dev (optional, both or neither): BF16 [batch, tokens, head_dim]
 * rotary tables; the new key rows then arrive pre-RoPE and (k * cos) + (rotate_half(k) * sin)
 * is applied first, in BF16 tensor arithmetic (every product and the sum rounded to BF16).
 * Requires head_dim = 64, page_size = 16, q = 14, equal beta counts.
 * Replaces: append_hot_k1_graph_safe / ragged sub-page and segment writers
 * (nestquant/runtime/nqkv_graph_writer.py:263-473), launch_pack_full_hot_pages_graph_safe
 * (nestquant/runtime/nqkv_graph_pack.py:76-193) and the multi-round planner that feeds them
 * (nestquant/runtime/nqkv_segment_plan.py:61-144).
 */
int nq_nqkv_write(const void *key_dev, const void *value_dev, int kv_dtype, const int32_t *slot_ids_dev,
                  const uint8_t *active_mask_dev, const int32_t *counts_dev, int uniform_count,
                  const int32_t *sequence_lengths_dev, const int32_t *page_indices_dev,
                  uint8_t *key_codes_dev, uint8_t *key_beta_ids_dev, float *key_norms_dev,
                  uint8_t *value_codes_dev, uint8_t *value_beta_ids_dev, float *value_norms_dev,
                  const float *key_betas_dev, int key_beta_count, const float *value_betas_dev,
                  int value_beta_count, void *hot_keys_dev, void *hot_values_dev, int batch, int tokens,
                  int slots, int max_pages, int kv_heads, int head_dim, int page_size, int rotate_keys,
                  const void *rope_cos_dev, const void *rope_sin_dev, uint8_t *key_hints_dev,
                  uint8_t *value_hints_dev, void *stream);

/*
 * Decode hints: an optional seventh and eighth stream of the page pool, beside the six of the
 * reference's format (which stay bit-identical): four bits per 8-value block, two blocks per byte,
 * [pages][page_size * kv_heads * head_dim / 16] bytes for keys and for values.  A block's hint
 * records the two decisions its undithered decode takes inside Q_E8(G c / 14): bit 0 = the
 * half-integer coset wins, bits 1..3 = the coordinate that the parity correction of that coset's D8
 * search moves.  With the hints a reader decodes a block with about 140 instead of 280 vector
 * instructions and gets the same floats bit for bit (nq_nqkv_verify_hints checks every code word).
 * Writers (nq_nqkv_write, nq_nqkv_append_attention_decode) fill the hints of every page they pack when
 * given the two pointers; readers (nq_nqkv_attention_decode, nq_nqkv_append_attention_decode,
 * nq_nqkv_attention_prefill) use them when given; NULL, NULL is the path without hints.  Hints
 * must belong to the code words beside them: a pool filled by other means gets them from
 * nq_nqkv_page_hints (`blocks` code words -> blocks / 2 bytes; code stream 8-byte aligned).
 * nq_nqkv_verify_hints decodes the `count` code words from index `first` on (digits below 14; all
 * 14^8 of them are 0 .. 1475789055) with and without their hint and adds the number of blocks that
 * differ to *mismatches_dev (a self-check; the tests run it over the whole range).
 * No counterpart in the reference (its kernels search both cosets in every decode,
 * nestquant/runtime/nqkv_attention_k1.py:243-342).
 */
int nq_nqkv_page_hints(const uint8_t *codes_dev, int64_t blocks, uint8_t *hints_dev, void *stream);
int nq_nqkv_verify_hints(int64_t first, int64_t count, uint64_t *mismatches_dev, void *stream);

/*
 * Paged NQKV4 decode attention for a ragged batch: for batch row r with slot s (clamped to
 * range; the row is live iff active_mask[r] and, when given, cache_active[s]) and query
 * head h (KV head h / (q_heads / kv_heads)), softmax(q . K^T * scale) . V over the slot's
 * page_counts[s] cold pages (all full except the last, which holds last_page_lens[s]
 * tokens), decoded on the fly, followed by its hot_lengths[s] BF16 hot rows.  FP32
 * online-softmax in two stages; rows that are not live or have no tokens give zeros.
 * query / out: [batch, q_heads, head_dim] of query_dtype; rotate_query != 0 applies the
 * normalized Hadamard transform over head_dim to the query first (float32, rounded to
 * query_dtype), matching keys stored with rotate_keys.  out_dev may be NULL: then only the first
 * stage runs (see nq_attention_output_stage).  rope_cos_dev / rope_sin_dev (optional,
 * both or neither): BF16 [batch, head_dim] rotary tables applied to the (BF16) query before
 * that, as nq_nqkv_write applies them to keys.  Alignment: a BF16 query 16 bytes (its rows are
 * read eight values at a time; a sliced view must be made contiguous first), float32 4, float16
 * and the rotary rows 2, hot tails 16, page streams 4; anything else returns NQ_ERR_ARGUMENT.
 * Workspace: at least
 * nq_nqkv_attention_workspace_bytes() bytes.  Requires head_dim = 64, page_size = 16,
 * q = 14, q_heads / kv_heads in {1, 2, 4, 8}; any max_pages.
 * Replaces: nqkv_decode_attention_batched_k1 and its three Triton kernels
 * (nestquant/runtime/nqkv_attention_k1.py:763-942, 243-471); oracle
 * nestquant/runtime/nqkv_attention.py:14-86.
 */
int nq_nqkv_attention_decode(
    const void *query_dev, int query_dtype, const uint8_t *key_codes_dev, const uint8_t *key_beta_ids_dev,
    const float *key_norms_dev, const uint8_t *value_codes_dev, const uint8_t *value_beta_ids_dev,
    const float *value_norms_dev, const float *key_betas_dev, const float *value_betas_dev,
    const int32_t *page_indices_dev, const int32_t *page_counts_dev, const int32_t *last_page_lens_dev,
    const int32_t *hot_lengths_dev, const uint8_t *cache_active_dev, const void *hot_keys_dev,
    const void *hot_values_dev, const int32_t *slot_ids_dev, const uint8_t *active_mask_dev, int batch,
    int slots, int max_pages, int q_heads, int kv_heads, int head_dim, int page_size, float scale,
    int rotate_query, const void *rope_cos_dev, const void *rope_sin_dev, void *out_dev, void *workspace_dev,
    size_t workspace_bytes, const uint8_t *key_hints_dev, const uint8_t *value_hints_dev, void *stream);

size_t nq_nqkv_attention_workspace_bytes(int batch, int q_heads, int head_dim, int max_pages);

/*
 * One decode step's KV append and attention of a layer in one launch: what nq_nqkv_write (one
 * new BF16 token per row, uniform count 1) followed by nq_nqkv_attention_decode computes, for
 * tables nq_nqkv_advance / nq_decode_step_begin have already advanced by this token.  The
 * workgroup that attends over a row's hot tail takes the row's new key and value
 * [batch, kv_heads, head_dim] as the projections left them, applies the rotary tables (the
 * same BF16 [batch, head_dim] rows serve the query and the key: they share the position) and,
 * with rotate != 0, the Hadamard rotation to both, and appends the pair to the slot's hot tail;
 * a token that completes a page is encoded with the page (codes, beta ids and norms bit-equal
 * to nq_nqkv_write's) into page_indices[slot, (length - 1) / page_size], and this launch
 * attends over that page through the codes it has just made.  Rows write under
 * nq_nqkv_write's conditions (active, slot in range, length > 0) whether or not cache_active
 * lets them attend.  The attention output equals the two-call form but for the order in which
 * the completed page's part is merged (float32 rounding).  out_dev may be NULL as for
 * nq_nqkv_attention_decode.  BF16 only; same shape limits as the two calls it replaces.
 * Replaces: append_hot_k1_graph_safe + launch_pack_full_hot_pages_graph_safe
 * (nestquant/runtime/nqkv_graph_writer.py:263-473, nqkv_graph_pack.py:76-193) followed by
 * nqkv_decode_attention_batched_k1 (nestquant/runtime/nqkv_attention_k1.py:763-942) in
 * BatchedNQKVLlamaCache's decode update (nestquant/runtime/nqkv_batched_hf_backend.py:357-631).
 */
int nq_nqkv_append_attention_decode(
    const void *query_dev, const void *key_dev, const void *value_dev, const int32_t *sequence_lengths_dev,
    uint8_t *key_codes_dev, uint8_t *key_beta_ids_dev, float *key_norms_dev, uint8_t *value_codes_dev,
    uint8_t *value_beta_ids_dev, float *value_norms_dev, const float *key_betas_dev, int key_beta_count,
    const float *value_betas_dev, int value_beta_count, const int32_t *page_indices_dev,
    const int32_t *page_counts_dev, const int32_t *last_page_lens_dev, const int32_t *hot_lengths_dev,
    const uint8_t *cache_active_dev, void *hot_keys_dev, void *hot_values_dev, const int32_t *slot_ids_dev,
    const uint8_t *active_mask_dev, int batch, int slots, int max_pages, int q_heads, int kv_heads, int head_dim,
    int page_size, float scale, int rotate, const void *rope_cos_dev, const void *rope_sin_dev, void *out_dev,
    void *workspace_dev, size_t workspace_bytes, uint8_t *key_hints_dev, uint8_t *value_hints_dev, void *stream);

/*
 * The second stage of the decode attention done where its result is consumed.  With
 * out_dev == NULL nq_nqkv_attention_decode leaves the per-chunk partial results (maxima, sums
 * and numerators of nq_nqkv_attention_parts(batch, max_pages) chunks per head) in its workspace;
 * this call merges them into the BF16 attention output [rows = batch, q_heads * head_dim]
 * (staged_out_dev, optional) and, when codes_dev is given, rotates, norms, encodes and packs
 * those rows as nq_quantize_rows does for the o_proj input.  Same stream, same batch, q_heads
 * and max_pages as the attention call.  The merged rows equal nq_nqkv_attention_decode's BF16
 * output but for the summation order of the softmax denominator (at most one BF16 step).
 * Replaces: the stage-2 kernel of nqkv_decode_attention_batched_k1
 * (nestquant/runtime/nqkv_attention_k1.py:400-471) together with the input stage of
 * FusedNQRTLinear.forward (nestquant/models/fused_linear.py:287-306) of o_proj.
 */
int nq_nqkv_attention_parts(int batch, int max_pages);
int nq_attention_output_stage(const void *workspace_dev, int64_t rows, int q_heads, int head_dim, int parts,
                              void *staged_out_dev, int q, const float *betas_dev, int beta_count,
                              int hadamard, uint8_t *codes_dev, uint8_t *beta_ids_dev, float *norms_dev,
                              void *decoded_bf16_dev, void *stream);

/*
 * A decode step's input stage and the packed linear(s) that consume its rows, in one launch: what
 * nq_fused_input_stage (mode 1: residual + RMSNorm, mode 2: SiLU(gate) * x) or
 * nq_attention_output_stage (mode 3: attention merge) with the Hadamard rotation and q = 14, or
 * nq_quantize_rows of the BF16 rows x_dev themselves (mode 0: rotated first, what
 * FusedNQRTLinear.forward does with its input; mode 4: as they are, rows that were rotated already), leaves
 * in codes / beta ids / norms / decoded BF16 rows, followed by nq_w4a4_gemv_grouped of `count`
 * (1..4) resolved weights on those rows; all outputs bit for bit those of the two calls.  The first
 * rows * slices workgroups of the grid run the encoder; the others decode their weights while the
 * encoder is still busy, wait until every encoder workgroup has set its flag word, and then
 * multiply.  rows in [1, 16], n = K in {2048, 8192}, four betas.
 *   flags_dev            nq_fused_stage_linear_flag_words(rows, n) words of device memory, 16-byte
 *                        aligned (the library keeps several copies of a launch's flags, each in a
 *                        memory channel of its own, because every consumer polls them at once; a poll
 *                        reads four words per lane), zero when
 *                        the launch starts and owned by it until the next launch on the stream that
 *                        names them as previous_flags_dev (which clears them) has finished;
 *   previous_flags_dev   the flag words of the launch before this one on the same stream (any
 *                        earlier launch that has completed), cleared here; NULL with 0 words for
 *                        none: a step of several launches hands each launch's words to the next and
 *                        the last launch's words to the first launch of the next step;
 *   status_dev           one word, device or pinned host memory: set to 1 by a workgroup whose wait
 *                        ended after spin_limit polls without all flags set; that workgroup stores no
 *                        outputs and exits, so the launch always ends.  A caller that finds it set
 *                        must not trust the outputs and should go back to the two calls;
 *   spin_limit           polls (about half a microsecond each) a consumer makes before it gives up;
 *                        0 makes a consumer give up after one look (a test of the failure path).
 * attention_workspace_dev / q_heads / parts: as for nq_attention_output_stage (mode 3 only); the
 * other encoder arguments as for nq_fused_input_stage; the weight arrays as for nq_w4a4_gemv_grouped.
 * No counterpart in the reference, which launches the input stage and the linear separately
 * (nestquant/models/fused_linear.py:287-306, 316-407).
 */
int nq_fused_stage_linear_flag_words(int64_t rows, int64_t n);
int nq_fused_stage_linear(
    const void *x_dev, int64_t rows, int64_t n, int mode, const void *residual_dev, void *residual_out_dev,
    const void *norm_weight_dev, float eps, const void *gate_dev, const void *attention_workspace_dev, int q_heads,
    int parts, void *staged_out_dev, const float *betas_dev, int beta_count, uint8_t *codes_dev, uint8_t *beta_ids_dev,
    float *norms_dev, void *decoded_bf16_dev, int count, const uint32_t *const *w_resolved_words_dev,
    const uint16_t *const *w_resolved_tails_dev, const float *const *w_norms_dev, const float *const *w_betas_dev,
    const int *w_n, const int64_t *weight_offsets, const int64_t *weight_seeds, void *const *out_dev, int out_dtype,
    uint32_t *flags_dev, uint32_t *previous_flags_dev, int previous_flag_words, uint32_t *status_dev, int spin_limit,
    void *stream);

/*
 * Causal attention of a chunk of new tokens over the packed cache (prefill, chunked prefill,
 * continuation).  Call after nq_nqkv_advance + nq_nqkv_write of the same chunk: query token t
 * of batch row r (t < counts[r], or uniform_count when counts is NULL) sits at absolute
 * position sequence_lengths[s] - count + t and attends to cache tokens 0 .. that position of
 * its slot s: cold pages decoded on the fly, then the BF16 hot tail.  Tokens past counts[r]
 * and rows that are not active give zeros.
 *   query_dev / out_dev: BF16 [batch, tokens, q_heads, head_dim]; queries already rotated the
 *   way the stored keys are.  FP32 online softmax; no workspace.
 * Requires head_dim = 64, page_size = 16, q = 14, q_heads / kv_heads in {1, 2, 4, 8}.
 * Replaces, for prompts that should not be held in BF16: the SDPA prefill over the current
 * keys and values, nestquant/runtime/nqkv_batched_hf_backend.py:569-589 (which cannot see
 * tokens already in the cache); semantics of the oracle nestquant/runtime/nqkv_attention.py:14-86
 * applied per query token with a causal prefix.
 */
int nq_nqkv_attention_prefill(
    const void *query_dev, const uint8_t *key_codes_dev, const uint8_t *key_beta_ids_dev, const float *key_norms_dev,
    const uint8_t *value_codes_dev, const uint8_t *value_beta_ids_dev, const float *value_norms_dev,
    const float *key_betas_dev, const float *value_betas_dev, const int32_t *page_indices_dev,
    const int32_t *page_counts_dev, const int32_t *last_page_lens_dev, const int32_t *hot_lengths_dev,
    const int32_t *sequence_lengths_dev, const void *hot_keys_dev, const void *hot_values_dev,
    const int32_t *slot_ids_dev, const uint8_t *active_mask_dev, const int32_t *counts_dev, int uniform_count,
    int batch, int tokens, int slots, int max_pages, int q_heads, int kv_heads, int head_dim, int page_size,
    float scale, void *out_dev, void *workspace_dev, size_t workspace_bytes, const uint8_t *key_hints_dev,
    const uint8_t *value_hints_dev, void *stream);

/*
 * Bytes of the optional workspace of nq_nqkv_attention_prefill (0 when the launch has enough
 * workgroups as it is).  Given at least this much (16-byte aligned), the call splits every slot's page
 * table into ranges that workgroups of their own attend over, and a second launch merges the
 * partial results per query vector in range order: the work of a row then spreads over the chip in
 * proportion to its context.  Without it (NULL, 0) one workgroup walks a (row, token tile, KV head)
 * from the first page to the last.  Same result up to the rounding of the merged sums.
 */
size_t nq_nqkv_attention_prefill_workspace_bytes(int batch, int tokens, int max_pages, int q_heads, int kv_heads);

/*
 * Greedy sampling inside the decode step: for every row r (all rows when active_mask_dev is NULL,
 * else those with active_mask[r] != 0) the first index of the largest of logits[r, 0..vocab)
 * (rows row_stride elements apart; NaN counts as the largest) is written to tokens_dev[r];
 * positions_dev[r] (optional) is advanced by one and, when history_dev is given, the token is
 * stored at history[cursors[r] % history_steps][r] (int64 [history_steps, rows]) and cursors[r]
 * advanced by one.  Pointing tokens_dev / positions_dev at the captured step's own input
 * tensors lets a graph be replayed many times without the host reading a token in between.
 * Workspace: nq_greedy_sample_workspace_bytes(rows) bytes, 16-byte aligned, zeroed once by the
 * caller before the first call (every call leaves it ready for the next); calls that share a
 * workspace must not overlap.
 * Replaces: GreedyHostSampler (nestquant/runtime/inference_engine.py:63-69) and the per-step
 * host read of the sampled tokens (nestquant/runtime/cuda_graph_decode.py:166-182).
 */
int nq_greedy_sample(const void *logits_dev, int logits_dtype, int rows, int64_t vocab, int64_t row_stride,
                     const uint8_t *active_mask_dev, int64_t *tokens_dev, int64_t *positions_dev,
                     int64_t *history_dev, int history_steps, int32_t *cursors_dev, void *workspace_dev,
                     size_t workspace_bytes, void *stream);

size_t nq_greedy_sample_workspace_bytes(int rows);

/*
 * out[r, j] = sum_k act[r, k] weight[j, k] for a few rows (rows in [1, 16], K 2048, 4096 or 8192)
 * of a BF16 activation [rows, K] against a BF16 weight [N, K], both dense row-major and 16-byte
 * aligned; FP32 accumulation, BF16 out [rows, N].  One stream over the weight on the matrix
 * cores: the LM head of a decode step (a library GEMM of this shape leaves a third of the memory
 * rate unused), or a packed projection whose weight nq_w4a4_decode_weight has expanded to the
 * BF16 values the packed kernels multiply by, applied to the decoded activation the encoder
 * emits.  No bias.  The grouped form splits the N rows of one concatenated weight into up to
 * three outputs (q, k, v or gate, up of one activation): group g holds group_n[g] rows and writes
 * outs_bf16_dev[g], BF16 [rows, group_n[g]]; group_n and outs_bf16_dev are host arrays.
 * Replaces: the lm_head call inside the model forward of a decode step
 * (nestquant/runtime/nqkv_batched_runner.py:162-169).
 */
int nq_bf16_rows_linear(const void *act_bf16_dev, const void *weight_bf16_dev, int rows, int64_t k, int64_t n,
                        void *out_bf16_dev, void *stream);
int nq_bf16_rows_linear_grouped(const void *act_bf16_dev, const void *weight_bf16_dev, int rows, int64_t k, int groups,
                                const int64_t *group_n, void *const *outs_bf16_dev, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* NQHIP_H */
