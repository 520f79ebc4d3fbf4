// Causal attention of a chunk of new tokens over the packed NQKV4 cache (prefill, chunked
// prefill, continuation of a sequence that already has cold pages).
//
// The chunk's keys and values are written to the cache first (nq_nqkv_write); then query
// token t of batch row r, at absolute position start_r + t, attends to cache tokens
// 0 .. start_r + t of its slot: cold pages decoded on the fly, then the BF16 hot tail.  No BF16
// copy of the context is ever materialised (the reference's prefill runs SDPA on the BF16
// keys and values of the current prompt only, nestquant/runtime/nqkv_batched_hf_backend.py:569-589).
//
// grid = (query tiles, batch * kv_heads), 256 lanes.  A workgroup owns 64 query vectors: the
// G query heads of one KV head for 64 / G consecutive tokens.  Lane (v, part) = (tid / 4,
// tid % 4) holds query vector v's dims 16 part .. + 16, its running max / denominator and
// 16 output dims.  Per page of 16 tokens:
//   * every lane decodes one E8 block of the page (lanes 0..127 keys, 128..255 values; the
//     exact float order of nq_e8.hip.h, as in the decode kernel) into LDS as float32: a page
//     is decoded once per workgroup and serves all 64 query vectors;
//   * scores: 16 partial dot products per lane, summed over the 4 lanes of a vector with two
//     register exchanges; causal and length masks; online softmax in FP32;
//   * output: 16 x 16 multiply-adds per lane from the value page in LDS.
// Pages past the last position of the tile are never visited.
#include "nq_e8.hip.h"
#include "nq_host.h"

#include <math.h>

namespace nq {

constexpr int kPrefillThreads = 256;

struct PrefillAttentionArgs {
    const uint16_t *query;             // BF16 [batch, tokens, q_heads, D], already rotated like the stored keys
    uint16_t *out;                     // BF16 [batch, tokens, q_heads, D]
    const uint32_t *key_codes, *value_codes;
    const uint8_t *key_beta_ids, *value_beta_ids;
    const float *key_norms, *value_norms, *key_betas, *value_betas;
    const int32_t *page_indices, *page_counts, *last_page_lens, *hot_lengths, *sequence_lengths;
    const uint16_t *hot_keys, *hot_values;
    const int32_t *slot_ids, *counts;  // counts may be null (uniform_count)
    const uint8_t *active_mask;
    int batch, tokens, uniform_count, slots, max_pages, q_heads, kv_heads;
    float scale;
};

__device__ __forceinline__ float quad_sum(float v) {
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    return v;
}

template <int D, int P, int G>
__global__ void __launch_bounds__(kPrefillThreads) attention_prefill_kernel(PrefillAttentionArgs a) {
    static_assert(D == 64 && P == 16, "lane roles assume 64-dim heads and 16-token pages");
    constexpr int kBlocks = D / 8;
    constexpr int kTileTokens = 64 / G;                  // query tokens per workgroup
    __shared__ float k_page[P][D + 4], v_page[P][D + 4];  // padded rows: the 4 parts of a vector hit distinct banks

    const int tid = threadIdx.x;
    const int row = blockIdx.y / a.kv_heads, g = blockIdx.y % a.kv_heads;
    const int vec = tid >> 2, part = tid & 3;
    const int t = blockIdx.x * kTileTokens + vec / G;    // token of this lane's query vector inside the chunk
    const int head = g * G + vec % G;
    const int64_t q_at = (((int64_t)row * a.tokens + t) * a.q_heads + head) * D + 16 * part;

    int slot = a.slot_ids[row];
    const bool live = a.active_mask[row] && slot >= 0 && slot < a.slots;
    slot = slot < 0 ? 0 : (slot >= a.slots ? a.slots - 1 : slot);
    int count = a.counts ? a.counts[row] : a.uniform_count;
    const int length = a.sequence_lengths[slot];         // already includes this chunk
    if (count > a.tokens) count = a.tokens;
    if (count > length) count = length;
    if (!live) count = 0;
    const int start = length - count;
    const bool has_query = t < count && t < a.tokens;
    const int position = start + t;                      // attends to cache tokens 0 .. position
    const int page_count = a.page_counts[slot], last_len = a.last_page_lens[slot], hot_len = a.hot_lengths[slot];

    // last position any vector of this tile looks at (uniform over the workgroup)
    const int tile_first = blockIdx.x * kTileTokens;
    const int tile_last_token = (tile_first + kTileTokens < count ? tile_first + kTileTokens : count) - 1;
    const int pages_needed = tile_last_token >= tile_first ? (start + tile_last_token) / P + 1 : 0;

    float q[16], o[16];
#pragma unroll
    for (int j = 0; j < 16; j++) { q[j] = 0.0f; o[j] = 0.0f; }
    if (has_query) {
        const uint4 lo = *reinterpret_cast<const uint4 *>(a.query + q_at), hi = *reinterpret_cast<const uint4 *>(a.query + q_at + 8);
        const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
        for (int j = 0; j < 8; j++) {
            q[2 * j] = __uint_as_float(w[j] << 16) * a.scale;
            q[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u) * a.scale;
        }
    }
    float running_max = -INFINITY, denom = 0.0f;

    // decode role: lanes 0..127 keys, 128..255 values; (token, block) of the page
    const bool decodes_values = tid >= 128;
    const int dec_token = (tid & 127) >> 3, dec_blk = tid & 7;
    const int row_in_page = dec_token * a.kv_heads + g;
    const int64_t page_words = (int64_t)P * a.kv_heads * kBlocks, page_rows = (int64_t)P * a.kv_heads;
    const float sqrt_d = __builtin_sqrtf((float)D);

    for (int ordinal = 0; ordinal < pages_needed; ordinal++) {
        // ---- stage the page ---------------------------------------------------------------------
        float staged[8];
#pragma unroll
        for (int j = 0; j < 8; j++) staged[j] = 0.0f;
        const bool cold = ordinal < page_count;
        const int tokens_here = cold ? (ordinal < page_count - 1 ? P : last_len) : (ordinal == page_count ? hot_len : 0);
        if (dec_token < tokens_here) {
            if (cold) {
                const int64_t page = a.page_indices[(int64_t)slot * a.max_pages + ordinal];
                const int64_t word = page * page_words + (int64_t)row_in_page * kBlocks + dec_blk;
                const uint32_t code = decodes_values ? a.value_codes[word] : a.key_codes[word];
                const uint32_t ids = decodes_values ? a.value_beta_ids[word >> 2] : a.key_beta_ids[word >> 2];
                const float norm = decodes_values ? a.value_norms[page * page_rows + row_in_page]
                                                  : a.key_norms[page * page_rows + row_in_page];
                decode_codeword<false>(code, 14.0f, 0u, staged);
                const float beta = (decodes_values ? a.value_betas : a.key_betas)[(ids >> (2 * (dec_blk & 3))) & 3];
                const float back = norm / sqrt_d;
#pragma unroll
                for (int j = 0; j < 8; j++) staged[j] = (staged[j] * beta) * back;
            } else {
                const uint16_t *hot = decodes_values ? a.hot_values : a.hot_keys;
                const uint4 raw = *reinterpret_cast<const uint4 *>(
                    hot + (((int64_t)slot * P + dec_token) * a.kv_heads + g) * D + dec_blk * 8);
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    staged[2 * j] = __uint_as_float(w[j] << 16);
                    staged[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
                }
            }
        }
        __syncthreads();                                 // the previous page has been consumed
        {
            float *dst = decodes_values ? &v_page[dec_token][dec_blk * 8] : &k_page[dec_token][dec_blk * 8];
            *reinterpret_cast<float4 *>(dst) = make_float4(staged[0], staged[1], staged[2], staged[3]);
            *reinterpret_cast<float4 *>(dst + 4) = make_float4(staged[4], staged[5], staged[6], staged[7]);
        }
        __syncthreads();

        // ---- scores of this vector against the 16 tokens ------------------------------------------
        float s[P];
        float page_max = -INFINITY;
#pragma unroll
        for (int tok = 0; tok < P; tok++) {
            const float *k = &k_page[tok][16 * part];
            float partial = 0.0f;
#pragma unroll
            for (int j = 0; j < 16; j += 4) {
                const float4 kv = *reinterpret_cast<const float4 *>(k + j);
                partial = __builtin_fmaf(q[j], kv.x, partial);
                partial = __builtin_fmaf(q[j + 1], kv.y, partial);
                partial = __builtin_fmaf(q[j + 2], kv.z, partial);
                partial = __builtin_fmaf(q[j + 3], kv.w, partial);
            }
            const float total = quad_sum(partial);
            const int index = ordinal * P + tok;
            const bool visible = has_query && tok < tokens_here && index <= position;
            s[tok] = visible ? total : -INFINITY;
            page_max = fmaxf(page_max, s[tok]);
        }
        if (page_max > -INFINITY) {                      // divergent per vector, no barrier inside
            const float new_max = fmaxf(running_max, page_max);
            const float keep = __expf(running_max - new_max);        // exp(-inf) = 0 on the first visible page
            denom = denom * keep;
#pragma unroll
            for (int j = 0; j < 16; j++) o[j] = o[j] * keep;
#pragma unroll
            for (int tok = 0; tok < P; tok++) {
                const float p = s[tok] == -INFINITY ? 0.0f : __expf(s[tok] - new_max);
                denom = denom + p;
                const float *v = &v_page[tok][16 * part];
#pragma unroll
                for (int j = 0; j < 16; j += 4) {
                    const float4 vv = *reinterpret_cast<const float4 *>(v + j);
                    o[j] = __builtin_fmaf(p, vv.x, o[j]);
                    o[j + 1] = __builtin_fmaf(p, vv.y, o[j + 1]);
                    o[j + 2] = __builtin_fmaf(p, vv.z, o[j + 2]);
                    o[j + 3] = __builtin_fmaf(p, vv.w, o[j + 3]);
                }
            }
            running_max = new_max;
        }
    }
    if (t < a.tokens) {
        const float inv = denom > 0.0f ? 1.0f / denom : 0.0f;          // padding tokens and inactive rows give zeros
        uint32_t packed[8];
#pragma unroll
        for (int j = 0; j < 8; j++)
            packed[j] = (uint32_t)f32_to_bf16(o[2 * j] * inv) | ((uint32_t)f32_to_bf16(o[2 * j + 1] * inv) << 16);
        *reinterpret_cast<uint4 *>(a.out + q_at) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        *reinterpret_cast<uint4 *>(a.out + q_at + 8) = make_uint4(packed[4], packed[5], packed[6], packed[7]);
    }
}

}  // namespace nq

extern "C" int nq_nqkv_attention_prefill(
    const void *query_dev, const uint8_t *key_codes_dev, const uint8_t *key_beta_ids_dev, const float *key_norms_dev,
    const uint8_t *value_codes_dev, const uint8_t *value_beta_ids_dev, const float *value_norms_dev,
    const float *key_betas_dev, const float *value_betas_dev, const int32_t *page_indices_dev,
    const int32_t *page_counts_dev, const int32_t *last_page_lens_dev, const int32_t *hot_lengths_dev,
    const int32_t *sequence_lengths_dev, const void *hot_keys_dev, const void *hot_values_dev,
    const int32_t *slot_ids_dev, const uint8_t *active_mask_dev, const int32_t *counts_dev, int uniform_count,
    int batch, int tokens, int slots, int max_pages, int q_heads, int kv_heads, int head_dim, int page_size,
    float scale, void *out_dev, void *stream) {
    NQ_REQUIRE(batch >= 1 && tokens >= 1 && slots >= 1 && max_pages >= 1, NQ_ERR_SHAPE,
               "nq_nqkv_attention_prefill: batch, tokens, slots and max_pages must be positive");
    NQ_REQUIRE(kv_heads >= 1 && q_heads >= kv_heads && q_heads % kv_heads == 0, NQ_ERR_SHAPE,
               "nq_nqkv_attention_prefill: q_heads must be a positive multiple of kv_heads");
    const int group = q_heads / kv_heads;
    NQ_REQUIRE(group == 1 || group == 2 || group == 4 || group == 8, NQ_ERR_SHAPE,
               "nq_nqkv_attention_prefill: %d query heads per KV head (supported: 1, 2, 4, 8)", group);
    NQ_REQUIRE(head_dim == 64 && page_size == 16, NQ_ERR_SHAPE,
               "nq_nqkv_attention_prefill: built for head_dim 64 and 16-token pages (got %d, %d)", head_dim, page_size);
    NQ_REQUIRE(query_dev && key_codes_dev && key_beta_ids_dev && key_norms_dev && value_codes_dev &&
                   value_beta_ids_dev && value_norms_dev && key_betas_dev && value_betas_dev && page_indices_dev &&
                   page_counts_dev && last_page_lens_dev && hot_lengths_dev && sequence_lengths_dev && hot_keys_dev &&
                   hot_values_dev && slot_ids_dev && active_mask_dev && out_dev,
               NQ_ERR_ARGUMENT, "nq_nqkv_attention_prefill: null pointer");
    NQ_REQUIRE(nq::aligned(query_dev, 16) && nq::aligned(out_dev, 16) && nq::aligned(key_codes_dev, 4) &&
                   nq::aligned(value_codes_dev, 4) && nq::aligned(hot_keys_dev, 16) && nq::aligned(hot_values_dev, 16),
               NQ_ERR_ARGUMENT, "nq_nqkv_attention_prefill: queries, output and hot tails need 16-byte, page streams 4-byte alignment");
    NQ_REQUIRE(isfinite(scale), NQ_ERR_ARGUMENT, "nq_nqkv_attention_prefill: scale must be finite");
    NQ_REQUIRE(counts_dev || (uniform_count >= 0 && uniform_count <= tokens), NQ_ERR_ARGUMENT,
               "nq_nqkv_attention_prefill: uniform token count %d is outside [0, %d]", uniform_count, tokens);
    nq::PrefillAttentionArgs a;
    a.query = reinterpret_cast<const uint16_t *>(query_dev);
    a.out = reinterpret_cast<uint16_t *>(out_dev);
    a.key_codes = reinterpret_cast<const uint32_t *>(key_codes_dev);
    a.value_codes = reinterpret_cast<const uint32_t *>(value_codes_dev);
    a.key_beta_ids = key_beta_ids_dev; a.value_beta_ids = value_beta_ids_dev;
    a.key_norms = key_norms_dev; a.value_norms = value_norms_dev;
    a.key_betas = key_betas_dev; a.value_betas = value_betas_dev;
    a.page_indices = page_indices_dev; a.page_counts = page_counts_dev; a.last_page_lens = last_page_lens_dev;
    a.hot_lengths = hot_lengths_dev; a.sequence_lengths = sequence_lengths_dev;
    a.hot_keys = reinterpret_cast<const uint16_t *>(hot_keys_dev);
    a.hot_values = reinterpret_cast<const uint16_t *>(hot_values_dev);
    a.slot_ids = slot_ids_dev; a.counts = counts_dev; a.active_mask = active_mask_dev;
    a.batch = batch; a.tokens = tokens; a.uniform_count = uniform_count; a.slots = slots; a.max_pages = max_pages;
    a.q_heads = q_heads; a.kv_heads = kv_heads; a.scale = scale;
    const int tile_tokens = 64 / group;
    const dim3 grid((unsigned)((tokens + tile_tokens - 1) / tile_tokens), (unsigned)(batch * kv_heads));
    hipStream_t s = (hipStream_t)stream;
    switch (group) {
        case 1: hipLaunchKernelGGL((nq::attention_prefill_kernel<64, 16, 1>), grid, dim3(nq::kPrefillThreads), 0, s, a); break;
        case 2: hipLaunchKernelGGL((nq::attention_prefill_kernel<64, 16, 2>), grid, dim3(nq::kPrefillThreads), 0, s, a); break;
        case 4: hipLaunchKernelGGL((nq::attention_prefill_kernel<64, 16, 4>), grid, dim3(nq::kPrefillThreads), 0, s, a); break;
        default: hipLaunchKernelGGL((nq::attention_prefill_kernel<64, 16, 8>), grid, dim3(nq::kPrefillThreads), 0, s, a); break;
    }
    return nq::check_launch("nq_nqkv_attention_prefill");
}
