// Causal attention of a chunk of new tokens over the packed NQKV4 cache (prefill, chunked
// prefill, continuation of a sequence that already has cold pages).
//
// The chunk's keys and values are written to the cache first (nq_nqkv_write); then query
// token t of batch row r, at absolute position start_r + t, attends to cache tokens
// 0 .. start_r + t of its slot: cold pages decoded on the fly, then the BF16 hot tail.  No BF16
// copy of the context is ever materialised (the reference's prefill runs SDPA on the BF16
// keys and values of the current prompt only, nestquant/runtime/nqkv_batched_hf_backend.py:569-589).
//
// grid = (query tiles, batch * kv_heads), 512 lanes.  A workgroup owns 128 query vectors (the
// G query heads of one KV head for 128 / G consecutive tokens), 16 per wavefront.  Pages are
// taken two at a time, one per half of the workgroup; per page of 16 tokens:
//   * every lane decodes one E8 block of the page (128 lanes keys, 128 lanes values; the
//     exact float order of nq_e8.hip.h, as in the decode kernel) and stores it to LDS as BF16:
//     keys row-major, values transposed.  A page is decoded once per workgroup and serves
//     all 128 query vectors; its packed operands are requested one trip ahead.
//   * scores on the matrix cores, transposed: S^T[token, vector] = K . Q^T with two
//     v_mfma_f32_16x16x32_bf16 per wavefront (Q^T fragments live in registers for the whole
//     kernel).  A lane then holds 4 tokens of one query vector: causal and length masks, the
//     online softmax in FP32 (two cross-row exchanges per statistic), and its four
//     probabilities are already laid out as the B operand of the next product;
//   * output, transposed: O^T[dim, vector] += V^T . P^T over the pair's 32 tokens, four
//     v_mfma_f32_16x16x32_bf16.
// LDS tiles are double-buffered (one barrier per pair of pages).  Pages past the last position of the
// tile are never visited.
#include "nq_e8.hip.h"
#include "nq_host.h"

#include <math.h>

#include <type_traits>

namespace nq {

constexpr int kPrefillThreads = 512;

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

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// the value held by the lane whose id differs in bit 4 / bit 5
__device__ __forceinline__ float lane_xor16(float v) { return __shfl_xor(v, 16, 64); }
__device__ __forceinline__ float lane_xor32(float v) { return __shfl_xor(v, 32, 64); }

template <int D, int P, int G>
__global__ void __launch_bounds__(kPrefillThreads) attention_prefill_kernel(PrefillAttentionArgs a) {
    static_assert(D == 64 && P == 16, "lane roles assume 64-dim heads and 16-token pages");
    constexpr int kBlocks = D / 8;
    constexpr int kTileTokens = 128 / G;                 // query tokens per workgroup
    constexpr int kKeyRow = D + 8;                       // BF16 elements per key row: 144 bytes, conflict-free 16-byte reads
    __shared__ __attribute__((aligned(16))) uint16_t k_page[2][2][P][kKeyRow];   // [buffer][page of the pair][token][dim]
    // transposed: [dim][token], rows of 40 bytes, and the rows of dims 32..63 keep their two halves of
    // eight tokens swapped: the 64 lanes of a decode wavefront (8 tokens x 8 blocks) that store one
    // value each then hit 16 banks instead of 4, and the 8-byte fragment reads stay aligned
    constexpr int kValueRow = P + 4;
    __shared__ __attribute__((aligned(16))) uint16_t v_page[2][2][D][kValueRow];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // The workgroups of one (row, token tile) -- one per KV head -- read the same cache lines of every
    // page (a page keeps the blocks of all KV heads of a token side by side): they are numbered so
    // that they share an XCD, hence an L2 (index = 8 * (kv_heads * (pair / 8) + head) + pair % 8;
    // workgroups go to the eight XCDs in turn).
    const int tiles = (a.tokens + kTileTokens - 1) / kTileTokens;
    const int place = blockIdx.x >> 3, pair = (place / a.kv_heads) * 8 + (blockIdx.x & 7);
    const int g = place % a.kv_heads, tile = pair % tiles, row = pair / tiles;
    if (row >= a.batch) return;                          // padding of the last group of eight pairs
    const int vec = 16 * wave + (lane & 15);             // this lane's query vector (column of S^T and O^T)
    const int quarter = lane >> 4;                       // which 4 tokens / 4 dims of a 16-row tile the lane holds
    const int t = tile * kTileTokens + vec / G;          // token of the query vector inside the chunk
    const int head = g * G + vec % G;
    const int64_t q_at = (((int64_t)row * a.tokens + t) * a.q_heads + head) * D;

    int slot = a.slot_ids[row];
    const bool live = a.active_mask[row] && slot >= 0 && slot < a.slots;
    slot = slot < 0 ? 0 : (slot >= a.slots ? a.slots - 1 : slot);
    int count = a.counts ? a.counts[row] : a.uniform_count;
    const int length = a.sequence_lengths[slot];         // already includes this chunk
    if (count > a.tokens) count = a.tokens;
    if (count > length) count = length;
    if (!live) count = 0;
    const int start = length - count;
    const bool has_query = t < count;
    const int position = start + t;                      // attends to cache tokens 0 .. position
    const int page_count = a.page_counts[slot], last_len = a.last_page_lens[slot], hot_len = a.hot_lengths[slot];

    // last position any vector of this tile looks at (uniform over the workgroup)
    const int tile_first = tile * kTileTokens;
    const int tile_last_token = (tile_first + kTileTokens < count ? tile_first + kTileTokens : count) - 1;
    const int pages_needed = tile_last_token >= tile_first ? (start + tile_last_token) / P + 1 : 0;

    // Q^T fragments of the two 32-dim steps: lane (vector, quarter) holds dims 32 step + 8 quarter .. + 8
    bf16x8 q_frag[2];
#pragma unroll
    for (int step = 0; step < 2; step++) {
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (has_query) raw = *reinterpret_cast<const uint4 *>(a.query + q_at + 32 * step + 8 * quarter);
        q_frag[step] = __builtin_bit_cast(bf16x8, raw);
    }
    floatx4 o[4];                                        // O^T tiles: dims 16 tile + 4 quarter + r of this lane's vector
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    float running_max = -INFINITY, denom = 0.0f;

    // decode role: lanes 0..255 stage the first page of a pair, 256..511 the second; of each
    // half, 128 lanes take keys and 128 values; (token, block) of the page
    const int dec_half = tid >> 8;
    const bool decodes_values = (tid & 255) >= 128;
    const int dec_token = (tid & 127) >> 3, dec_blk = tid & 7;
    const int row_in_page = dec_token * a.kv_heads + g;
    const uint32_t page_words = (uint32_t)(P * a.kv_heads * kBlocks), page_rows = (uint32_t)(P * a.kv_heads);
    const uint32_t lane_word = (uint32_t)(row_in_page * kBlocks + dec_blk);
    const uint32_t *side_codes = decodes_values ? a.value_codes : a.key_codes;
    const uint8_t *side_ids = decodes_values ? a.value_beta_ids : a.key_beta_ids;
    const float *side_norms = decodes_values ? a.value_norms : a.key_norms;
    const float *side_betas = decodes_values ? a.value_betas : a.key_betas;
    const uint16_t *side_hot = (decodes_values ? a.hot_values : a.hot_keys) +
                               (((int64_t)slot * P + dec_token) * a.kv_heads + g) * D + dec_blk * 8;
    const float beta_table[4] = {side_betas[0], side_betas[1], side_betas[2], side_betas[3]};
    const float sqrt_d = __builtin_sqrtf((float)D);
    const int32_t *slot_pages = a.page_indices + (int64_t)slot * a.max_pages;

    struct ColdOperands { uint32_t code, ids; float norm; };
    auto request_cold = [&](int ordinal) {               // operands of this lane's block of a full cold page
        const uint32_t page = (uint32_t)slot_pages[ordinal];
        const uint32_t word = page * page_words + lane_word;
        return ColdOperands{side_codes[word], (uint32_t)side_ids[word >> 2], side_norms[page * page_rows + (uint32_t)row_in_page]};
    };
    auto decode_cold = [&](const ColdOperands &operands) {
        float v[8];
        decode_codeword<false>(operands.code, 14.0f, 0u, v);
        const float beta = beta_table[(operands.ids >> (2 * (dec_blk & 3))) & 3];
        const float back = operands.norm / sqrt_d;
        const bf16x2 h0 = pack_bf16x2((v[0] * beta) * back, (v[1] * beta) * back);
        const bf16x2 h1 = pack_bf16x2((v[2] * beta) * back, (v[3] * beta) * back);
        const bf16x2 h2 = pack_bf16x2((v[4] * beta) * back, (v[5] * beta) * back);
        const bf16x2 h3 = pack_bf16x2((v[6] * beta) * back, (v[7] * beta) * back);
        return make_uint4(__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1),
                          __builtin_bit_cast(uint32_t, h2), __builtin_bit_cast(uint32_t, h3));
    };
    auto write_page = [&](int buf, int half, const uint4 packed) {
        if (decodes_values) {
            const uint32_t w[4] = {packed.x, packed.y, packed.z, packed.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v_page[buf][half][dec_blk * 8 + 2 * j][dec_token ^ (8 * (dec_blk >> 2))] = (uint16_t)(w[j] & 0xffffu);
                v_page[buf][half][dec_blk * 8 + 2 * j + 1][dec_token ^ (8 * (dec_blk >> 2))] = (uint16_t)(w[j] >> 16);
            }
        } else {
            *reinterpret_cast<uint4 *>(&k_page[buf][half][dec_token][dec_blk * 8]) = packed;
        }
    };
    auto tokens_of = [&](int ordinal) {
        if (ordinal >= pages_needed) return 0;
        if (ordinal < page_count) return ordinal < page_count - 1 ? P : last_len;
        return ordinal == page_count ? hot_len : 0;
    };
    // scores, online softmax and output update for the two staged pages of buffer `buf`;
    // kMasked = false when all 32 tokens exist and are visible to every vector of the tile
    auto attend = [&](auto masked, int buf, int first) {
        constexpr bool kMasked = decltype(masked)::value;
        float s[8], trip_max = -INFINITY;
#pragma unroll
        for (int half = 0; half < 2; half++) {
            floatx4 st = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int step = 0; step < 2; step++) {
                const bf16x8 k_frag = __builtin_bit_cast(
                    bf16x8, *reinterpret_cast<const uint4 *>(&k_page[buf][half][lane & 15][32 * step + 8 * quarter]));
                st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_frag, q_frag[step], st, 0, 0, 0);
            }
            const int tokens_here = kMasked ? tokens_of(first + half) : P;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int tok = 4 * quarter + r;
                const bool visible = !kMasked || (has_query && tok < tokens_here && (first + half) * P + tok <= position);
                s[4 * half + r] = visible ? st[r] * a.scale : -INFINITY;
                trip_max = fmaxf(trip_max, s[4 * half + r]);
            }
        }
        trip_max = fmaxf(trip_max, lane_xor16(trip_max));
        trip_max = fmaxf(trip_max, lane_xor32(trip_max));
        const float new_max = fmaxf(running_max, trip_max);
        // a vector that has seen nothing yet keeps max = -inf: exponents are forced to zero weight
        const float keep = (kMasked && new_max == -INFINITY) ? 1.0f : __expf(running_max - new_max);
        float p[8], trip_sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 8; r++) {
            p[r] = (kMasked && s[r] == -INFINITY) ? 0.0f : __expf(s[r] - new_max);
            trip_sum = trip_sum + p[r];
        }
        trip_sum = trip_sum + lane_xor16(trip_sum);
        trip_sum = trip_sum + lane_xor32(trip_sum);
        denom = denom * keep + trip_sum;
        running_max = new_max;
        // B operand of the 32-deep product: slots 0..3 = this lane's tokens of the first page, 4..7 of the second
        const uint4 p_bits = make_uint4(__builtin_bit_cast(uint32_t, pack_bf16x2(p[0], p[1])),
                                        __builtin_bit_cast(uint32_t, pack_bf16x2(p[2], p[3])),
                                        __builtin_bit_cast(uint32_t, pack_bf16x2(p[4], p[5])),
                                        __builtin_bit_cast(uint32_t, pack_bf16x2(p[6], p[7])));
        const bf16x8 p_frag = __builtin_bit_cast(bf16x8, p_bits);
#pragma unroll
        for (int tile = 0; tile < 4; tile++) {
            const int column = (4 * quarter) ^ (8 * (tile >> 1));
            const uint2 v0 = *reinterpret_cast<const uint2 *>(&v_page[buf][0][16 * tile + (lane & 15)][column]);
            const uint2 v1 = *reinterpret_cast<const uint2 *>(&v_page[buf][1][16 * tile + (lane & 15)][column]);
#pragma unroll
            for (int r = 0; r < 4; r++) o[tile][r] = o[tile][r] * keep;
            o[tile] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, make_uint4(v0.x, v0.y, v1.x, v1.y)),
                                                             p_frag, o[tile], 0, 0, 0);
        }
    };

    // Leading trips whose 32 tokens are full cold pages visible to the whole tile: no masks, operands
    // requested one trip ahead.  The rest (causal edge, partial page, hot tail) takes the masked path.
    const int visible_pages = (start + tile_first + 1) / P;
    const int full_cold_pages = page_count > 0 ? page_count - (last_len == P ? 0 : 1) : 0;
    int fast_pages = visible_pages < full_cold_pages ? visible_pages : full_cold_pages;
    if (fast_pages > pages_needed) fast_pages = pages_needed;
    if (tile_first >= count || fast_pages < 0) fast_pages = 0;
    fast_pages &= ~1;
    int trip = 0;
    if (fast_pages > 0) {
        ColdOperands next = request_cold(dec_half);
        for (int first = 0; first < fast_pages; first += 2, trip++) {
            const ColdOperands now = next;
            if (first + 2 < fast_pages) next = request_cold(first + 2 + dec_half);
            write_page(trip & 1, dec_half, decode_cold(now));
            __syncthreads();     // pages staged; also orders the reads of this buffer two trips ago before these writes
            attend(std::false_type{}, trip & 1, first);
        }
    }
    for (int first = fast_pages; first < pages_needed; first += 2, trip++) {
        {
            const int ordinal = first + dec_half;
            uint4 packed = make_uint4(0, 0, 0, 0);
            if (dec_token < tokens_of(ordinal)) {
                if (ordinal < page_count) packed = decode_cold(request_cold(ordinal));
                else packed = *reinterpret_cast<const uint4 *>(side_hot);
            }
            write_page(trip & 1, dec_half, packed);
        }
        __syncthreads();
        attend(std::true_type{}, trip & 1, first);
    }
    if (t < a.tokens) {
        const float inv = (has_query && denom > 0.0f) ? 1.0f / denom : 0.0f;   // padding tokens and inactive rows give zeros
#pragma unroll
        for (int tile = 0; tile < 4; tile++) {
            const uint32_t lo = (uint32_t)f32_to_bf16(o[tile][0] * inv) | ((uint32_t)f32_to_bf16(o[tile][1] * inv) << 16);
            const uint32_t hi = (uint32_t)f32_to_bf16(o[tile][2] * inv) | ((uint32_t)f32_to_bf16(o[tile][3] * inv) << 16);
            *reinterpret_cast<uint2 *>(a.out + q_at + 16 * tile + 4 * quarter) = make_uint2(lo, hi);
        }
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
    NQ_REQUIRE(nq::aligned(query_dev, 16) && nq::aligned(out_dev, 8) && nq::aligned(key_codes_dev, 4) &&
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
    const int tile_tokens = 128 / group;
    const int64_t pairs = (int64_t)((tokens + tile_tokens - 1) / tile_tokens) * batch;     // (row, token tile), padded to eights
    const dim3 grid((unsigned)((pairs + 7) / 8 * 8 * kv_heads));
    hipStream_t s = (hipStream_t)stream;
    switch (group) {
        case 1: hipLaunchKernelGGL((nq::attention_prefill_kernel<64, 16, 1>), grid, dim3(nq::kPrefillThreads), 0, s, a); break;
        case 2: hipLaunchKernelGGL((nq::attention_prefill_kernel<64, 16, 2>), grid, dim3(nq::kPrefillThreads), 0, s, a); break;
        case 4: hipLaunchKernelGGL((nq::attention_prefill_kernel<64, 16, 4>), grid, dim3(nq::kPrefillThreads), 0, s, a); break;
        default: hipLaunchKernelGGL((nq::attention_prefill_kernel<64, 16, 8>), grid, dim3(nq::kPrefillThreads), 0, s, a); break;
    }
    return nq::check_launch("nq_nqkv_attention_prefill");
}
