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
//     online softmax in FP32 (two register exchanges per statistic), and its four
//     probabilities are already laid out as the B operand of the next product;
//   * output, transposed: O^T[dim, vector] += V^T . P^T over the pair's 32 tokens, four
//     v_mfma_f32_16x16x32_bf16.
// LDS tiles are double-buffered (one barrier per pair of pages).  Pages past the last position of the
// tile are never visited.
//
// kSets: a lane serves kSets query vectors (vector v, v + 128, ...), so a workgroup owns kSets x 128
// of them and a decoded page serves them all: the decode is the kernel's largest cost, and the G
// heads x 128 / G tokens of one set would decode every page once per 32 tokens (G = 4).
// With a workspace the context is also split: workgroup (pair, head, s) takes pages
// [s L, (s + 1) L) of the slot's table and leaves its unnormalised outputs, maxima and denominators
// per query vector for attention_prefill_merge_kernel; a row's work then spreads over the chip in
// proportion to its context instead of running on one workgroup per (tile, head) from the first page
// to the last (batch 8, contexts 495 .. 3967, 128 new tokens: the longest row alone set the time).
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
    const uint8_t *key_hints, *value_hints;        // optional decode hints, two blocks per byte (decode_codeword_hinted)
    const float *key_norms, *value_norms, *key_betas, *value_betas;
    const int32_t *page_indices, *page_counts, *last_page_lens, *hot_lengths, *sequence_lengths;
    const uint16_t *hot_keys, *hot_values;
    const int32_t *slot_ids, *counts;  // counts may be null (uniform_count)
    const uint8_t *active_mask;
    int batch, tokens, uniform_count, slots, max_pages, q_heads, kv_heads;
    float scale;
    // split form: pages per split (even), number of splits (grid.y), partial results
    int pages_per_split, splits;
    float *part_out;                   // [batch, tokens, q_heads, splits, D] unnormalised
    float *part_stats;                 // [batch, tokens, q_heads, splits, 2]: maximum, denominator
};

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// maximum / sum over the four lanes l % 16, + 16, + 32, + 48 (the four quarters of a query vector's
// column), the same in all four: two register exchanges each (v_permlane16_swap, v_permlane32_swap
// hand a lane its own value and that of the lane 16 / 32 further on), no trip through the LDS crossbar
__device__ __forceinline__ float quarters_max(float v) {
    const int bits = __builtin_bit_cast(int, v);
    const auto by16 = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    const float half = fmaxf(__builtin_bit_cast(float, (int)by16[0]), __builtin_bit_cast(float, (int)by16[1]));
    const int half_bits = __builtin_bit_cast(int, half);
    const auto by32 = __builtin_amdgcn_permlane32_swap(half_bits, half_bits, false, false);
    return fmaxf(__builtin_bit_cast(float, (int)by32[0]), __builtin_bit_cast(float, (int)by32[1]));
}
__device__ __forceinline__ float quarters_sum(float v) {
    const int bits = __builtin_bit_cast(int, v);
    const auto by16 = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    const float half = __builtin_bit_cast(float, (int)by16[0]) + __builtin_bit_cast(float, (int)by16[1]);
    const int half_bits = __builtin_bit_cast(int, half);
    const auto by32 = __builtin_amdgcn_permlane32_swap(half_bits, half_bits, false, false);
    return __builtin_bit_cast(float, (int)by32[0]) + __builtin_bit_cast(float, (int)by32[1]);
}

template <int D, int P, int G, int kSets, bool kSplit>
__global__ void __launch_bounds__(kPrefillThreads) attention_prefill_kernel(PrefillAttentionArgs a) {
    static_assert(D == 64 && P == 16, "lane roles assume 64-dim heads and 16-token pages");
    constexpr int kBlocks = D / 8;
    constexpr int kSetTokens = 128 / G;                  // query tokens per set of 128 vectors
    constexpr int kTileTokens = kSets * kSetTokens;      // query tokens per workgroup
    constexpr int kKeyRow = D + 8;                       // BF16 elements per key row: 144 bytes, conflict-free 16-byte reads
    __shared__ __attribute__((aligned(16))) uint16_t k_page[2][2][P][kKeyRow];   // [buffer][page of the pair][token][dim]
    // What the BF16 rounding of a decoded key leaves behind, as a second BF16 value: the scores take both
    // parts (two matrix instructions instead of one).  Of the roundings on this kernel's way (keys, softmax
    // weights and values to BF16 for the matrix cores, the output to BF16) the keys' moves the result most:
    // it sits in the exponent of every weight.
    __shared__ __attribute__((aligned(16))) uint16_t k_rest[2][2][P][kKeyRow];
    // transposed: [dim][token], rows of 40 bytes, and the rows of dims 32..63 keep their two halves of
    // eight tokens swapped: the 64 lanes of a decode wavefront (8 tokens x 8 blocks) that store one
    // value each then hit 16 banks instead of 4, and the 8-byte fragment reads stay aligned
    constexpr int kValueRow = P + 4;
    __shared__ __attribute__((aligned(16))) uint16_t v_page[2][2][D][kValueRow];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // The workgroups of one (row, token tile) -- one per KV head -- read the same cache lines of every
    // page (a page keeps the blocks of all KV heads of a token side by side): they are numbered so
    // that they share an XCD, hence an L2 (index = 8 * (kv_heads * (pair / 8) + head) + pair % 8;
    // workgroups go to the eight XCDs in turn).  A row's work is its context length, and the same eight
    // pairs would meet the same XCD in every split of the context: the pairs of a group of eight move one
    // place round per split, so that a long row's splits spread over the XCDs.
    const int tiles = (a.tokens + kTileTokens - 1) / kTileTokens;
    const int place = blockIdx.x >> 3, pair = (place / a.kv_heads) * 8 + ((blockIdx.x + blockIdx.y) & 7);
    const int g = place % a.kv_heads, tile = pair % tiles, row = pair / tiles;
    if (row >= a.batch) return;                          // padding of the last group of eight pairs
    const int vec = 16 * wave + (lane & 15);             // this lane's query vector of every set (column of S^T and O^T)
    const int quarter = lane >> 4;                       // which 4 tokens / 4 dims of a 16-row tile the lane holds
    const int head = g * G + vec % G;
    int t[kSets];                                        // token of the set's query vector inside the chunk
    int64_t q_at[kSets];
#pragma unroll
    for (int i = 0; i < kSets; i++) {
        t[i] = tile * kTileTokens + i * kSetTokens + vec / G;
        q_at[i] = (((int64_t)row * a.tokens + t[i]) * a.q_heads + head) * D;
    }

    int slot = a.slot_ids[row];
    const bool live = a.active_mask[row] && slot >= 0 && slot < a.slots;
    slot = slot < 0 ? 0 : (slot >= a.slots ? a.slots - 1 : slot);
    int count = a.counts ? a.counts[row] : a.uniform_count;
    const int length = a.sequence_lengths[slot];         // already includes this chunk
    if (count > a.tokens) count = a.tokens;
    if (count > length) count = length;
    if (!live) count = 0;
    const int start = length - count;
    bool has_query[kSets];
    int position[kSets];                                 // attends to cache tokens 0 .. position
#pragma unroll
    for (int i = 0; i < kSets; i++) {
        has_query[i] = t[i] < count;
        position[i] = start + t[i];
    }
    const int page_count = a.page_counts[slot], last_len = a.last_page_lens[slot], hot_len = a.hot_lengths[slot];

    // last position any vector of this tile looks at (uniform over the workgroup)
    const int tile_first = tile * kTileTokens;
    const int tile_last_token = (tile_first + kTileTokens < count ? tile_first + kTileTokens : count) - 1;
    const int all_pages = tile_last_token >= tile_first ? (start + tile_last_token) / P + 1 : 0;
    // this workgroup's pages of the table: [first_page, pages_needed)
    // (the last ranges, which only long contexts have, are dispatched first: the launch then ends on the
    // first ranges, which every row has)
    const int split_index = kSplit ? (int)(gridDim.y - 1 - blockIdx.y) : 0;
    const int first_page = split_index * a.pages_per_split;
    const int pages_needed = kSplit && first_page + a.pages_per_split < all_pages ? first_page + a.pages_per_split : all_pages;

    // Q^T fragments of the two 32-dim steps: lane (vector, quarter) holds dims 32 step + 8 quarter .. + 8
    bf16x8 q_frag[kSets][2];
    floatx4 o[kSets][4];                                 // O^T tiles: dims 16 tile + 4 quarter + r of this lane's vector
    float running_max[kSets], denom[kSets];
#pragma unroll
    for (int i = 0; i < kSets; i++) {
#pragma unroll
        for (int step = 0; step < 2; step++) {
            uint4 raw = make_uint4(0, 0, 0, 0);
            if (has_query[i]) raw = *reinterpret_cast<const uint4 *>(a.query + q_at[i] + 32 * step + 8 * quarter);
            q_frag[i][step] = __builtin_bit_cast(bf16x8, raw);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) o[i][j] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        running_max[i] = -INFINITY;
        denom[i] = 0.0f;
    }

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
    const uint8_t *side_hints = decodes_values ? a.value_hints : a.key_hints;
    const bool hinted = side_hints != nullptr;
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
        // the hint byte of the block's pair rides above the beta byte
        const uint32_t ids = (uint32_t)side_ids[word >> 2] | (hinted ? (uint32_t)side_hints[word >> 1] << 8 : 0u);
        return ColdOperands{side_codes[word], ids, side_norms[page * page_rows + (uint32_t)row_in_page]};
    };
    struct Staged { uint4 value, rest; };               // eight BF16 values, and for keys what their rounding left
    auto decode_cold = [&](const ColdOperands &operands) {
        float v[8];
        if (hinted) decode_codeword_hinted(operands.code, (operands.ids >> (8 + 4 * (dec_blk & 1))) & 15u, v);
        else decode_codeword<false>(operands.code, 14.0f, 0u, v);
        const float beta = beta_table[(operands.ids >> (2 * (dec_blk & 3))) & 3];
        const float back = operands.norm / sqrt_d;
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = (v[j] * beta) * back;
        uint32_t head[4], rest[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < 4; j++) head[j] = __builtin_bit_cast(uint32_t, pack_bf16x2(v[2 * j], v[2 * j + 1]));
        if (!decodes_values) {
#pragma unroll
            for (int j = 0; j < 4; j++)
                rest[j] = __builtin_bit_cast(uint32_t, pack_bf16x2(v[2 * j] - __uint_as_float(head[j] << 16),
                                                                   v[2 * j + 1] - __uint_as_float(head[j] & 0xffff0000u)));
        }
        return Staged{make_uint4(head[0], head[1], head[2], head[3]), make_uint4(rest[0], rest[1], rest[2], rest[3])};
    };
    auto write_page = [&](int buf, int half, const Staged &staged) {
        const uint4 packed = staged.value;
        if (decodes_values) {
            const uint32_t w[4] = {packed.x, packed.y, packed.z, packed.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v_page[buf][half][dec_blk * 8 + 2 * j][dec_token ^ (8 * (dec_blk >> 2))] = (uint16_t)(w[j] & 0xffffu);
                v_page[buf][half][dec_blk * 8 + 2 * j + 1][dec_token ^ (8 * (dec_blk >> 2))] = (uint16_t)(w[j] >> 16);
            }
        } else {
            *reinterpret_cast<uint4 *>(&k_page[buf][half][dec_token][dec_blk * 8]) = packed;
            *reinterpret_cast<uint4 *>(&k_rest[buf][half][dec_token][dec_blk * 8]) = staged.rest;
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
        bf16x8 k_frag[2][2], k_rest_frag[2][2];
#pragma unroll
        for (int half = 0; half < 2; half++)
#pragma unroll
            for (int step = 0; step < 2; step++) {
                k_frag[half][step] = __builtin_bit_cast(
                    bf16x8, *reinterpret_cast<const uint4 *>(&k_page[buf][half][lane & 15][32 * step + 8 * quarter]));
                k_rest_frag[half][step] = __builtin_bit_cast(
                    bf16x8, *reinterpret_cast<const uint4 *>(&k_rest[buf][half][lane & 15][32 * step + 8 * quarter]));
            }
        bf16x8 v_frag[4];
#pragma unroll
        for (int tile = 0; tile < 4; tile++) {
            const int column = (4 * quarter) ^ (8 * (tile >> 1));
            const uint2 v0 = *reinterpret_cast<const uint2 *>(&v_page[buf][0][16 * tile + (lane & 15)][column]);
            const uint2 v1 = *reinterpret_cast<const uint2 *>(&v_page[buf][1][16 * tile + (lane & 15)][column]);
            v_frag[tile] = __builtin_bit_cast(bf16x8, make_uint4(v0.x, v0.y, v1.x, v1.y));
        }
#pragma unroll
        for (int i = 0; i < kSets; i++) {
            float s[8], trip_max = -INFINITY;
#pragma unroll
            for (int half = 0; half < 2; half++) {
                floatx4 st = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int step = 0; step < 2; step++) {
                    st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_rest_frag[half][step], q_frag[i][step], st, 0, 0, 0);
                    st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_frag[half][step], q_frag[i][step], st, 0, 0, 0);
                }
                const int tokens_here = kMasked ? tokens_of(first + half) : P;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int tok = 4 * quarter + r;
                    const bool visible = !kMasked || (has_query[i] && tok < tokens_here && (first + half) * P + tok <= position[i]);
                    s[4 * half + r] = visible ? st[r] * a.scale : -INFINITY;
                    trip_max = fmaxf(trip_max, s[4 * half + r]);
                }
            }
            trip_max = quarters_max(trip_max);
            const float new_max = fmaxf(running_max[i], trip_max);
            // a vector that has seen nothing yet keeps max = -inf: exponents are forced to zero weight
            const float keep = (kMasked && new_max == -INFINITY) ? 1.0f : __expf(running_max[i] - new_max);
            float p[8], trip_sum = 0.0f;
#pragma unroll
            for (int r = 0; r < 8; r++) {
                p[r] = (kMasked && s[r] == -INFINITY) ? 0.0f : __expf(s[r] - new_max);
                trip_sum = trip_sum + p[r];
            }
            trip_sum = quarters_sum(trip_sum);
            denom[i] = denom[i] * keep + trip_sum;
            running_max[i] = new_max;
            // B operand of the 32-deep product: slots 0..3 = this lane's tokens of the first page, 4..7 of the second
            const uint4 p_bits = make_uint4(__builtin_bit_cast(uint32_t, pack_bf16x2(p[0], p[1])),
                                            __builtin_bit_cast(uint32_t, pack_bf16x2(p[2], p[3])),
                                            __builtin_bit_cast(uint32_t, pack_bf16x2(p[4], p[5])),
                                            __builtin_bit_cast(uint32_t, pack_bf16x2(p[6], p[7])));
            const bf16x8 p_frag = __builtin_bit_cast(bf16x8, p_bits);
#pragma unroll
            for (int tile = 0; tile < 4; tile++) {
#pragma unroll
                for (int r = 0; r < 4; r++) o[i][tile][r] = o[i][tile][r] * keep;
                o[i][tile] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_frag[tile], p_frag, o[i][tile], 0, 0, 0);
            }
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
    if (fast_pages < first_page) fast_pages = first_page;          // (first_page is even)
    int trip = 0;
    if (fast_pages > first_page) {
        ColdOperands next = request_cold(first_page + dec_half);
        for (int first = first_page; first < fast_pages; first += 2, trip++) {
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
            Staged staged{make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
            if (dec_token < tokens_of(ordinal)) {
                if (ordinal < page_count) staged = decode_cold(request_cold(ordinal));
                else staged.value = *reinterpret_cast<const uint4 *>(side_hot);      // BF16 rows: nothing left behind
            }
            write_page(trip & 1, dec_half, staged);
        }
        __syncthreads();
        attend(std::true_type{}, trip & 1, first);
    }
#pragma unroll
    for (int i = 0; i < kSets; i++) {
        if (t[i] >= a.tokens) continue;
        if (kSplit) {
            // unnormalised sums, maximum and denominator of this split (a split without a visible
            // token leaves -inf and 0: the merge gives it no weight)
            const int64_t at = (q_at[i] / D) * a.splits + split_index;
            if (first_page < all_pages) {                // (uniform; the merge reads no sums of a split without a denominator)
#pragma unroll
                for (int tile = 0; tile < 4; tile++)
                    *reinterpret_cast<float4 *>(a.part_out + at * D + 16 * tile + 4 * quarter) =
                        make_float4(o[i][tile][0], o[i][tile][1], o[i][tile][2], o[i][tile][3]);
            }
            // (a padding token's vector multiplied zeros on the unmasked trips: it gets no weight either)
            if (quarter == 0)
                *reinterpret_cast<float2 *>(a.part_stats + at * 2) =
                    has_query[i] ? make_float2(running_max[i], denom[i]) : make_float2(-INFINITY, 0.0f);
        } else {
            const float inv = (has_query[i] && denom[i] > 0.0f) ? 1.0f / denom[i] : 0.0f;   // padding tokens and inactive rows give zeros
#pragma unroll
            for (int tile = 0; tile < 4; tile++) {
                const uint32_t lo = (uint32_t)f32_to_bf16(o[i][tile][0] * inv) | ((uint32_t)f32_to_bf16(o[i][tile][1] * inv) << 16);
                const uint32_t hi = (uint32_t)f32_to_bf16(o[i][tile][2] * inv) | ((uint32_t)f32_to_bf16(o[i][tile][3] * inv) << 16);
                *reinterpret_cast<uint2 *>(a.out + q_at[i] + 16 * tile + 4 * quarter) = make_uint2(lo, hi);
            }
        }
    }
}

// One wavefront per query vector: out[d] = sum_s o_s[d] w_s / sum_s denom_s w_s with
// w_s = exp(max_s - max), splits in index order; a vector no split saw anything of gives zeros.
// All statistics are requested together, then all sums: two memory round trips per vector.
constexpr int kPrefillMaxSplits = 16;

template <int kSplits>
__global__ void __launch_bounds__(256)
attention_prefill_merge_kernel(const float *__restrict__ part_out, const float *__restrict__ part_stats, int64_t vectors,
                               uint16_t *__restrict__ out) {
    const int64_t vector = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int d = threadIdx.x & 63;
    if (vector >= vectors) return;
    const float2 *stats = reinterpret_cast<const float2 *>(part_stats) + vector * kSplits;
    float2 st[kSplits];
#pragma unroll
    for (int s = 0; s < kSplits; s++) st[s] = stats[s];
    float top = -INFINITY;
#pragma unroll
    for (int s = 0; s < kSplits; s++) top = fmaxf(top, st[s].x);
    float sums[kSplits];
#pragma unroll
    for (int s = 0; s < kSplits; s++)                    // (a split without a denominator wrote no sums)
        sums[s] = st[s].y > 0.0f ? part_out[(vector * kSplits + s) * 64 + d] : 0.0f;
    float total = 0.0f, weight_sum = 0.0f;
#pragma unroll
    for (int s = 0; s < kSplits; s++) {
        const float w = st[s].y > 0.0f ? __expf(st[s].x - top) : 0.0f;
        weight_sum = weight_sum + st[s].y * w;
        total = total + sums[s] * w;
    }
    out[vector * 64 + d] = f32_to_bf16(weight_sum > 0.0f ? total / weight_sum : 0.0f);
}

}  // namespace nq

namespace {

constexpr int kPrefillSets = 1;        // query-vector sets per lane (see the kernel)
constexpr int kPrefillWorkgroups = 2048;

// Splits of the page table: enough workgroups for the chip however few (row, tile, head) triples a
// launch has, with at least eight pages (four trips) per split.
int prefill_splits(int batch, int tokens, int max_pages, int group, int kv_heads) {
    const int tile_tokens = kPrefillSets * 128 / group;
    const int64_t workgroups = (int64_t)((tokens + tile_tokens - 1) / tile_tokens) * batch * kv_heads;
    int splits = 1;
    while (splits < nq::kPrefillMaxSplits && workgroups * splits < kPrefillWorkgroups && (max_pages + splits * 2 - 1) / (splits * 2) >= 8) splits *= 2;
    return splits;
}

}  // namespace

extern "C" size_t nq_nqkv_attention_prefill_workspace_bytes(int batch, int tokens, int max_pages, int q_heads,
                                                            int kv_heads) {
    if (batch < 1 || tokens < 1 || max_pages < 1 || kv_heads < 1 || q_heads < kv_heads || q_heads % kv_heads) return 0;
    const int splits = prefill_splits(batch, tokens, max_pages, q_heads / kv_heads, kv_heads);
    if (splits == 1) return 0;
    return (size_t)batch * tokens * q_heads * splits * (64 + 2) * sizeof(float);
}

extern "C" int nq_nqkv_attention_prefill(
    const void *query_dev, const uint8_t *key_codes_dev, const uint8_t *key_beta_ids_dev, const float *key_norms_dev,
    const uint8_t *value_codes_dev, const uint8_t *value_beta_ids_dev, const float *value_norms_dev,
    const float *key_betas_dev, const float *value_betas_dev, const int32_t *page_indices_dev,
    const int32_t *page_counts_dev, const int32_t *last_page_lens_dev, const int32_t *hot_lengths_dev,
    const int32_t *sequence_lengths_dev, const void *hot_keys_dev, const void *hot_values_dev,
    const int32_t *slot_ids_dev, const uint8_t *active_mask_dev, const int32_t *counts_dev, int uniform_count,
    int batch, int tokens, int slots, int max_pages, int q_heads, int kv_heads, int head_dim, int page_size,
    float scale, void *out_dev, void *workspace_dev, size_t workspace_bytes, const uint8_t *key_hints_dev,
    const uint8_t *value_hints_dev, void *stream) {
    NQ_REQUIRE(batch >= 1 && tokens >= 1 && slots >= 1 && max_pages >= 1, NQ_ERR_SHAPE,
               "nq_nqkv_attention_prefill: batch, tokens, slots and max_pages must be positive");
    NQ_REQUIRE((key_hints_dev == nullptr) == (value_hints_dev == nullptr), NQ_ERR_ARGUMENT,
               "nq_nqkv_attention_prefill: key and value hint streams come together");
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
    a.key_hints = key_hints_dev; a.value_hints = value_hints_dev;
    a.key_norms = key_norms_dev; a.value_norms = value_norms_dev;
    a.key_betas = key_betas_dev; a.value_betas = value_betas_dev;
    a.page_indices = page_indices_dev; a.page_counts = page_counts_dev; a.last_page_lens = last_page_lens_dev;
    a.hot_lengths = hot_lengths_dev; a.sequence_lengths = sequence_lengths_dev;
    a.hot_keys = reinterpret_cast<const uint16_t *>(hot_keys_dev);
    a.hot_values = reinterpret_cast<const uint16_t *>(hot_values_dev);
    a.slot_ids = slot_ids_dev; a.counts = counts_dev; a.active_mask = active_mask_dev;
    a.batch = batch; a.tokens = tokens; a.uniform_count = uniform_count; a.slots = slots; a.max_pages = max_pages;
    a.q_heads = q_heads; a.kv_heads = kv_heads; a.scale = scale;
    // the context is split when the caller's workspace has room for the partial results
    const size_t need = nq_nqkv_attention_prefill_workspace_bytes(batch, tokens, max_pages, q_heads, kv_heads);
    const bool split = need > 0 && workspace_dev && workspace_bytes >= need && nq::aligned(workspace_dev, 16);
    const int splits = split ? prefill_splits(batch, tokens, max_pages, group, kv_heads) : 1;
    const int64_t vectors = (int64_t)batch * tokens * q_heads;
    a.splits = splits;
    a.pages_per_split = ((max_pages + splits - 1) / splits + 1) & ~1;
    a.part_out = reinterpret_cast<float *>(workspace_dev);
    a.part_stats = a.part_out ? a.part_out + vectors * splits * 64 : nullptr;
    const int tile_tokens = kPrefillSets * 128 / group;
    const int64_t pairs = (int64_t)((tokens + tile_tokens - 1) / tile_tokens) * batch;     // (row, token tile), padded to eights
    const dim3 grid((unsigned)((pairs + 7) / 8 * 8 * kv_heads), (unsigned)splits);
    hipStream_t s = (hipStream_t)stream;
#define NQ_LAUNCH_PREFILL(GROUP)                                                                                     \
    if (split)                                                                                                       \
        hipLaunchKernelGGL((nq::attention_prefill_kernel<64, 16, GROUP, kPrefillSets, true>), grid,                  \
                           dim3(nq::kPrefillThreads), 0, s, a);                                                      \
    else                                                                                                             \
        hipLaunchKernelGGL((nq::attention_prefill_kernel<64, 16, GROUP, kPrefillSets, false>), grid,                 \
                           dim3(nq::kPrefillThreads), 0, s, a)
    switch (group) {
        case 1: NQ_LAUNCH_PREFILL(1); break;
        case 2: NQ_LAUNCH_PREFILL(2); break;
        case 4: NQ_LAUNCH_PREFILL(4); break;
        default: NQ_LAUNCH_PREFILL(8); break;
    }
#undef NQ_LAUNCH_PREFILL
    if (split) {
        const int status = nq::check_launch("nq_nqkv_attention_prefill");
        if (status != NQ_OK) return status;
        const dim3 merge_grid((unsigned)((vectors + 3) / 4));
        switch (splits) {                                // a power of two in [2, kPrefillMaxSplits]
            case 2: hipLaunchKernelGGL(nq::attention_prefill_merge_kernel<2>, merge_grid, dim3(256), 0, s, a.part_out, a.part_stats, vectors, a.out); break;
            case 4: hipLaunchKernelGGL(nq::attention_prefill_merge_kernel<4>, merge_grid, dim3(256), 0, s, a.part_out, a.part_stats, vectors, a.out); break;
            case 8: hipLaunchKernelGGL(nq::attention_prefill_merge_kernel<8>, merge_grid, dim3(256), 0, s, a.part_out, a.part_stats, vectors, a.out); break;
            default: hipLaunchKernelGGL(nq::attention_prefill_merge_kernel<16>, merge_grid, dim3(256), 0, s, a.part_out, a.part_stats, vectors, a.out); break;
        }
    }
    return nq::check_launch("nq_nqkv_attention_prefill");
}
