// Paged NQKV4 decode attention: one query token per batch row against that row's packed
// cold pages (4-bit E8 codes, decoded on the fly) plus its BF16 hot tail.
//
// Stage 1, grid = (chunks + 1, batch * kv_heads), 256 lanes.  A workgroup owns one batch
// row, one KV head and one chunk of 2, 4, 8 or 16 pages (the fewer rows and pages a launch
// covers, the smaller the chunks, so that short contexts still spread over the chip); the
// extra chunk is the hot tail.
//   * Every K and V block of the chunk is decoded exactly once and serves all query heads of
//     the GQA group (the reference decodes it once per query head,
//     nestquant/runtime/nqkv_attention_k1.py:243-342).
//   * K pass: lane (page, token, block) decodes its 8 keys, dots them with the group's
//     queries (kept in registers) and an 8-lane exchange yields scores in LDS.
//   * softmax over the chunk in LDS (FP32), then the V pass: every lane accumulates
//     p * v for its block over the pages it visits; lanes are merged through LDS in a fixed
//     order.  The chunk's (max, denominator, numerator[D]) go to the workspace.
// Stage 2, one wavefront per (row, head): log-sum-exp merge of the parts.
// Lengths, page tables and activity flags are read on the device, so the launch is
// replayable in a HIP graph; inactive rows produce zeros; there is no page-count limit
// beyond the table width (the reference stops at 64 pages, nqkv_attention_k1.py:696-698).
// Decoded K/V stay FP32 (as in the reference's fused kernel); K/V decode follows the exact
// float32 order of nq_e8.hip.h because undithered codes sit on exact Voronoi ties.
//
// A decode step can append as it attends (kWrites launches): the hot-tail workgroup of a row
// takes the row's new key and value straight from the projections, applies the rotary embedding
// and the Hadamard rotation to the key, stores the pair in the slot's hot tail and attends over
// the tail from LDS.  When the new token completes a page the workgroup encodes the page as the
// KV writer does (same device routine, same bits), stores it in the pool and attends over the
// 16 tokens through the codes it has just made; the workgroups of the cold chunks leave that
// page alone in this launch.  One launch per layer instead of the writer's and the attention's.
#define NQ_PHASE_STAMP_ARRAY g_attention_stamps
#include "nq_rowquant.hip.h"
#include "nq_host.h"

#include <math.h>

#ifdef NQ_PHASE_STAMPS
// Measuring builds only: the stamps the last stage-1 launch left (wall clock, 10 ns units).
extern "C" int nq_debug_attention_stamps(unsigned long long *out16) {
    if (hipDeviceSynchronize() != hipSuccess) return NQ_ERR_LAUNCH;
    return hipMemcpyFromSymbol(out16, HIP_SYMBOL(nq::g_attention_stamps), 16 * sizeof(unsigned long long)) == hipSuccess
               ? NQ_OK : NQ_ERR_LAUNCH;
}
#endif

namespace nq {

constexpr int kAttnThreads = 512;
constexpr int kAttnMaxPagesPerChunk = 16;

struct AttentionArgs {
    const void *query;                 // [batch, q_heads, D]
    const uint16_t *rope_cos, *rope_sin;   // optional BF16 [batch, D]: rotary embedding of the queries
    const uint32_t *key_codes, *value_codes;     // [pages][P * kv_heads * D / 8] words
    const uint8_t *key_beta_ids, *value_beta_ids; // [pages][P * kv_heads * D / 32]
    const float *key_norms, *value_norms;         // [pages][P * kv_heads]
    const float *key_betas, *value_betas;         // [4]
    const int32_t *page_indices;       // [slots, max_pages]
    const int32_t *page_counts, *last_page_lens, *hot_lengths;   // [slots]
    const uint8_t *cache_active;       // [slots] or null
    const uint16_t *hot_keys, *hot_values;        // BF16 [slots, P, kv_heads, D]
    const int32_t *slot_ids;           // [batch]
    const uint8_t *active_mask;        // [batch]
    int batch, slots, max_pages, q_heads, kv_heads, chunks, query_dtype, rotate_query;
    float scale;
    float *part_max, *part_sum, *part_acc;        // [batch, q_heads, chunks + 1] (x D)
    // kWrites launches only: one new token per active row
    const uint16_t *new_key, *new_value;          // BF16 [batch, kv_heads, D], the key before RoPE and rotation
    const int32_t *sequence_lengths;              // [slots], this step's token already counted
    int key_beta_count, rotate_keys;
    // optional decode hints [pages][P * kv_heads * D / 16], two blocks per byte (see decode_codeword_hinted):
    // read by every launch, written by a kWrites launch for the page it completes; null for none
    const uint8_t *key_hints, *value_hints;
};

// Rotary embedding ((x * cos) + (rotate_half(x) * sin) in BF16 tensor arithmetic), then optionally
// the Hadamard rotation (float32 butterflies over the head, scaled by 1 / sqrt(D), rounded to
// `dtype`: hadamard(x.float()).to(dtype), nestquant/runtime/nqkv_batched_hf_backend.py:381, 549) of a
// head vector of 64 held by eight neighbouring lanes, lane `piece` elements 8 piece .. 8 piece + 7.
__device__ __forceinline__ void rope_then_rotate(float (&x)[8], const float (&rope_c)[8], const float (&rope_s)[8],
                                                 bool rope, bool rotate, int dtype, int lane) {
    if (rope) {
        const bool upper = (lane & 7) >= 4;
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            const float o0 = lane_xor<4>(x[j]), o1 = lane_xor<4>(x[j + 1]);
            float a0 = x[j] * rope_c[j], a1 = x[j + 1] * rope_c[j + 1];
            round_pair<1>(a0, a1);
            float b0 = o0 * rope_s[j], b1 = o1 * rope_s[j + 1];
            round_pair<1>(b0, b1);
            x[j] = upper ? a0 + b0 : a0 - b0;
            x[j + 1] = upper ? a1 + b1 : a1 - b1;
            round_pair<1>(x[j], x[j + 1]);
        }
    }
    if (rotate) {
#pragma unroll
        for (int s = 0; s < 3; s++) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                if (j & (1 << s)) continue;
                const float left = x[j], right = x[j + (1 << s)];
                x[j] = left + right;
                x[j + (1 << s)] = left - right;
            }
        }
        lane_stage<1, 0>(x, lane);
        lane_stage<2, 0>(x, lane);
        lane_stage<4, 0>(x, lane);
        const float inv = 1.0f / __builtin_sqrtf(64.0f);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float scaled = x[j] * inv;
            x[j] = dtype == NQ_BF16 ? bf16_to_f32(f32_to_bf16(scaled)) : (dtype == NQ_F16 ? (float)(_Float16)scaled : scaled);
        }
    }
}

__device__ __forceinline__ void unpack_bf16_row(const uint4 &raw, float (&x)[8]) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        x[2 * j] = __uint_as_float(w[j] << 16);
        x[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
}

__device__ __forceinline__ float load_query(const void *q, int dtype, int64_t i) {
    if (dtype == NQ_BF16) return bf16_to_f32(reinterpret_cast<const uint16_t *>(q)[i]);
    if (dtype == NQ_F16) return f16_to_f32(reinterpret_cast<const uint16_t *>(q)[i]);
    return reinterpret_cast<const float *>(q)[i];
}

__device__ __forceinline__ float dpp_quad_xor1(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_quad_xor2(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_half_mirror(float v) {      // lane i <- lane 7 - i inside groups of 8
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_rotate8(float v) {          // lane i <- lane i ^ 8 inside rows of 16
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x128, 0xF, 0xF, true));
}

// sum over the 8 lanes that share a token (lane id bits 0..2), register exchanges only
__device__ __forceinline__ float sum8(float v) {
    v = v + dpp_quad_xor1(v);
    v = v + dpp_quad_xor2(v);
    v = v + dpp_half_mirror(v);
    return v;
}

// maximum / sum over the 64 lanes of a wavefront, the same value in every lane: register exchanges
// inside rows of 16 lanes, then the four rows through scalar registers
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_quad_xor1(v));
    v = fmaxf(v, dpp_quad_xor2(v));
    v = fmaxf(v, dpp_half_mirror(v));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true)));
    const int bits = __builtin_bit_cast(int, v);
    return fmaxf(fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0)),
                       __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16))),
                 fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32)),
                       __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48))));
}
__device__ __forceinline__ float wave_sum(float v) {
    v = v + dpp_quad_xor1(v);
    v = v + dpp_quad_xor2(v);
    v = v + dpp_half_mirror(v);
    v = v + __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    const int bits = __builtin_bit_cast(int, v);
    return (__builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0)) +
            __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16))) +
           (__builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32)) +
            __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48)));
}
// v + the value of the lane 16 / 32 further on (the same in both lanes)
__device__ __forceinline__ float fold_rows(float v) {
    const int bits = __builtin_bit_cast(int, v);
    const auto by16 = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    const float half = __builtin_bit_cast(float, (int)by16[0]) + __builtin_bit_cast(float, (int)by16[1]);
    const int half_bits = __builtin_bit_cast(int, half);
    const auto by32 = __builtin_amdgcn_permlane32_swap(half_bits, half_bits, false, false);
    return __builtin_bit_cast(float, (int)by32[0]) + __builtin_bit_cast(float, (int)by32[1]);
}

// The dependent loads of a workgroup are what a short context pays for, so they are arranged in
// three rounds, each requested as early as its addresses are known: (1) the row's slot and
// activity flag, the group's queries and their rotary rows; (2) the slot's lengths and the page
// ids of the chunk (requested for every ordinal of the chunk before the count says which exist);
// (3) the packed keys and values of every pass together.
template <int D, int P, int G, int kAttnPagesPerChunk, bool kWrites>   // head_dim, page_size, query heads per KV head, pages per chunk
__global__ void __launch_bounds__(kAttnThreads) attention_stage1_kernel(AttentionArgs a) {
    constexpr int kBlocks = D / 8;                       // E8 blocks per head vector
    constexpr int kTokenBlocks = P * kBlocks;            // lanes needed per page
    constexpr int kPagesPerPass = kAttnThreads / kTokenBlocks;
    constexpr int kPasses = kAttnPagesPerChunk / kPagesPerPass;
    constexpr int kChunkTokens = kAttnPagesPerChunk * P;
    constexpr int kWaves = kAttnThreads / 64;
    static_assert(kTokenBlocks * kPagesPerPass == kAttnThreads && kPasses * kPagesPerPass == kAttnPagesPerChunk,
                  "page does not tile the workgroup");
    static_assert(D == 64 && G * 8 <= 64 && kBlocks == 8, "eight lanes of the first wavefront prepare one head's query");
    static_assert(kChunkTokens % 64 == 0, "every lane of a wavefront takes the same number of scores");
    static_assert(2 * kTokenBlocks <= kAttnThreads, "one lane per block of the tail's keys and values");
    __shared__ float scores[G][kChunkTokens];
    __shared__ __align__(16) float acc_lds[kWaves][kBlocks][G * 8];    // one entry per wavefront; holds the queries first
    // kWrites: the slot's hot tail with the new token (keys, then values), and the page made from it
    __shared__ float tail[kWrites ? 2 * P : 1][kWrites ? D : 1];
    __shared__ float tail_scale[kWrites ? 2 * P : 1], tail_norm[kWrites ? 2 * P : 1];
    __shared__ uint32_t tail_code[kWrites ? 2 * P : 1][kWrites ? kBlocks : 1];
    __shared__ uint32_t tail_ids[kWrites ? 2 * P : 1][kWrites ? kBlocks / 4 : 1];
    __shared__ uint32_t tail_hint[kWrites ? 2 * P : 1][kWrites ? kBlocks / 2 : 1];

    const int tid = threadIdx.x;
    NQ_STAMP(0);
    // Workgroups go to the eight XCDs in turn by their linear index, and every XCD has its own L2.
    // A page stores the blocks of all KV heads of a token side by side, so the workgroups of one
    // (row, chunk) -- one per KV head -- fetch the same cache lines: they are numbered so that they
    // share an XCD and follow each other there (index = 8 * (kv_heads * (pair / 8) + head) + pair % 8).
    // Pair p lands on XCD p % 8.  The pairs are numbered part by part, the rows of a part side by side
    // and one place further round for every part (p = part * batch + (row + part) % batch): the rows'
    // early chunks, the ones that every row has, then spread over the XCDs, and so do the chunks of a
    // long row.  (Numbered row by row, chunk 0 of every row of a table of eight parts fell to XCD 0:
    // 13.6 against 10 us for 8 rows of 150 tokens in a 25-page table.)  The hot tails, whose workgroups
    // also append the step's token, are the first part.
    const int place = blockIdx.x >> 3, pair = (place / a.kv_heads) * 8 + (blockIdx.x & 7);
    const int g = place % a.kv_heads;
    const int order = pair / a.batch, seat = pair - order * a.batch;
    if (order > a.chunks) return;                        // padding of the last group of eight pairs
    const int row = (seat + a.batch - order % a.batch) % a.batch;
    const int chunk = order == 0 ? a.chunks : order - 1;
    const bool is_hot = chunk == a.chunks;
    const bool appends = kWrites && is_hot;              // this workgroup owns the row's new token
    const int first_page = chunk * kAttnPagesPerChunk;
    const int64_t part = ((int64_t)row * a.q_heads + (int64_t)g * G) * (a.chunks + 1) + chunk;   // + h * (chunks + 1)

    // lane role inside a pass
    const int pass_page = tid / kTokenBlocks, token = (tid % kTokenBlocks) / kBlocks, blk = tid % kBlocks;
    const int row_in_page = token * a.kv_heads + g;
    const int64_t page_words = (int64_t)P * a.kv_heads * kBlocks, page_rows = (int64_t)P * a.kv_heads;

    // ---- first loads: slot, activity, queries (and the new key and value) --------------------------
    const int given_slot = a.slot_ids[row];
    const bool row_active = a.active_mask[row] != 0;
    // lane 8 h + piece of the first wavefront holds elements 8 piece .. 8 piece + 7 of head h; the
    // first eight lanes of the second wavefront hold the new key the same way
    const int qh = tid >> 3, piece = tid & 7;
    const bool key_lane = appends && tid >= 64 && tid < 72;
    float qv[8], rope_c[8], rope_s[8];
    uint4 new_value = make_uint4(0, 0, 0, 0);
    if (tid < G * 8 || key_lane) {
        if (key_lane) {
            unpack_bf16_row(*reinterpret_cast<const uint4 *>(a.new_key + ((int64_t)row * a.kv_heads + g) * D + piece * 8), qv);
        } else {
            const int64_t at = ((int64_t)row * a.q_heads + g * G + qh) * D + piece * 8;
            if (a.query_dtype == NQ_BF16) {
                unpack_bf16_row(*reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(a.query) + at), qv);
            } else {
#pragma unroll
                for (int j = 0; j < 8; j++) qv[j] = load_query(a.query, a.query_dtype, at + j);
            }
        }
        if (a.rope_cos) {
            const int64_t rope_at = (int64_t)row * D + piece * 8;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                rope_c[j] = bf16_to_f32(a.rope_cos[rope_at + j]);
                rope_s[j] = bf16_to_f32(a.rope_sin[rope_at + j]);
            }
        }
    }
    // lanes 128 .. 255 stage the tail's values: each requests the new value's piece it may need
    if (appends && tid >= kTokenBlocks && tid < 2 * kTokenBlocks)
        new_value = *reinterpret_cast<const uint4 *>(a.new_value + ((int64_t)row * a.kv_heads + g) * D + blk * 8);
    // beta tables in registers: a table lookup from memory would sit behind every decode
    const float key_beta[4] = {a.key_betas[0], a.key_betas[1], a.key_betas[2], a.key_betas[3]};
    const float value_beta[4] = {a.value_betas[0], a.value_betas[1], a.value_betas[2], a.value_betas[3]};

    // ---- second loads: lengths and page ids of the slot -------------------------------------------
    const bool slot_known = given_slot >= 0 && given_slot < a.slots;
    const int slot = given_slot < 0 ? 0 : (given_slot >= a.slots ? a.slots - 1 : given_slot);
    const int page_count = a.page_counts[slot], last_len = a.last_page_lens[slot], hot_len = a.hot_lengths[slot];
    const int length = kWrites ? a.sequence_lengths[slot] : 0;
    const bool cache_live = !a.cache_active || a.cache_active[slot];
    int64_t pass_pageid[kPasses];
#pragma unroll
    for (int pass = 0; pass < kPasses; pass++) {
        const int ordinal = first_page + pass * kPagesPerPass + pass_page;
        pass_pageid[pass] = (!is_hot && ordinal < a.max_pages) ? a.page_indices[(int64_t)slot * a.max_pages + ordinal] : 0;
    }
    NQ_STAMP(1);
    // the row's new token (as the KV writer decides it: an active row with a known slot that holds
    // at least this token) sits at position length - 1; it completes a page when length % P == 0
    const bool writes = kWrites && row_active && slot_known && length > 0;
    const bool packs = writes && length % P == 0;
    const int new_at = writes ? (length - 1) % P : -1;           // the new token's place in the tail
    const int tail_old = writes ? new_at : hot_len;              // tokens the tail held before this step
    const int hot_tokens = packs ? P : hot_len;                  // tokens the hot workgroup attends over
    const int cold_pages = page_count - (packs ? 1 : 0);         // the page being made is the hot workgroup's
    const bool live = row_active && cache_live;
    const bool empty = !live || (is_hot ? hot_tokens <= 0 : first_page >= cold_pages);
    if (empty && !(appends && writes)) {                 // uniform over the workgroup
        if (tid < G) {
            a.part_max[part + (int64_t)tid * (a.chunks + 1)] = -INFINITY;
            a.part_sum[part + (int64_t)tid * (a.chunks + 1)] = 0.0f;
        }
        return;
    }

    // ---- third loads: the packed operands of all passes, keys and values --------------------------------
    const bool hinted = a.key_hints != nullptr;
    bool pass_valid[kPasses];
    uint32_t k_code[kPasses], k_ids[kPasses], v_code[kPasses], v_ids[kPasses];
    float k_norm[kPasses], v_norm[kPasses];
    uint4 hot_k = make_uint4(0, 0, 0, 0), hot_v = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int pass = 0; pass < kPasses; pass++) {
        const int ordinal = first_page + pass * kPagesPerPass + pass_page;
        pass_valid[pass] = is_hot ? (pass == 0 && pass_page == 0 && token < hot_tokens)
                                  : (ordinal < cold_pages && (ordinal < cold_pages - 1 || token < last_len));
        k_code[pass] = 0u; k_ids[pass] = 0u; k_norm[pass] = 0.0f;
        v_code[pass] = 0u; v_ids[pass] = 0u; v_norm[pass] = 0.0f;
        if (!is_hot && pass_valid[pass]) {
            const int64_t word = pass_pageid[pass] * page_words + (int64_t)row_in_page * kBlocks + blk;
            const int64_t norm = pass_pageid[pass] * page_rows + row_in_page;
            k_code[pass] = a.key_codes[word];
            k_ids[pass] = a.key_beta_ids[word >> 2];
            k_norm[pass] = a.key_norms[norm];
            v_code[pass] = a.value_codes[word];
            v_ids[pass] = a.value_beta_ids[word >> 2];
            v_norm[pass] = a.value_norms[norm];
            if (hinted) {                        // the hint byte of the block's pair rides above the beta byte
                k_ids[pass] |= (uint32_t)a.key_hints[word >> 1] << 8;
                v_ids[pass] |= (uint32_t)a.value_hints[word >> 1] << 8;
            }
        }
    }
    int64_t new_page = -1;
    if (appends) {
        // lanes 0 .. 127 stage the tail's keys, lanes 128 .. 255 its values (lane = token * 8 + block)
        if (tid < 2 * kTokenBlocks && token < tail_old) {
            const int64_t at = (((int64_t)slot * P + token) * a.kv_heads + g) * D + blk * 8;
            hot_k = *reinterpret_cast<const uint4 *>((tid < kTokenBlocks ? a.hot_keys : a.hot_values) + at);
        }
        if (packs) new_page = a.page_indices[(int64_t)slot * a.max_pages + (length - 1) / P];
    } else if (is_hot && pass_valid[0]) {
        const int64_t at = (((int64_t)slot * P + token) * a.kv_heads + g) * D + blk * 8;
        hot_k = *reinterpret_cast<const uint4 *>(a.hot_keys + at);
        hot_v = *reinterpret_cast<const uint4 *>(a.hot_values + at);
    }

    // the group's queries (and the new key): rotary embedding, then the Hadamard rotation
    float *q_lds = &acc_lds[0][0][0];                    // free until the V pass ends
    static_assert(sizeof(acc_lds) >= sizeof(float) * G * D, "the query staging fits the accumulator buffer");
    if (tid < G * 8 || key_lane) {
        rope_then_rotate(qv, rope_c, rope_s, a.rope_cos != nullptr, key_lane ? a.rotate_keys != 0 : a.rotate_query != 0,
                         key_lane ? (int)NQ_BF16 : a.query_dtype, tid);
        if (!key_lane) {
#pragma unroll
            for (int j = 0; j < 8; j++) q_lds[qh * D + piece * 8 + j] = qv[j];
        } else if (writes) {
#pragma unroll
            for (int j = 0; j < 8; j++) tail[new_at][piece * 8 + j] = qv[j];
            if (!packs) {                                // the rotated key joins the slot's hot tail
                uint4 packed;
                packed.x = f32_to_bf16(qv[0]) | ((uint32_t)f32_to_bf16(qv[1]) << 16);
                packed.y = f32_to_bf16(qv[2]) | ((uint32_t)f32_to_bf16(qv[3]) << 16);
                packed.z = f32_to_bf16(qv[4]) | ((uint32_t)f32_to_bf16(qv[5]) << 16);
                packed.w = f32_to_bf16(qv[6]) | ((uint32_t)f32_to_bf16(qv[7]) << 16);
                *reinterpret_cast<uint4 *>(const_cast<uint16_t *>(a.hot_keys) +
                                           (((int64_t)slot * P + new_at) * a.kv_heads + g) * D + piece * 8) = packed;
            }
        }
    }
    if (appends && tid < 2 * kTokenBlocks) {
        const bool of_values = tid >= kTokenBlocks;
        const bool is_new = token == new_at;             // never for a row that writes nothing
        if (is_new && of_values && !packs)
            *reinterpret_cast<uint4 *>(const_cast<uint16_t *>(a.hot_values) +
                                       (((int64_t)slot * P + new_at) * a.kv_heads + g) * D + blk * 8) = new_value;
        if (!is_new || of_values) {                      // the new key comes from its eight lanes above
            float x[8];
            unpack_bf16_row(is_new ? new_value : hot_k, x);      // rows past the tail are zeros
#pragma unroll
            for (int j = 0; j < 8; j++) tail[(of_values ? P : 0) + token][blk * 8 + j] = x[j];
        }
    }
    __syncthreads();
    NQ_STAMP(2);
    if constexpr (kWrites) {
        if (packs) {
            // the tail is a complete page: norms, codes and beta ids as the KV writer makes them, kept in
            // LDS for this launch's attention and stored in the pool
            const float sqrt_d = __builtin_sqrtf((float)D);
            staged_row_norms(&tail[0][0], 2 * P, D, sqrt_d, tail_scale, tail_norm);
            if (new_page >= 0 && tid < 2 * P)
                const_cast<float *>(tid < P ? a.key_norms : a.value_norms)[new_page * page_rows + (tid % P) * a.kv_heads + g] =
                    tail_norm[tid];
            struct Sink {
                uint32_t *key_codes, *value_codes; uint8_t *key_beta_ids, *value_beta_ids;
                uint32_t (*code_lds)[kBlocks]; uint32_t (*ids_lds)[kBlocks / 4];
                int64_t page_word0; int kv_heads, g; bool mapped;
                __device__ __forceinline__ bool wants(int) const { return true; }
                __device__ __forceinline__ int64_t word(int r, int b) const {
                    return page_word0 + ((int64_t)(r % P) * kv_heads + g) * kBlocks + b;
                }
                __device__ __forceinline__ void code(int r, int b, uint32_t w, const float (&)[8], float) const {
                    code_lds[r][b] = w;
                    if (mapped) (r < P ? key_codes : value_codes)[word(r, b)] = w;
                }
                __device__ __forceinline__ void beta_byte(int r, int b, uint32_t byte) const {
                    ids_lds[r][b >> 2] = byte;
                    if (mapped) (r < P ? key_beta_ids : value_beta_ids)[word(r, b) >> 2] = (uint8_t)byte;
                }
                __device__ __forceinline__ uint32_t counter(int, int) const { return 0u; }
            } sink{const_cast<uint32_t *>(a.key_codes), const_cast<uint32_t *>(a.value_codes),
                   const_cast<uint8_t *>(a.key_beta_ids), const_cast<uint8_t *>(a.value_beta_ids), tail_code, tail_ids,
                   new_page * page_words, a.kv_heads, g, new_page >= 0};
            struct Betas {
                const float *key, *value;
                __device__ __forceinline__ const float *operator()(int r) const { return r < P ? key : value; }
            } betas_of{a.key_betas, a.value_betas};
            quantize_staged_pairs<false>(&tail[0][0], tail_scale, D, 14.0f, 1.0f / 14.0f, betas_of, a.key_beta_count,
                                         0u, 0, 2 * P * kBlocks * 4, sink);
            __syncthreads();
            if (hinted) {                                // the new page's decode hints, from its code words
                if (tid < 2 * P * (kBlocks / 2)) {
                    const int r = tid / (kBlocks / 2), pair = tid % (kBlocks / 2);
                    const uint32_t byte = hint_of_codeword(tail_code[r][2 * pair]) | (hint_of_codeword(tail_code[r][2 * pair + 1]) << 4);
                    tail_hint[r][pair] = byte;
                    if (new_page >= 0)
                        const_cast<uint8_t *>(r < P ? a.key_hints : a.value_hints)[sink.word(r, 2 * pair) >> 1] = (uint8_t)byte;
                }
                __syncthreads();
            }
        }
    }
    if (empty) {                                         // the row's cache is switched off: the append was all
        if (tid < G) {
            a.part_max[part + (int64_t)tid * (a.chunks + 1)] = -INFINITY;
            a.part_sum[part + (int64_t)tid * (a.chunks + 1)] = 0.0f;
        }
        return;
    }
    if (appends && packs && pass_valid[0]) {
        k_code[0] = tail_code[token][blk]; k_ids[0] = tail_ids[token][blk >> 2]; k_norm[0] = tail_norm[token];
        v_code[0] = tail_code[P + token][blk]; v_ids[0] = tail_ids[P + token][blk >> 2]; v_norm[0] = tail_norm[P + token];
        if (hinted) {
            k_ids[0] |= tail_hint[token][blk >> 1] << 8;
            v_ids[0] |= tail_hint[P + token][blk >> 1] << 8;
        }
    }
    const bool bf16_rows = is_hot && !packs;             // the pass reads BF16 rows, not codes
    float q[G][8];
#pragma unroll
    for (int h = 0; h < G; h++)
#pragma unroll
        for (int j = 0; j < 8; j++) q[h][j] = q_lds[h * D + blk * 8 + j];
    const float sqrt_d = __builtin_sqrtf((float)D);

    // ---- K pass -----------------------------------------------------------------------------
    NQ_STAMP(3);
#pragma unroll
    for (int pass = 0; pass < kPasses; pass++) {
        const int page_in_chunk = pass * kPagesPerPass + pass_page;
        const bool valid = pass_valid[pass];
        float k[8];
#pragma unroll
        for (int j = 0; j < 8; j++) k[j] = 0.0f;
        if (bf16_rows) {
            if (appends) {
                if (valid) {
#pragma unroll
                    for (int j = 0; j < 8; j++) k[j] = tail[token][blk * 8 + j];
                }
            } else {
                unpack_bf16_row(hot_k, k);
            }
        } else if (valid) {
            if (hinted) decode_codeword_hinted(k_code[pass], (k_ids[pass] >> (8 + 4 * (blk & 1))) & 15u, k);
            else decode_codeword<false>(k_code[pass], 14.0f, 0u, k);
            const float beta = key_beta[(k_ids[pass] >> (2 * (blk & 3))) & 3];     // word index % 4 == blk % 4
            const float back = k_norm[pass] / sqrt_d;
#pragma unroll
            for (int j = 0; j < 8; j++) k[j] = (k[j] * beta) * back;
        }
        // every pass writes its scores, so a hot or ragged chunk leaves no stale entry (the sums of
        // all heads first, then one predicated stretch of stores: a store between two sums would end
        // the basic block and keep the sums from overlapping)
        float s[G];
#pragma unroll
        for (int h = 0; h < G; h++) {
            s[h] = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) s[h] = __builtin_fmaf(q[h][j], k[j], s[h]);
            s[h] = sum8(s[h]);
        }
        if (blk == 0) {
#pragma unroll
            for (int h = 0; h < G; h++) scores[h][page_in_chunk * P + token] = valid ? s[h] * a.scale : -INFINITY;
        }
    }
    __syncthreads();                                     // scores complete; the queries in acc_lds are no longer needed
    NQ_STAMP(4);

    // ---- softmax over the chunk: every wavefront works out the maximum and the denominator for
    // itself (no hand-over between wavefronts), every lane the weights of its own tokens -------------
    float chunk_max[G], chunk_sum[G];
#pragma unroll
    for (int h = 0; h < G; h++) {
        float m = -INFINITY;
#pragma unroll
        for (int t = 0; t < kChunkTokens / 64; t++) m = fmaxf(m, scores[h][(tid & 63) + 64 * t]);
        chunk_max[h] = wave_max(m);                      // finite: the chunk holds at least one token
        float s = 0.0f;
#pragma unroll
        for (int t = 0; t < kChunkTokens / 64; t++) s = s + __expf(scores[h][(tid & 63) + 64 * t] - chunk_max[h]);
        chunk_sum[h] = wave_sum(s);
    }

    // ---- V pass ------------------------------------------------------------------------------
    NQ_STAMP(5);
    float acc[G][8];
#pragma unroll
    for (int h = 0; h < G; h++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[h][j] = 0.0f;
#pragma unroll
    for (int pass = 0; pass < kPasses; pass++) {
        const int page_in_chunk = pass * kPagesPerPass + pass_page;
        const bool valid = pass_valid[pass];
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = 0.0f;
        if (bf16_rows) {
            if (appends) {
                if (valid) {
#pragma unroll
                    for (int j = 0; j < 8; j++) v[j] = tail[P + token][blk * 8 + j];
                }
            } else {
                unpack_bf16_row(hot_v, v);
            }
        } else if (valid) {
            if (hinted) decode_codeword_hinted(v_code[pass], (v_ids[pass] >> (8 + 4 * (blk & 1))) & 15u, v);
            else decode_codeword<false>(v_code[pass], 14.0f, 0u, v);
            const float beta = value_beta[(v_ids[pass] >> (2 * (blk & 3))) & 3];
            const float back = v_norm[pass] / sqrt_d;
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = (v[j] * beta) * back;
        }
#pragma unroll
        for (int h = 0; h < G; h++) {
            // exp(-inf - max) = 0 for a token that does not exist
            const float p = __expf(scores[h][page_in_chunk * P + token] - chunk_max[h]);
#pragma unroll
            for (int j = 0; j < 8; j++) acc[h][j] = __builtin_fmaf(p, v[j], acc[h][j]);
        }
    }
    NQ_STAMP(6);
    // lanes that share a block index hold partial sums of the same 8 output dims: folded inside the
    // wavefront with register exchanges (the two tokens of a 16-lane row, then the four rows),
    // wavefronts through LDS in order
    // (all the sums first, then one predicated stretch of 128-bit stores, as above)
#pragma unroll
    for (int h = 0; h < G; h++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[h][j] = fold_rows(acc[h][j] + dpp_rotate8(acc[h][j]));
    if ((tid & 63) < 8) {
#pragma unroll
        for (int h = 0; h < G; h++) {
            float4 *to = reinterpret_cast<float4 *>(&acc_lds[tid >> 6][tid & 7][h * 8]);
            to[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
            to[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
        }
    }
    NQ_STAMP(8);
    __syncthreads();
    NQ_STAMP(9);
    for (int o = tid; o < G * D; o += kAttnThreads) {
        const int h = o / D, d = o % D;
        float total = acc_lds[0][d / 8][h * 8 + d % 8];
#pragma unroll
        for (int w = 1; w < kWaves; w++) total = total + acc_lds[w][d / 8][h * 8 + d % 8];
        a.part_acc[(part + (int64_t)h * (a.chunks + 1)) * D + d] = total;
    }
    if (tid < G) {
#pragma unroll
        for (int h = 0; h < G; h++) {
            if (tid == h) {
                a.part_max[part + (int64_t)h * (a.chunks + 1)] = chunk_max[h];
                a.part_sum[part + (int64_t)h * (a.chunks + 1)] = chunk_sum[h];
            }
        }
    }
    NQ_STAMP(7);
}

// Stage 2, one wavefront per (row, head): out[d] = sum_c acc_c[d] w_c / sum_c sum_c w_c with
// w_c = exp(max_c - max).  Lanes first take one part each (max, weights), then one output
// dimension each; every load of a phase is independent of the others.
template <int D>
__global__ void __launch_bounds__(64)
attention_merge_kernel(const float *__restrict__ part_max, const float *__restrict__ part_sum,
                       const float *__restrict__ part_acc, int parts, int64_t heads_total,
                       void *__restrict__ out, int out_dtype) {
    static_assert(D == 64, "one output dimension per lane");
    constexpr int kMaxParts = 512;
    __shared__ float weight[kMaxParts];
    const int64_t head = blockIdx.x;
    const int lane = threadIdx.x;
    const float *m = part_max + head * parts, *s = part_sum + head * parts;
    float top = -INFINITY;
    for (int c = lane; c < parts; c += 64) top = fmaxf(top, m[c]);
#pragma unroll
    for (int offset = 32; offset >= 1; offset >>= 1) top = fmaxf(top, __shfl_xor(top, offset, 64));
    float denom = 0.0f;
    for (int c = lane; c < parts; c += 64) {
        const float sc = s[c];
        const float w = (sc > 0.0f && top > -INFINITY) ? __expf(m[c] - top) : 0.0f;
        weight[c] = w;
        denom = denom + sc * w;
    }
#pragma unroll
    for (int offset = 32; offset >= 1; offset >>= 1) denom = denom + __shfl_xor(denom, offset, 64);
    __syncthreads();
    // empty parts hold no numerator: their (unwritten) entry is read but never used
    float numer = 0.0f;
    const float *acc = part_acc + head * parts * D + lane;
#pragma unroll 8
    for (int c = 0; c < parts; c++) {
        const float value = acc[(int64_t)c * D], w = weight[c];
        numer = numer + (w > 0.0f ? value * w : 0.0f);
    }
    const float result = denom > 0.0f ? numer / denom : 0.0f;      // inactive or empty rows give zeros
    const int64_t i = head * D + lane;
    if (out_dtype == NQ_BF16) reinterpret_cast<uint16_t *>(out)[i] = f32_to_bf16(result);
    else if (out_dtype == NQ_F16) reinterpret_cast<_Float16 *>(out)[i] = (_Float16)result;
    else reinterpret_cast<float *>(out)[i] = result;
}

}  // namespace nq

namespace {

// Pages per chunk, from measurements of the appending launch over batches of 1 to 16, tables of 21 to
// 512 pages and contexts from 150 tokens to the whole table (a launch has one workgroup per (row,
// chunk, KV head) of the table, whatever the rows hold: the host does not know their lengths).  A
// workgroup alone on the chip takes 9 us with up to 4 pages, 10 with 8 and 11 to 13.5 with 16, mostly
// the latency of its dependent loads; two workgroups on a compute unit share its vector units for the
// decode of their pages, and every chunk is a part to merge.  With eight KV heads 32 (row, chunk)
// pairs are one workgroup per compute unit: 4 pages while the launch stays within that, 8 pages up
// to 100 pairs, 16 beyond (us with 4 / 8 / 16 pages: 8 rows of a 21-page table, 150 tokens 9.3 /
// 10.2 / 11.4, full 13.6 / 10.1 / 13.6; 8 rows of 64 pages full 27.1 / 18.5 / 17.4, half 16.9 / 12.5 /
// 13.7; 8 rows of 256 pages with mixed lengths 52.5 / 33.2 / 32.1, full 89.6 / 50.0 / 42.1).
int pages_per_chunk_for(int batch, int max_pages) {
#ifdef NQ_ATTN_FORCE_PAGES                       // measuring builds only
    return NQ_ATTN_FORCE_PAGES;
#endif
    const auto pairs = [&](int pages) { return (int64_t)batch * ((max_pages + pages - 1) / pages + 1); };
    if (pairs(4) <= 32) return 4;
    return pairs(8) <= 100 ? 8 : nq::kAttnMaxPagesPerChunk;
}

int chunks_for(int batch, int max_pages) {
    const int pages = pages_per_chunk_for(batch, max_pages);
    return (max_pages + pages - 1) / pages;
}

}  // namespace

extern "C" int nq_nqkv_attention_parts(int batch, int max_pages) {
    if (batch < 1 || max_pages < 1) return 0;
    return chunks_for(batch, max_pages) + 1;
}

extern "C" size_t nq_nqkv_attention_workspace_bytes(int batch, int q_heads, int head_dim, int max_pages) {
    if (batch < 1 || q_heads < 1 || head_dim < 1 || max_pages < 1) return 0;
    const size_t parts = (size_t)chunks_for(batch, max_pages) + 1;
    return (size_t)batch * q_heads * parts * ((size_t)head_dim + 2) * sizeof(float);
}

namespace {

// What a launch that appends as it attends adds to the attention's operands.
struct AppendOperands {
    const void *key, *value;               // BF16 [batch, kv_heads, head_dim]
    const int32_t *sequence_lengths;
    int key_beta_count, value_beta_count, rotate_keys;
};

int launch_decode_attention(
    const char *entry, const AppendOperands *append,
    const void *query_dev, int query_dtype, const uint8_t *key_codes_dev, const uint8_t *key_beta_ids_dev,
    const float *key_norms_dev, const uint8_t *value_codes_dev, const uint8_t *value_beta_ids_dev,
    const float *value_norms_dev, const float *key_betas_dev, const float *value_betas_dev,
    const int32_t *page_indices_dev, const int32_t *page_counts_dev, const int32_t *last_page_lens_dev,
    const int32_t *hot_lengths_dev, const uint8_t *cache_active_dev, const void *hot_keys_dev,
    const void *hot_values_dev, const int32_t *slot_ids_dev, const uint8_t *active_mask_dev, int batch,
    int slots, int max_pages, int q_heads, int kv_heads, int head_dim, int page_size, float scale,
    int rotate_query, const void *rope_cos_dev, const void *rope_sin_dev, void *out_dev, void *workspace_dev,
    size_t workspace_bytes, const uint8_t *key_hints_dev, const uint8_t *value_hints_dev, void *stream) {
    NQ_REQUIRE(batch >= 1 && slots >= 1 && max_pages >= 1, NQ_ERR_SHAPE,
               "%s: batch, slots and max_pages must be positive", entry);
    NQ_REQUIRE((key_hints_dev == nullptr) == (value_hints_dev == nullptr), NQ_ERR_ARGUMENT,
               "%s: key and value hint streams come together", entry);
    NQ_REQUIRE(kv_heads >= 1 && q_heads >= kv_heads && q_heads % kv_heads == 0, NQ_ERR_SHAPE,
               "%s: q_heads must be a positive multiple of kv_heads", entry);
    const int group = q_heads / kv_heads;
    NQ_REQUIRE(head_dim == 64 && page_size == 16, NQ_ERR_SHAPE,
               "%s: built for head_dim 64 and 16-token pages (got %d, %d)", entry, head_dim, page_size);
    NQ_REQUIRE(group == 1 || group == 2 || group == 4 || group == 8, NQ_ERR_SHAPE,
               "%s: %d query heads per KV head is not 1, 2, 4 or 8", entry, group);
    NQ_REQUIRE(query_dtype == NQ_F32 || query_dtype == NQ_BF16 || query_dtype == NQ_F16, NQ_ERR_ARGUMENT,
               "%s: unknown dtype tag %d", entry, query_dtype);
    NQ_REQUIRE(query_dev && key_codes_dev && key_beta_ids_dev && key_norms_dev && value_codes_dev &&
                   value_beta_ids_dev && value_norms_dev && key_betas_dev && value_betas_dev && page_indices_dev &&
                   page_counts_dev && last_page_lens_dev && hot_lengths_dev && hot_keys_dev && hot_values_dev &&
                   slot_ids_dev && active_mask_dev,
               NQ_ERR_ARGUMENT, "%s: null pointer", entry);
    NQ_REQUIRE(nq::aligned(key_codes_dev, 4) && nq::aligned(value_codes_dev, 4) && nq::aligned(hot_keys_dev, 16) &&
                   nq::aligned(hot_values_dev, 16),
               NQ_ERR_ARGUMENT, "%s: page streams need 4-byte, hot tails 16-byte alignment", entry);
    // a BF16 query row is read eight values (16 bytes) at a time; the other element types and the
    // BF16 rotary rows one value at a time
    NQ_REQUIRE(nq::aligned(query_dev, query_dtype == NQ_BF16 ? 16 : (query_dtype == NQ_F32 ? 4 : 2)), NQ_ERR_ARGUMENT,
               "%s: a BF16 query needs 16-byte alignment (float32 4, float16 2)", entry);
    NQ_REQUIRE(nq::aligned(rope_cos_dev, 2) && nq::aligned(rope_sin_dev, 2), NQ_ERR_ARGUMENT,
               "%s: rotary rows need 2-byte alignment", entry);
    NQ_REQUIRE(isfinite(scale), NQ_ERR_ARGUMENT, "%s: scale must be finite", entry);
    NQ_REQUIRE(chunks_for(batch, max_pages) + 1 <= 512, NQ_ERR_SHAPE,
               "%s: a page table of %d pages needs more than 512 context chunks", entry, max_pages);
    const size_t need = nq_nqkv_attention_workspace_bytes(batch, q_heads, head_dim, max_pages);
    NQ_REQUIRE(workspace_dev && workspace_bytes >= need, NQ_ERR_WORKSPACE,
               "%s: needs a %zu-byte workspace, got %zu", entry, need, workspace_bytes);

    nq::AttentionArgs a;
    a.query = query_dev;
    a.key_codes = reinterpret_cast<const uint32_t *>(key_codes_dev);
    a.value_codes = reinterpret_cast<const uint32_t *>(value_codes_dev);
    a.key_beta_ids = key_beta_ids_dev; a.value_beta_ids = value_beta_ids_dev;
    a.key_hints = key_hints_dev; a.value_hints = value_hints_dev;
    a.key_norms = key_norms_dev; a.value_norms = value_norms_dev;
    a.key_betas = key_betas_dev; a.value_betas = value_betas_dev;
    a.page_indices = page_indices_dev; a.page_counts = page_counts_dev;
    a.last_page_lens = last_page_lens_dev; a.hot_lengths = hot_lengths_dev;
    a.cache_active = cache_active_dev;
    a.hot_keys = reinterpret_cast<const uint16_t *>(hot_keys_dev);
    a.hot_values = reinterpret_cast<const uint16_t *>(hot_values_dev);
    a.slot_ids = slot_ids_dev; a.active_mask = active_mask_dev;
    a.batch = batch; a.slots = slots; a.max_pages = max_pages; a.q_heads = q_heads; a.kv_heads = kv_heads;
    a.chunks = chunks_for(batch, max_pages); a.query_dtype = query_dtype; a.scale = scale;
    a.rotate_query = rotate_query;
    NQ_REQUIRE((rope_cos_dev == nullptr) == (rope_sin_dev == nullptr), NQ_ERR_ARGUMENT,
               "%s: rotary cos and sin tables come together", entry);
    NQ_REQUIRE(!rope_cos_dev || query_dtype == NQ_BF16, NQ_ERR_ARGUMENT,
               "%s: the fused rotary embedding takes BF16 queries", entry);
    a.rope_cos = reinterpret_cast<const uint16_t *>(rope_cos_dev);
    a.rope_sin = reinterpret_cast<const uint16_t *>(rope_sin_dev);
    a.new_key = a.new_value = nullptr;
    a.sequence_lengths = nullptr;
    a.key_beta_count = 4; a.rotate_keys = 0;
    if (append) {
        NQ_REQUIRE(append->key && append->value && append->sequence_lengths, NQ_ERR_ARGUMENT, "%s: null pointer", entry);
        NQ_REQUIRE(nq::aligned(append->key, 16) && nq::aligned(append->value, 16), NQ_ERR_ARGUMENT,
                   "%s: the new keys and values need 16-byte alignment", entry);
        NQ_REQUIRE(append->key_beta_count >= 1 && append->key_beta_count <= 4 &&
                       append->value_beta_count == append->key_beta_count,
                   NQ_ERR_SHAPE, "%s: key and value tables must hold the same number (1..4) of betas", entry);
        NQ_REQUIRE(query_dtype == NQ_BF16, NQ_ERR_ARGUMENT, "%s: a step that appends takes BF16 queries, keys and values",
                   entry);
        a.new_key = reinterpret_cast<const uint16_t *>(append->key);
        a.new_value = reinterpret_cast<const uint16_t *>(append->value);
        a.sequence_lengths = append->sequence_lengths;
        a.key_beta_count = append->key_beta_count; a.rotate_keys = append->rotate_keys;
    }
    const size_t parts = (size_t)a.chunks + 1, heads_total = (size_t)batch * q_heads;
    a.part_max = reinterpret_cast<float *>(workspace_dev);
    a.part_sum = a.part_max + heads_total * parts;
    a.part_acc = a.part_sum + heads_total * parts;

    hipStream_t s = (hipStream_t)stream;
    const size_t pairs = parts * (size_t)batch;                    // (row, chunk) pairs, padded to whole groups of eight
    const dim3 grid((unsigned)((pairs + 7) / 8 * 8 * kv_heads));
#define NQ_LAUNCH_STAGE1_AS(GROUP, PAGES, WRITES)                                                                 \
    hipLaunchKernelGGL((nq::attention_stage1_kernel<64, 16, GROUP, PAGES, WRITES>), grid, dim3(nq::kAttnThreads), 0, s, a)
#define NQ_LAUNCH_STAGE1(GROUP, WRITES)                                                                           \
    switch (pages_per_chunk_for(batch, max_pages)) {                                                              \
        case 4: NQ_LAUNCH_STAGE1_AS(GROUP, 4, WRITES); break;                                                     \
        case 8: NQ_LAUNCH_STAGE1_AS(GROUP, 8, WRITES); break;                                                     \
        default: NQ_LAUNCH_STAGE1_AS(GROUP, 16, WRITES); break;                                                   \
    }
#define NQ_LAUNCH_STAGE1_GROUPS(WRITES)                                                                           \
    switch (group) {                                                                                              \
        case 1: NQ_LAUNCH_STAGE1(1, WRITES); break;                                                               \
        case 2: NQ_LAUNCH_STAGE1(2, WRITES); break;                                                               \
        case 4: NQ_LAUNCH_STAGE1(4, WRITES); break;                                                               \
        default: NQ_LAUNCH_STAGE1(8, WRITES); break;                                                              \
    }
    if (append) { NQ_LAUNCH_STAGE1_GROUPS(true) } else { NQ_LAUNCH_STAGE1_GROUPS(false) }
#undef NQ_LAUNCH_STAGE1_GROUPS
#undef NQ_LAUNCH_STAGE1
#undef NQ_LAUNCH_STAGE1_AS
    int status = nq::check_launch(entry);
    // without an output the partial results stay in the workspace for nq_attention_output_stage
    if (status != NQ_OK || out_dev == nullptr) return status;
    hipLaunchKernelGGL(nq::attention_merge_kernel<64>, dim3((unsigned)heads_total), dim3(64), 0, s,
                       a.part_max, a.part_sum, a.part_acc, (int)parts, (int64_t)heads_total, out_dev, query_dtype);
    return nq::check_launch(entry);
}

}  // namespace

extern "C" int nq_nqkv_attention_decode(
    const void *query_dev, int query_dtype, const uint8_t *key_codes_dev, const uint8_t *key_beta_ids_dev,
    const float *key_norms_dev, const uint8_t *value_codes_dev, const uint8_t *value_beta_ids_dev,
    const float *value_norms_dev, const float *key_betas_dev, const float *value_betas_dev,
    const int32_t *page_indices_dev, const int32_t *page_counts_dev, const int32_t *last_page_lens_dev,
    const int32_t *hot_lengths_dev, const uint8_t *cache_active_dev, const void *hot_keys_dev,
    const void *hot_values_dev, const int32_t *slot_ids_dev, const uint8_t *active_mask_dev, int batch,
    int slots, int max_pages, int q_heads, int kv_heads, int head_dim, int page_size, float scale,
    int rotate_query, const void *rope_cos_dev, const void *rope_sin_dev, void *out_dev, void *workspace_dev,
    size_t workspace_bytes, const uint8_t *key_hints_dev, const uint8_t *value_hints_dev, void *stream) {
    return launch_decode_attention(
        "nq_nqkv_attention_decode", nullptr, query_dev, query_dtype, key_codes_dev, key_beta_ids_dev, key_norms_dev,
        value_codes_dev, value_beta_ids_dev, value_norms_dev, key_betas_dev, value_betas_dev, page_indices_dev,
        page_counts_dev, last_page_lens_dev, hot_lengths_dev, cache_active_dev, hot_keys_dev, hot_values_dev,
        slot_ids_dev, active_mask_dev, batch, slots, max_pages, q_heads, kv_heads, head_dim, page_size, scale,
        rotate_query, rope_cos_dev, rope_sin_dev, out_dev, workspace_dev, workspace_bytes, key_hints_dev, value_hints_dev,
        stream);
}

extern "C" int nq_nqkv_append_attention_decode(
    const void *query_dev, const void *key_dev, const void *value_dev, const int32_t *sequence_lengths_dev,
    uint8_t *key_codes_dev, uint8_t *key_beta_ids_dev, float *key_norms_dev, uint8_t *value_codes_dev,
    uint8_t *value_beta_ids_dev, float *value_norms_dev, const float *key_betas_dev, int key_beta_count,
    const float *value_betas_dev, int value_beta_count, const int32_t *page_indices_dev,
    const int32_t *page_counts_dev, const int32_t *last_page_lens_dev, const int32_t *hot_lengths_dev,
    const uint8_t *cache_active_dev, void *hot_keys_dev, void *hot_values_dev, const int32_t *slot_ids_dev,
    const uint8_t *active_mask_dev, int batch, int slots, int max_pages, int q_heads, int kv_heads, int head_dim,
    int page_size, float scale, int rotate, const void *rope_cos_dev, const void *rope_sin_dev, void *out_dev,
    void *workspace_dev, size_t workspace_bytes, uint8_t *key_hints_dev, uint8_t *value_hints_dev, void *stream) {
    const AppendOperands append{key_dev, value_dev, sequence_lengths_dev, key_beta_count, value_beta_count, rotate};
    return launch_decode_attention(
        "nq_nqkv_append_attention_decode", &append, query_dev, NQ_BF16, key_codes_dev, key_beta_ids_dev, key_norms_dev,
        value_codes_dev, value_beta_ids_dev, value_norms_dev, key_betas_dev, value_betas_dev, page_indices_dev,
        page_counts_dev, last_page_lens_dev, hot_lengths_dev, cache_active_dev, hot_keys_dev, hot_values_dev,
        slot_ids_dev, active_mask_dev, batch, slots, max_pages, q_heads, kv_heads, head_dim, page_size, scale,
        rotate, rope_cos_dev, rope_sin_dev, out_dev, workspace_dev, workspace_bytes, key_hints_dev, value_hints_dev, stream);
}
