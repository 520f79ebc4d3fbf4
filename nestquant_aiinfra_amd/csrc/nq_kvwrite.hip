// Paged ragged NQKV writer: appends new K/V rows of a ragged batch to each slot's BF16 hot
// tail and, whenever a 16-token page fills, encodes it (4-bit E8 codes, per-block beta ids,
// FP32 row norms) straight into that slot's next cold page.  Decode (one token per row) and
// prefill (any number of tokens per row, ragged) are the same launch.
//
// Metadata model (device-resident, per slot; the reference keeps the same tensors,
// nestquant/runtime/paged_nqkv_cache.py:25-95): sequence_lengths, page_counts,
// last_page_lens, hot_lengths, page_indices[slot, ordinal].  nq_nqkv_advance bumps them
// for a whole step *before* the layers run; the writer and the attention kernel of every
// layer then read them without any host round trip or per-layer metadata kernel
// (the reference launches a data kernel plus a metadata kernel per layer and reserves pages
// on the host before each boundary step, nqkv_graph_writer.py:291-332, nqkv_batch_manager.py:648-689).
//
// Writer, grid = (pages a row can touch, batch * kv_heads), 256 lanes.  With L the new
// length of the slot and c the row's token count, the row touches page ordinals
// (L - c) / 16 .. (L - 1) / 16.  A complete page is gathered in LDS as float32 (its first
// tokens may come from the hot tail, the rest from the new rows), quantised with the same
// device routine as the stand-alone encoder (bit-identical results) and stored at
// page_indices[slot, ordinal]; rows follow the NHD rule row = token * kv_heads + head
// (nestquant/core/kv_format.py:99-131).  The trailing partial page goes to the hot tail.
// Workgroup 0 of a row handles its first page and then the trailing partial page, in that
// order, so hot-tail reads precede hot-tail writes; other workgroups own one middle page.
#include "nq_rowquant.hip.h"
#include "nq_host.h"

#include <math.h>

namespace nq {

constexpr int kKvThreads = 256;

__global__ void __launch_bounds__(256)
kv_advance_kernel(const int32_t *__restrict__ slot_ids, const uint8_t *__restrict__ active_mask,
                  const int32_t *__restrict__ counts, int uniform_count, int batch, int slots, int page_size,
                  int max_tokens, int32_t *__restrict__ sequence_lengths, int32_t *__restrict__ page_counts,
                  int32_t *__restrict__ last_page_lens, int32_t *__restrict__ hot_lengths) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= batch || !active_mask[r]) return;
    const int slot = slot_ids[r];
    if (slot < 0 || slot >= slots) return;                       // a stale replay writes nothing
    int count = counts ? counts[r] : uniform_count;
    int length = sequence_lengths[slot];
    if (count < 0) count = 0;
    if (length + count > max_tokens) count = max_tokens - length; // clamp at capacity
    length += count;
    sequence_lengths[slot] = length;
    page_counts[slot] = length / page_size;
    last_page_lens[slot] = length >= page_size ? page_size : 0;
    hot_lengths[slot] = length % page_size;
}

// One launch at the head of a step that writes prompts: workgroup r takes row r of `record` (the host's
// description of the step: slot, tokens to write, whether the slot starts a new sequence), resets a new
// sequence's tables, leaves the step's row state where the writer and the attention read it, fills the
// row's positions and the index of its last token, and advances the slot's tables as kv_advance_kernel.
struct PromptBeginArgs {
    const int32_t *record;          // [3][batch]: slot, count, fresh
    int batch, width, slots, page_size, max_tokens;
    int32_t *step_slot_ids, *step_counts;
    uint8_t *step_active;
    int32_t *sequence_lengths, *page_counts, *last_page_lens, *hot_lengths;
    uint8_t *cache_active;
    int64_t *positions;             // [batch][width], or null
    int64_t *last_token;            // [batch], or null
};

__global__ void __launch_bounds__(256) prompt_begin_kernel(PromptBeginArgs a) {
    const int r = blockIdx.x, tid = threadIdx.x;
    const int slot = a.record[r];
    int count = a.record[a.batch + r];
    const bool fresh = a.record[2 * a.batch + r] != 0;
    const bool known = slot >= 0 && slot < a.slots;
    if (count < 0) count = 0;
    if (count > a.width) count = a.width;
    // every lane reads the length before lane 0 stores the new one (a new sequence starts at zero)
    const int start = known && !fresh ? a.sequence_lengths[slot] : 0;
    __syncthreads();
    if (a.positions)
        for (int c = tid; c < a.width; c += blockDim.x) a.positions[(int64_t)r * a.width + c] = (int64_t)start + c;
    if (tid != 0) return;
    a.step_slot_ids[r] = slot;
    a.step_counts[r] = count;
    a.step_active[r] = count > 0;
    if (a.last_token) a.last_token[r] = count > 0 ? count - 1 : 0;
    if (!known) return;
    if (fresh) a.cache_active[slot] = 1;
    if (!fresh && count == 0) return;
    int length = start;
    if (length + count > a.max_tokens) count = a.max_tokens - length;   // clamp at capacity
    length += count;
    a.sequence_lengths[slot] = length;
    a.page_counts[slot] = length / a.page_size;
    a.last_page_lens[slot] = length >= a.page_size ? a.page_size : 0;
    a.hot_lengths[slot] = length % a.page_size;
}

// One launch at the head of a decode step: workgroup r advances row r's tables by one token
// (as kv_advance_kernel), copies the embedding row of its input token and the rotary
// embedding's cos and sin rows of its position.
struct StepBeginArgs {
    const int32_t *slot_ids;
    const uint8_t *active_mask;
    int batch, slots, page_size, max_tokens;
    int32_t *sequence_lengths, *page_counts, *last_page_lens, *hot_lengths;
    const int64_t *tokens;          // [batch]
    const uint4 *embedding;         // BF16 [vocab][hidden]
    uint4 *embedded;                // BF16 [batch][hidden]
    int64_t vocab;
    int hidden_vectors;             // hidden / 8
    const int64_t *positions;       // [batch]
    const uint4 *rotary;            // BF16 [2][rotary_positions][rotary_vectors * 8]: cos rows, then sin rows
    uint4 *rotary_rows;             // BF16 [2][batch][rotary_vectors * 8]
    int64_t rotary_positions;
    int rotary_vectors;             // head_dim / 8
};

__global__ void __launch_bounds__(256) decode_step_begin_kernel(StepBeginArgs a) {
    const int r = blockIdx.x, tid = threadIdx.x;
    const int64_t token = a.tokens[r];
    const bool known = token >= 0 && token < a.vocab;                  // an unknown token embeds as zero
    const uint4 *source = a.embedding + (known ? token : 0) * a.hidden_vectors;
    for (int v = tid; v < a.hidden_vectors; v += blockDim.x) {
        const uint4 value = source[v];
        a.embedded[(int64_t)r * a.hidden_vectors + v] = known ? value : make_uint4(0, 0, 0, 0);
    }
    if (tid < 2 * a.rotary_vectors) {
        int64_t position = a.positions[r];
        position = position < 0 ? 0 : (position >= a.rotary_positions ? a.rotary_positions - 1 : position);
        const int side = tid / a.rotary_vectors, v = tid % a.rotary_vectors;
        a.rotary_rows[((int64_t)side * a.batch + r) * a.rotary_vectors + v] =
            a.rotary[((int64_t)side * a.rotary_positions + position) * a.rotary_vectors + v];
    }
    if (tid != 0 || !a.active_mask[r]) return;
    const int slot = a.slot_ids[r];
    if (slot < 0 || slot >= a.slots) return;                          // a stale replay writes nothing
    int length = a.sequence_lengths[slot];
    if (length < a.max_tokens) length += 1;                           // clamp at capacity
    a.sequence_lengths[slot] = length;
    a.page_counts[slot] = length / a.page_size;
    a.last_page_lens[slot] = length >= a.page_size ? a.page_size : 0;
    a.hot_lengths[slot] = length % a.page_size;
}

struct KvWriteArgs {
    const uint16_t *key, *value;            // BF16 [batch, tokens, kv_heads, D]
    const int32_t *slot_ids, *counts;       // counts may be null (uniform_count)
    const uint8_t *active_mask;
    const int32_t *sequence_lengths, *page_indices;
    uint32_t *key_codes, *value_codes;
    uint8_t *key_beta_ids, *value_beta_ids;
    float *key_norms, *value_norms;
    const float *key_betas, *value_betas;
    uint16_t *hot_keys, *hot_values;        // BF16 [slots, P, kv_heads, D]
    const uint16_t *rope_cos, *rope_sin;    // optional BF16 [batch, tokens, D]: rotary embedding of the new keys
    uint8_t *key_hints, *value_hints;       // optional [pages][P * kv_heads * D / 16]: decode hints, two blocks per byte
    int batch, tokens, uniform_count, slots, max_pages, kv_heads, key_beta_count, value_beta_count, rotate_keys;
};

// kPairs: one lane per (block, beta) pair on 4 x 256 lanes instead of one lane per block with its betas in
// turn: three times the lanes for a third of a lane's instructions, the same bits.  A launch of few
// workgroups (the pages of one short prompt) is bound by the length of that chain, a launch of many
// by the instructions in all.
template <int D, int P, bool kPairs>
__global__ void __launch_bounds__(kPairs ? 4 * kKvThreads : kKvThreads) kv_write_kernel(KvWriteArgs a) {
    constexpr int kThreads = kPairs ? 4 * kKvThreads : kKvThreads;
    constexpr int kBlocks = D / 8;
    __shared__ float rows[2 * P][D];             // K tokens 0..P-1, then V tokens
    __shared__ float row_scale[2 * P], row_norm[2 * P];
    const int tid = threadIdx.x;
    const int row = blockIdx.y / a.kv_heads, g = blockIdx.y % a.kv_heads;
    if (!a.active_mask[row]) return;
    const int slot = a.slot_ids[row];
    if (slot < 0 || slot >= a.slots) return;
    int count = a.counts ? a.counts[row] : a.uniform_count;
    const int length = a.sequence_lengths[slot];             // already includes this step
    if (count > a.tokens) count = a.tokens;
    if (count > length) count = length;
    if (count <= 0) return;
    const int start = length - count;
    const int first_ordinal = start / P, last_ordinal = (length - 1) / P;
    const bool tail_partial = (length % P) != 0;

    const float sqrt_d = __builtin_sqrtf((float)D);
    const int64_t page_words = (int64_t)P * a.kv_heads * kBlocks, page_rows = (int64_t)P * a.kv_heads;

    // this workgroup's pages: blockIdx.x-th touched page; workgroup 0 also takes the trailing
    // partial page when that is a different page
    for (int turn = 0; turn < 2; turn++) {
        int ordinal;
        if (turn == 0) {
            ordinal = first_ordinal + (int)blockIdx.x;
            if (ordinal > last_ordinal) return;
            if (blockIdx.x != 0 && ordinal == last_ordinal && tail_partial) return;   // workgroup 0 does it
        } else {
            if (blockIdx.x != 0 || !tail_partial || last_ordinal == first_ordinal) return;
            ordinal = last_ordinal;
            __syncthreads();                 // the first page's LDS rows are done with
        }
        const int page_start = ordinal * P;
        const bool complete = page_start + P <= length;
        const int page_tokens = complete ? P : length - page_start;      // tokens of this page that exist
        const int first_new = start > page_start ? start - page_start : 0;
        // stage the page's tokens as float32: hot tail first, then the new rows
        for (int i = tid; i < 2 * P * (D / 8); i += kThreads) {
            const int which = i / (P * (D / 8)), rem = i % (P * (D / 8));
            const int t = rem / (D / 8), c = rem % (D / 8);
            float *dst = &rows[which * P + t][c * 8];
            if (t >= page_tokens) {
#pragma unroll
                for (int j = 0; j < 8; j++) dst[j] = 0.0f;
                continue;
            }
            const uint16_t *src;
            if (t < first_new)
                src = (which ? a.hot_values : a.hot_keys) + (((int64_t)slot * P + t) * a.kv_heads + g) * D + c * 8;
            else
                src = (which ? a.value : a.key) +
                      (((int64_t)row * a.tokens + (page_start + t - start)) * a.kv_heads + g) * D + c * 8;
            const uint4 raw = *reinterpret_cast<const uint4 *>(src);
            dst[0] = __uint_as_float(raw.x << 16); dst[1] = __uint_as_float(raw.x & 0xffff0000u);
            dst[2] = __uint_as_float(raw.y << 16); dst[3] = __uint_as_float(raw.y & 0xffff0000u);
            dst[4] = __uint_as_float(raw.z << 16); dst[5] = __uint_as_float(raw.z & 0xffff0000u);
            dst[6] = __uint_as_float(raw.w << 16); dst[7] = __uint_as_float(raw.w & 0xffff0000u);
        }
        __syncthreads();
        if (a.rope_cos) {
            // rotary position embedding of the new key rows in BF16 tensor arithmetic:
            // (k * cos) + (rotate_half(k) * sin), every product and the sum rounded to BF16
            const int new_rows = page_tokens - first_new;
            for (int i = tid; i < new_rows * (D / 2); i += kThreads) {
                const int r = first_new + i / (D / 2), k = i % (D / 2);
                const int64_t at = ((int64_t)row * a.tokens + (page_start + r - start)) * D;
                const float c_lo = bf16_to_f32(a.rope_cos[at + k]), c_hi = bf16_to_f32(a.rope_cos[at + k + D / 2]);
                const float s_lo = bf16_to_f32(a.rope_sin[at + k]), s_hi = bf16_to_f32(a.rope_sin[at + k + D / 2]);
                const float x1 = rows[r][k], x2 = rows[r][k + D / 2];
                rows[r][k] = bf16_to_f32(f32_to_bf16(bf16_to_f32(f32_to_bf16(x1 * c_lo)) - bf16_to_f32(f32_to_bf16(x2 * s_lo))));
                rows[r][k + D / 2] = bf16_to_f32(f32_to_bf16(bf16_to_f32(f32_to_bf16(x2 * c_hi)) + bf16_to_f32(f32_to_bf16(x1 * s_hi))));
            }
            __syncthreads();
        }
        if (a.rotate_keys) {
            // new key rows arrive unrotated: float32 Hadamard over the head, then BF16, as
            // hadamard(key.float()).to(bfloat16) (nestquant/runtime/nqkv_batched_hf_backend.py:381)
            const int new_rows = page_tokens - first_new;
            for (int width = 1; width < D; width <<= 1) {
                for (int i = tid; i < new_rows * (D / 2); i += kThreads) {
                    const int r = first_new + i / (D / 2), k = i % (D / 2);
                    const int x = (k / width) * 2 * width + (k % width), y = x + width;
                    const float left = rows[r][x], right = rows[r][y];
                    rows[r][x] = left + right;
                    rows[r][y] = left - right;
                }
                __syncthreads();
            }
            const float inv = 1.0f / sqrt_d;
            for (int i = tid; i < new_rows * D; i += kThreads) {
                float &v = rows[first_new + i / D][i % D];
                v = bf16_to_f32(f32_to_bf16(v * inv));
            }
            __syncthreads();
        }
        if (!complete) {
            // trailing partial page: the new rows of this head go to the hot tail
            for (int i = tid; i < 2 * (page_tokens - first_new) * (D / 8); i += kThreads) {
                const int which = i / ((page_tokens - first_new) * (D / 8)), rem = i % ((page_tokens - first_new) * (D / 8));
                const int t = first_new + rem / (D / 8), c = rem % (D / 8);
                const float *src = &rows[which * P + t][c * 8];
                uint4 packed;
                packed.x = f32_to_bf16(src[0]) | ((uint32_t)f32_to_bf16(src[1]) << 16);
                packed.y = f32_to_bf16(src[2]) | ((uint32_t)f32_to_bf16(src[3]) << 16);
                packed.z = f32_to_bf16(src[4]) | ((uint32_t)f32_to_bf16(src[5]) << 16);
                packed.w = f32_to_bf16(src[6]) | ((uint32_t)f32_to_bf16(src[7]) << 16);
                *reinterpret_cast<uint4 *>((which ? a.hot_values : a.hot_keys) +
                                           (((int64_t)slot * P + t) * a.kv_heads + g) * D + c * 8) = packed;
            }
            continue;
        }
        __syncthreads();
        staged_row_norms(&rows[0][0], 2 * P, D, sqrt_d, row_scale, row_norm);
        const int64_t page = a.page_indices[(int64_t)slot * a.max_pages + ordinal];
        if (page < 0) continue;                  // ordinal not mapped to a physical page: nothing to write to
        if (tid < 2 * P) {
            const int t = tid % P;
            (tid < P ? a.key_norms : a.value_norms)[page * page_rows + t * a.kv_heads + g] = row_norm[tid];
        }
        struct Sink {
            uint32_t *key_codes, *value_codes; uint8_t *key_beta_ids, *value_beta_ids;
            int64_t page_word0; int kv_heads, g;
            __device__ __forceinline__ bool wants(int) const { return true; }
            __device__ __forceinline__ int64_t word(int r, int b) const {
                return page_word0 + ((int64_t)(r % P) * kv_heads + g) * kBlocks + b;
            }
            __device__ __forceinline__ void code(int r, int b, uint32_t w, const float (&)[8], float) const {
                (r < P ? key_codes : value_codes)[word(r, b)] = w;
            }
            __device__ __forceinline__ void beta_byte(int r, int b, uint32_t byte) const {
                (r < P ? key_beta_ids : value_beta_ids)[word(r, b) >> 2] = (uint8_t)byte;
            }
            __device__ __forceinline__ uint32_t counter(int, int) const { return 0u; }
        } sink{a.key_codes, a.value_codes, a.key_beta_ids, a.value_beta_ids, page * page_words, a.kv_heads, g};
        struct Betas {
            const float *key, *value;
            __device__ __forceinline__ const float *operator()(int r) const { return r < P ? key : value; }
        } betas_of{a.key_betas, a.value_betas};
        // one lane per block, its betas in turn (the 2 P x 8 blocks of the page's key and value rows are the
        // workgroup's 256 lanes; a wavefront holds rows of one kind): fewer instructions per block than
        // a lane per (block, beta) pair, which is what a many-page prompt pays for
        if (kPairs)
            quantize_staged_pairs<false>(&rows[0][0], row_scale, D, 14.0f, 1.0f / 14.0f, betas_of, a.key_beta_count, 0u,
                                         0, 2 * P * kBlocks * 4, sink);
        else
            quantize_staged_blocks(&rows[0][0], row_scale, D, 14.0f, 1.0f / 14.0f, betas_of, a.key_beta_count, 0,
                                   2 * P * kBlocks, sink);
        if (a.key_hints) {
            // the decode hints of the page's blocks, from the code words this workgroup has just stored
            __syncthreads();
            for (int i = tid; i < 2 * P * (kBlocks / 2); i += kThreads) {
                const int which = i / (P * (kBlocks / 2)), rem = i % (P * (kBlocks / 2));
                const int64_t word = sink.word(rem / (kBlocks / 2), 2 * (rem % (kBlocks / 2)));
                const uint2 pair = *reinterpret_cast<const uint2 *>((which ? a.value_codes : a.key_codes) + word);
                (which ? a.value_hints : a.key_hints)[word >> 1] =
                    (uint8_t)(hint_of_codeword(pair.x) | (hint_of_codeword(pair.y) << 4));
            }
        }
    }
}

// Decode hints of a stream of undithered code words (a page brought in from a container, a test).
__global__ void __launch_bounds__(256) page_hints_kernel(const uint2 *__restrict__ codes, int64_t pairs, uint8_t *__restrict__ hints) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= pairs) return;
    const uint2 pair = codes[i];
    hints[i] = (uint8_t)(hint_of_codeword(pair.x) | (hint_of_codeword(pair.y) << 4));
}

// Every code word with digits below 14 whose index lies in [first, first + count): the hinted decode
// against the plain one; mismatching blocks are counted.
__global__ void __launch_bounds__(256) verify_hints_kernel(int64_t first, int64_t count, unsigned long long *mismatches) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    int64_t index = first + i;
    uint32_t word = 0u;
#pragma unroll
    for (int j = 0; j < 8; j++) { word |= (uint32_t)(index % 14) << (4 * j); index /= 14; }
    float plain[8], hinted[8];
    decode_codeword<false>(word, 14.0f, 0u, plain);
    decode_codeword_hinted(word, hint_of_codeword(word), hinted);
    bool same = true;
#pragma unroll
    for (int j = 0; j < 8; j++) same = same && __float_as_uint(plain[j]) == __float_as_uint(hinted[j]);
    if (!same) atomicAdd(mismatches, 1ull);
}

}  // namespace nq

extern "C" int nq_nqkv_advance(const int32_t *slot_ids_dev, const uint8_t *active_mask_dev,
                               const int32_t *counts_dev, int uniform_count, int batch, int slots,
                               int page_size, int max_tokens, int32_t *sequence_lengths_dev,
                               int32_t *page_counts_dev, int32_t *last_page_lens_dev,
                               int32_t *hot_lengths_dev, void *stream) {
    NQ_REQUIRE(batch >= 1 && slots >= 1 && page_size >= 1 && max_tokens >= 1, NQ_ERR_SHAPE,
               "nq_nqkv_advance: batch, slots, page_size and max_tokens must be positive");
    NQ_REQUIRE(slot_ids_dev && active_mask_dev && sequence_lengths_dev && page_counts_dev && last_page_lens_dev &&
                   hot_lengths_dev,
               NQ_ERR_ARGUMENT, "nq_nqkv_advance: null pointer");
    NQ_REQUIRE(counts_dev || uniform_count >= 0, NQ_ERR_ARGUMENT, "nq_nqkv_advance: negative token count");
    hipLaunchKernelGGL(nq::kv_advance_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       slot_ids_dev, active_mask_dev, counts_dev, uniform_count, batch, slots, page_size, max_tokens,
                       sequence_lengths_dev, page_counts_dev, last_page_lens_dev, hot_lengths_dev);
    return nq::check_launch("nq_nqkv_advance");
}

extern "C" int nq_prompt_step_begin(const int32_t *record_dev, int batch, int width, int slots, int page_size,
                                    int max_tokens, int32_t *step_slot_ids_dev, int32_t *step_counts_dev,
                                    uint8_t *step_active_dev, int32_t *sequence_lengths_dev, int32_t *page_counts_dev,
                                    int32_t *last_page_lens_dev, int32_t *hot_lengths_dev, uint8_t *cache_active_dev,
                                    int64_t *positions_dev, int64_t *last_token_dev, void *stream) {
    NQ_REQUIRE(batch >= 1 && batch <= 65535 && width >= 1 && slots >= 1 && page_size >= 1 && max_tokens >= 1,
               NQ_ERR_SHAPE,
               "nq_prompt_step_begin: batch (at most 65535), width, slots, page_size and max_tokens must be positive");
    NQ_REQUIRE(record_dev && step_slot_ids_dev && step_counts_dev && step_active_dev && sequence_lengths_dev &&
                   page_counts_dev && last_page_lens_dev && hot_lengths_dev && cache_active_dev,
               NQ_ERR_ARGUMENT, "nq_prompt_step_begin: null pointer");
    nq::PromptBeginArgs a;
    a.record = record_dev;
    a.batch = batch; a.width = width; a.slots = slots; a.page_size = page_size; a.max_tokens = max_tokens;
    a.step_slot_ids = step_slot_ids_dev; a.step_counts = step_counts_dev; a.step_active = step_active_dev;
    a.sequence_lengths = sequence_lengths_dev; a.page_counts = page_counts_dev;
    a.last_page_lens = last_page_lens_dev; a.hot_lengths = hot_lengths_dev; a.cache_active = cache_active_dev;
    a.positions = positions_dev; a.last_token = last_token_dev;
    hipLaunchKernelGGL(nq::prompt_begin_kernel, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream, a);
    return nq::check_launch("nq_prompt_step_begin");
}

extern "C" int nq_decode_step_begin(const int32_t *slot_ids_dev, const uint8_t *active_mask_dev, int batch, int slots,
                                    int page_size, int max_tokens, int32_t *sequence_lengths_dev,
                                    int32_t *page_counts_dev, int32_t *last_page_lens_dev, int32_t *hot_lengths_dev,
                                    const int64_t *tokens_dev, const void *embedding_bf16_dev, int64_t vocab,
                                    int hidden, void *embedded_bf16_dev, const int64_t *positions_dev,
                                    const void *rotary_bf16_dev, int64_t rotary_positions, int head_dim,
                                    void *rotary_rows_bf16_dev, void *stream) {
    NQ_REQUIRE(batch >= 1 && batch <= 65535 && slots >= 1 && page_size >= 1 && max_tokens >= 1, NQ_ERR_SHAPE,
               "nq_decode_step_begin: batch (at most 65535), slots, page_size and max_tokens must be positive");
    NQ_REQUIRE(vocab >= 1 && hidden >= 8 && hidden % 8 == 0 && rotary_positions >= 1 && head_dim >= 8 &&
                   head_dim % 8 == 0 && head_dim <= 1024,
               NQ_ERR_SHAPE, "nq_decode_step_begin: hidden and head_dim (at most 1024) must be positive multiples of 8");
    NQ_REQUIRE(slot_ids_dev && active_mask_dev && sequence_lengths_dev && page_counts_dev && last_page_lens_dev &&
                   hot_lengths_dev && tokens_dev && embedding_bf16_dev && embedded_bf16_dev && positions_dev &&
                   rotary_bf16_dev && rotary_rows_bf16_dev,
               NQ_ERR_ARGUMENT, "nq_decode_step_begin: null pointer");
    NQ_REQUIRE(nq::aligned(embedding_bf16_dev, 16) && nq::aligned(embedded_bf16_dev, 16) &&
                   nq::aligned(rotary_bf16_dev, 16) && nq::aligned(rotary_rows_bf16_dev, 16),
               NQ_ERR_ARGUMENT, "nq_decode_step_begin: tables and outputs must be 16-byte aligned");
    nq::StepBeginArgs a;
    a.slot_ids = slot_ids_dev; a.active_mask = active_mask_dev;
    a.batch = batch; a.slots = slots; a.page_size = page_size; a.max_tokens = max_tokens;
    a.sequence_lengths = sequence_lengths_dev; a.page_counts = page_counts_dev;
    a.last_page_lens = last_page_lens_dev; a.hot_lengths = hot_lengths_dev;
    a.tokens = tokens_dev;
    a.embedding = reinterpret_cast<const uint4 *>(embedding_bf16_dev);
    a.embedded = reinterpret_cast<uint4 *>(embedded_bf16_dev);
    a.vocab = vocab; a.hidden_vectors = hidden / 8;
    a.positions = positions_dev;
    a.rotary = reinterpret_cast<const uint4 *>(rotary_bf16_dev);
    a.rotary_rows = reinterpret_cast<uint4 *>(rotary_rows_bf16_dev);
    a.rotary_positions = rotary_positions; a.rotary_vectors = head_dim / 8;
    hipLaunchKernelGGL(nq::decode_step_begin_kernel, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream, a);
    return nq::check_launch("nq_decode_step_begin");
}

extern "C" int nq_nqkv_write(const void *key_dev, const void *value_dev, int kv_dtype, const int32_t *slot_ids_dev,
                             const uint8_t *active_mask_dev, const int32_t *counts_dev, int uniform_count,
                             const int32_t *sequence_lengths_dev, const int32_t *page_indices_dev,
                             uint8_t *key_codes_dev, uint8_t *key_beta_ids_dev, float *key_norms_dev,
                             uint8_t *value_codes_dev, uint8_t *value_beta_ids_dev, float *value_norms_dev,
                             const float *key_betas_dev, int key_beta_count, const float *value_betas_dev,
                             int value_beta_count, void *hot_keys_dev, void *hot_values_dev, int batch, int tokens,
                             int slots, int max_pages, int kv_heads, int head_dim, int page_size, int rotate_keys,
                             const void *rope_cos_dev, const void *rope_sin_dev, uint8_t *key_hints_dev,
                             uint8_t *value_hints_dev, void *stream) {
    NQ_REQUIRE(batch >= 1 && tokens >= 1 && slots >= 1 && max_pages >= 1 && kv_heads >= 1, NQ_ERR_SHAPE,
               "nq_nqkv_write: batch, tokens, slots, max_pages and kv_heads must be positive");
    NQ_REQUIRE((key_hints_dev == nullptr) == (value_hints_dev == nullptr), NQ_ERR_ARGUMENT,
               "nq_nqkv_write: key and value hint streams come together");
    NQ_REQUIRE(!key_hints_dev || (nq::aligned(key_codes_dev, 8) && nq::aligned(value_codes_dev, 8)), NQ_ERR_ARGUMENT,
               "nq_nqkv_write: with hint streams the code streams need 8-byte alignment");
    NQ_REQUIRE(head_dim == 64 && page_size == 16, NQ_ERR_SHAPE,
               "nq_nqkv_write: built for head_dim 64 and 16-token pages (got %d, %d)", head_dim, page_size);
    NQ_REQUIRE(kv_dtype == NQ_BF16, NQ_ERR_ARGUMENT, "nq_nqkv_write: keys and values must be BF16");
    NQ_REQUIRE(key_beta_count >= 1 && key_beta_count <= 4 && value_beta_count == key_beta_count, NQ_ERR_SHAPE,
               "nq_nqkv_write: key and value tables must hold the same number (1..4) of betas");
    NQ_REQUIRE(key_dev && value_dev && slot_ids_dev && active_mask_dev && sequence_lengths_dev && page_indices_dev &&
                   key_codes_dev && key_beta_ids_dev && key_norms_dev && value_codes_dev && value_beta_ids_dev &&
                   value_norms_dev && key_betas_dev && value_betas_dev && hot_keys_dev && hot_values_dev,
               NQ_ERR_ARGUMENT, "nq_nqkv_write: null pointer");
    NQ_REQUIRE(nq::aligned(key_dev, 16) && nq::aligned(value_dev, 16) && nq::aligned(hot_keys_dev, 16) &&
                   nq::aligned(hot_values_dev, 16) && nq::aligned(key_codes_dev, 4) && nq::aligned(value_codes_dev, 4),
               NQ_ERR_ARGUMENT, "nq_nqkv_write: K/V and hot tails need 16-byte, code streams 4-byte alignment");
    NQ_REQUIRE(counts_dev || (uniform_count >= 0 && uniform_count <= tokens), NQ_ERR_ARGUMENT,
               "nq_nqkv_write: uniform token count %d is outside [0, %d]", uniform_count, tokens);
    nq::KvWriteArgs a;
    a.key = reinterpret_cast<const uint16_t *>(key_dev);
    a.value = reinterpret_cast<const uint16_t *>(value_dev);
    a.slot_ids = slot_ids_dev; a.counts = counts_dev; a.active_mask = active_mask_dev;
    a.sequence_lengths = sequence_lengths_dev; a.page_indices = page_indices_dev;
    a.key_codes = reinterpret_cast<uint32_t *>(key_codes_dev);
    a.value_codes = reinterpret_cast<uint32_t *>(value_codes_dev);
    a.key_beta_ids = key_beta_ids_dev; a.value_beta_ids = value_beta_ids_dev;
    a.key_norms = key_norms_dev; a.value_norms = value_norms_dev;
    a.key_betas = key_betas_dev; a.value_betas = value_betas_dev;
    a.hot_keys = reinterpret_cast<uint16_t *>(hot_keys_dev);
    a.hot_values = reinterpret_cast<uint16_t *>(hot_values_dev);
    a.batch = batch; a.tokens = tokens; a.uniform_count = uniform_count; a.slots = slots; a.max_pages = max_pages;
    a.kv_heads = kv_heads; a.key_beta_count = key_beta_count; a.value_beta_count = value_beta_count;
    a.rotate_keys = rotate_keys;
    NQ_REQUIRE((rope_cos_dev == nullptr) == (rope_sin_dev == nullptr), NQ_ERR_ARGUMENT,
               "nq_nqkv_write: rotary cos and sin tables come together");
    a.rope_cos = reinterpret_cast<const uint16_t *>(rope_cos_dev);
    a.rope_sin = reinterpret_cast<const uint16_t *>(rope_sin_dev);
    a.key_hints = key_hints_dev; a.value_hints = value_hints_dev;
    // `tokens` new rows starting anywhere inside a page touch at most this many pages
    const int touched = (tokens + page_size - 2) / page_size + 1;
    // up to two workgroups per compute unit: the launch waits for one workgroup's chain of instructions
    if ((int64_t)touched * batch * kv_heads <= 512 && key_beta_count <= 4 && value_beta_count <= 4)
        hipLaunchKernelGGL((nq::kv_write_kernel<64, 16, true>), dim3((unsigned)touched, (unsigned)(batch * kv_heads)),
                           dim3(4 * nq::kKvThreads), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((nq::kv_write_kernel<64, 16, false>), dim3((unsigned)touched, (unsigned)(batch * kv_heads)),
                           dim3(nq::kKvThreads), 0, (hipStream_t)stream, a);
    return nq::check_launch("nq_nqkv_write");
}

extern "C" int nq_nqkv_page_hints(const uint8_t *codes_dev, int64_t blocks, uint8_t *hints_dev, void *stream) {
    NQ_REQUIRE(blocks >= 0 && blocks % 2 == 0, NQ_ERR_SHAPE, "nq_nqkv_page_hints: an even number of blocks (two per hint byte)");
    if (blocks == 0) return NQ_OK;
    NQ_REQUIRE(codes_dev && hints_dev && nq::aligned(codes_dev, 8), NQ_ERR_ARGUMENT,
               "nq_nqkv_page_hints: needs the code words (8-byte aligned) and the hint bytes");
    const int64_t pairs = blocks / 2, grid = (pairs + 255) / 256;
    NQ_REQUIRE(grid <= 0x7fffffff, NQ_ERR_SHAPE, "nq_nqkv_page_hints: too many blocks");
    hipLaunchKernelGGL(nq::page_hints_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<const uint2 *>(codes_dev), pairs, hints_dev);
    return nq::check_launch("nq_nqkv_page_hints");
}

extern "C" int nq_nqkv_verify_hints(int64_t first, int64_t count, uint64_t *mismatches_dev, void *stream) {
    const int64_t all = 14ll * 14 * 14 * 14 * 14 * 14 * 14 * 14;
    NQ_REQUIRE(first >= 0 && count >= 1 && first + count <= all, NQ_ERR_SHAPE,
               "nq_nqkv_verify_hints: the range must lie inside the 14^8 code words");
    NQ_REQUIRE(mismatches_dev && nq::aligned(mismatches_dev, 8), NQ_ERR_ARGUMENT, "nq_nqkv_verify_hints: needs the counter");
    const int64_t grid = (count + 255) / 256;
    NQ_REQUIRE(grid <= 0x7fffffff, NQ_ERR_SHAPE, "nq_nqkv_verify_hints: at most 2^31 workgroups of 256 code words per call");
    hipLaunchKernelGGL(nq::verify_hints_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, first, count,
                       reinterpret_cast<unsigned long long *>(mismatches_dev));
    return nq::check_launch("nq_nqkv_verify_hints");
}
