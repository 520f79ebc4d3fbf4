"""GPU parity of the NQKV4 cache path through the C ABI: page encoder, ragged writer
(hot tails + page packing) and batched decode attention, against the CPU oracle and the
reference's golden page.

Bars: packed page bytes, beta ids and norms bit-exact; hot tails bit-exact copies;
attention max |out - ref| / max |ref| <= 1e-2 against dense softmax attention over the
oracle-dequantised cache (the reference accepts atol 2e-2 between its kernels and its
oracle, tests/unit/runtime/test_nqkv_attention_k1.py:44-67)."""

import numpy as np
import pytest
import torch

from conftest import KEY_BETAS, Q, VALUE_BETAS
from gpu_util import bits, relative_error

pytestmark = pytest.mark.gpu

HEADS, DIM, PAGE = 8, 64, 16


@pytest.fixture(scope="module")
def kv():
    from nestquant_aiinfra_amd.runtime import nqkv
    return nqkv


def _bf16(x: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(x).to(torch.bfloat16)


def _f32(t: torch.Tensor) -> np.ndarray:
    return t.float().cpu().numpy()


def test_page_encoder_matches_reference_golden(kv, golden):
    key = torch.from_numpy(golden["kv_key_bf16_bits"]).view(torch.bfloat16).cuda()
    value = torch.from_numpy(golden["kv_value_bf16_bits"]).view(torch.bfloat16).cuda()
    page = kv.quantize_nqkv_page_cuda(key, value, page_size=PAGE, q=Q, key_betas=KEY_BETAS, value_betas=VALUE_BETAS)
    for ours, name in ((page.key_code_payload, "kv_key_codes"), (page.key_beta_payload, "kv_key_betas"),
                       (page.key_norms, "kv_key_norms"), (page.value_code_payload, "kv_value_codes"),
                       (page.value_beta_payload, "kv_value_betas"), (page.value_norms, "kv_value_norms")):
        assert np.array_equal(bits(ours), golden[name]), name
    assert page.payload_bytes == 9728
    dk, dv = kv.dequantize_nqkv_page(page, output_dtype=torch.float32)
    assert np.array_equal(bits(dk), golden["kv_key_deq"]) and np.array_equal(bits(dv), golden["kv_value_deq"])
    # a partially filled page: zero-padded rows, legacy shared table
    partial = kv.quantize_nqkv_page_cuda(key[:5], value[:5], page_size=PAGE, q=Q, betas=KEY_BETAS)
    assert np.array_equal(bits(partial.key_code_payload), golden["kv_partial_key_codes"])
    assert np.array_equal(bits(partial.key_norms), golden["kv_partial_key_norms"])
    dk, _ = kv.dequantize_nqkv_page(partial)
    assert tuple(dk.shape) == (5, HEADS, DIM) and dk.dtype == torch.bfloat16


def _manager(kv, capacity, max_len, layers=1):
    return kv.BatchedNQKVCacheManager(capacity=capacity, num_layers=layers, num_kv_heads=HEADS, head_dim=DIM,
                                      max_cache_len=max_len, page_size=PAGE, q=Q, key_betas=KEY_BETAS,
                                      value_betas=VALUE_BETAS, dtype=torch.bfloat16, device="cuda")


def _append(manager, slots, keys, values, layer=0):
    """Append ragged rows: keys[i] is [count_i, HEADS, DIM] BF16 for slot slots[i]."""
    rows = len(slots)
    counts = [k.shape[0] for k in keys]
    width = max(counts)
    key = torch.zeros((rows, width, HEADS, DIM), dtype=torch.bfloat16)
    value = torch.zeros_like(key)
    for i, (k, v) in enumerate(zip(keys, values)):
        key[i, : k.shape[0]], value[i, : v.shape[0]] = k, v
    manager.step_slot_ids[:rows] = torch.tensor(slots, dtype=torch.int32)
    manager.step_active[:rows] = True
    manager.step_counts[:rows] = torch.tensor(counts, dtype=torch.int32)
    uniform = counts[0] if len(set(counts)) == 1 else None
    manager.begin_step(rows=rows, uniform_count=uniform)
    for index in ([layer] if isinstance(layer, int) else layer):
        manager.write_layer(index, key.cuda(), value.cuda())


def _check_cache(kv, oracle, manager, slot, key_all, value_all, layer=0):
    """Every cold page equals the oracle's encoding of its 16 tokens; the hot tail holds the rest."""
    cache = manager.layers[layer]
    total = key_all.shape[0]
    assert manager.total_tokens(slot) == total
    meta = manager.metadata
    assert int(meta.page_counts[slot]) == total // PAGE and int(meta.hot_lengths[slot]) == total % PAGE
    for ordinal in range(total // PAGE):
        page_id = int(meta.page_indices[slot, ordinal])
        chunk = slice(ordinal * PAGE, (ordinal + 1) * PAGE)
        expect = oracle.nqkv_page_payload(_f32(key_all[chunk]), _f32(value_all[chunk]), page_size=PAGE, q=Q,
                                          key_betas=KEY_BETAS, value_betas=VALUE_BETAS)
        pool = cache.pool
        for ours, name in ((pool.key_codes, "key_codes"), (pool.key_betas, "key_betas"), (pool.key_norms, "key_norms"),
                           (pool.value_codes, "value_codes"), (pool.value_betas, "value_betas"),
                           (pool.value_norms, "value_norms")):
            assert np.array_equal(bits(ours[page_id]), expect[name]), (slot, ordinal, name)
    hot = total % PAGE
    if hot:
        assert torch.equal(cache.hot_keys[slot, :hot].cpu(), key_all[total - hot:])
        assert torch.equal(cache.hot_values[slot, :hot].cpu(), value_all[total - hot:])


def test_ragged_writer_packs_pages_bit_exactly(kv, oracle):
    rng = np.random.default_rng(11)
    manager = _manager(kv, capacity=4, max_len=256, layers=2)
    slots = [3, 0, 2]                                   # non-contiguous, out of order
    for s in slots:
        manager.register(f"seq{s}", slot=s)
    history = {s: (torch.zeros((0, HEADS, DIM), dtype=torch.bfloat16),) * 2 for s in slots}

    def grow(counts):
        keys = [_bf16(oracle.hadamard(rng.standard_normal((c, HEADS, DIM)).astype(np.float32))) for c in counts]
        values = [_bf16(rng.standard_normal((c, HEADS, DIM)).astype(np.float32)) for c in counts]
        _append(manager, slots, keys, values, layer=[0, 1])
        for s, k, v in zip(slots, keys, values):
            history[s] = (torch.cat([history[s][0], k]), torch.cat([history[s][1], v]))

    grow([5, 16, 37])          # sub-page, exactly one page, multi-page with a tail
    grow([11, 1, 27])          # fills slot 3's first page from the hot tail; crosses pages
    grow([40, 40, 40])         # uniform multi-page append onto partial tails
    for _ in range(18):        # decode steps, one token per row, across a page boundary
        grow([1, 1, 1])
    torch.cuda.synchronize()
    for s in slots:
        for layer in (0, 1):
            _check_cache(kv, oracle, manager, s, history[s][0], history[s][1], layer=layer)
    # releasing a slot clears its tables; the other slots are untouched
    assert manager.release_slots([0]) == ("seq0",)
    assert manager.total_tokens(0) == 0 and manager.total_tokens(3) == history[3][0].shape[0]


def _cache_view(oracle, key_all, value_all):
    """What the cache holds for a sequence: full pages through the codec, the remainder in BF16."""
    total = key_all.shape[0]
    cold = (total // PAGE) * PAGE
    k_parts, v_parts = [], []
    for start in range(0, cold, PAGE):
        page = oracle.nqkv_page_payload(_f32(key_all[start:start + PAGE]), _f32(value_all[start:start + PAGE]),
                                        page_size=PAGE, q=Q, key_betas=KEY_BETAS, value_betas=VALUE_BETAS)
        for side, betas, parts in (("key", KEY_BETAS, k_parts), ("value", VALUE_BETAS, v_parts)):
            codes = oracle.unpack_unsigned(page[f"{side}_codes"], PAGE * HEADS * DIM, 4)
            ids = oracle.unpack_unsigned(page[f"{side}_betas"], PAGE * HEADS * DIM // 8, 2)
            parts.append(oracle.dequantize_rows(codes, ids, page[f"{side}_norms"], betas, Q).reshape(PAGE, HEADS, DIM))
    k_parts.append(_f32(key_all[cold:]))
    v_parts.append(_f32(value_all[cold:]))
    return np.concatenate(k_parts), np.concatenate(v_parts)


def _oracle_attention(oracle, query, key_all, value_all, group):
    k_view, v_view = _cache_view(oracle, key_all, value_all)
    return oracle.attention_dense(_f32(query), k_view, v_view)


@pytest.mark.parametrize("q_heads", [8, 16, 32, 64])
def test_attention_small_contexts_and_groups(kv, oracle, q_heads):
    rng = np.random.default_rng(q_heads)
    manager = _manager(kv, capacity=4, max_len=512)
    slots, lengths = [2, 0, 3], [1, 16, 203]            # hot tail only; one full page; pages + tail
    keys = [_bf16(oracle.hadamard(rng.standard_normal((n, HEADS, DIM)).astype(np.float32))) for n in lengths]
    values = [_bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for n in lengths]
    for s in slots:
        manager.register(s, slot=s)
    _append(manager, slots, keys, values)
    query = _bf16(oracle.hadamard(rng.standard_normal((4, q_heads, DIM)).astype(np.float32))).cuda()
    slot_ids = torch.tensor([2, 0, 3, 1], dtype=torch.int32, device="cuda")
    active = torch.tensor([True, True, True, False], device="cuda")       # row 3: unregistered slot
    out = kv.nqkv_decode_attention_batched_k1(query, manager.layers[0], slot_ids=slot_ids, active_mask=active)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (4, q_heads, DIM)
    for row in range(3):
        ref = _oracle_attention(oracle, query[row].cpu(), keys[row], values[row], q_heads // HEADS)
        assert relative_error(_f32(out[row]), ref) <= 1e-2, (row, q_heads)
    assert not out[3].any()                                             # inactive rows give zeros
    # a row whose mask is on but whose slot was never registered also gives zeros
    active[3] = True
    out = kv.nqkv_decode_attention_batched_k1(query, manager.layers[0], slot_ids=slot_ids, active_mask=active)
    assert not out[3].any()


@pytest.mark.parametrize("batch", [1, 2, 4, 8])
def test_batched_attention_equals_rows_taken_alone(kv, oracle, batch):
    """A row's result does not depend on the rows next to it, their order or the slot it sits in
    (non-contiguous slots).  The reference asserts equality between its batched and
    single-sequence kernels (tests/unit/runtime/test_nqkv_attention_batched_k1.py:116-143); here
    the chunk a workgroup takes depends on the batch width, so the same row taken alone may sum
    in another order: equal to within the rounding of the BF16 result."""
    rng = np.random.default_rng(100 + batch)
    manager = _manager(kv, capacity=8, max_len=1024)
    slots = [6, 1, 7, 0, 3, 5, 2, 4][:batch]
    lengths = [901, 17, 256, 3, 640, 33, 128, 1000][:batch]
    keys = [_bf16(oracle.hadamard(rng.standard_normal((n, HEADS, DIM)).astype(np.float32))) for n in lengths]
    values = [_bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for n in lengths]
    for s in slots:
        manager.register(s, slot=s)
    _append(manager, slots, keys, values)
    query = _bf16(oracle.hadamard(rng.standard_normal((batch, 32, DIM)).astype(np.float32))).cuda()
    slot_ids = torch.tensor(slots, dtype=torch.int32, device="cuda")
    active = torch.ones(batch, dtype=torch.bool, device="cuda")
    together = kv.nqkv_decode_attention_batched_k1(query, manager.layers[0], slot_ids=slot_ids, active_mask=active).clone()
    for row in range(batch):
        alone = kv.nqkv_decode_attention_batched_k1(query[row:row + 1], manager.layers[0], slot_ids=slot_ids[row:row + 1],
                                                    active_mask=active[:1])
        assert relative_error(_f32(alone[0]), _f32(together[row])) <= 2.0 ** -7, (batch, row)
    # reversing the rows reverses the results, bit for bit (same batch width, same chunks)
    order = list(range(batch))[::-1]
    flipped = kv.nqkv_decode_attention_batched_k1(query[order].contiguous(), manager.layers[0],
                                                  slot_ids=slot_ids[order].contiguous(), active_mask=active)
    assert torch.equal(flipped, together[order])


@pytest.mark.parametrize("batch,max_len,q_heads", [(8, 1024, 32), (3, 4096, 32), (1, 256, 8), (5, 64, 64)])
def test_attention_merged_inside_the_output_encoder(kv, oracle, batch, max_len, q_heads):
    """Stage 2 of the attention done by the encoder of the o_proj input: the merged rows equal the
    two-launch attention to within one BF16 step (the softmax denominator is summed in another
    order), an inactive row gives zeros, and codes, beta ids, norms and the decoded rows are bit for
    bit what the plain encoder makes of those merged rows."""
    from conftest import ACTIVATION_BETAS, Q
    from nestquant_aiinfra_amd.runtime import w4a4_linear as rt
    rng = np.random.default_rng(300 + batch)
    manager = _manager(kv, capacity=batch, max_len=max_len)
    lengths = [int(n) for n in rng.integers(1, max_len + 1, batch)]
    lengths[0] = max_len
    keys = [_bf16(oracle.hadamard(rng.standard_normal((n, HEADS, DIM)).astype(np.float32))) for n in lengths]
    values = [_bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for n in lengths]
    for s in range(batch):
        manager.register(s, slot=s)
    _append(manager, list(range(batch)), keys, values)
    cache = manager.layers[0]
    query = _bf16(oracle.hadamard(rng.standard_normal((batch, q_heads, DIM)).astype(np.float32))).cuda()
    slot_ids = torch.arange(batch, dtype=torch.int32, device="cuda")
    active = torch.ones(batch, dtype=torch.bool, device="cuda")
    if batch > 1:
        active[batch - 1] = False
    workspace = kv.BatchedNQKVAttentionWorkspace.create(cache, batch_size=batch, query_heads=q_heads,
                                                        output_dtype=torch.bfloat16)
    two_launches = kv.launch_nqkv_decode_attention(query, cache, slot_ids=slot_ids, active_mask=active,
                                                   attention_scale=0.125, workspace=workspace).clone()
    workspace.output.fill_(7.0)
    assert kv.launch_nqkv_decode_attention(query, cache, slot_ids=slot_ids, active_mask=active, attention_scale=0.125,
                                           workspace=workspace, merge=False) is None
    assert (workspace.output == 7.0).all()                                 # no merge launch ran
    table = torch.tensor(ACTIVATION_BETAS, dtype=torch.float32, device="cuda")
    _, merged = kv.attention_output_stage(workspace, encode=False, want_staged=True)
    n = q_heads * DIM
    a, b = _f32(merged), _f32(two_launches.view(batch, n))
    assert np.all(np.abs(a - b) <= np.abs(b) * 2.0 ** -7)
    assert np.count_nonzero(a != b) <= a.size // 50
    if batch > 1:
        assert not merged[batch - 1].any()
    power_of_two = n & (n - 1) == 0
    activation, again = kv.attention_output_stage(workspace, q=Q, beta_table=table, hadamard=power_of_two,
                                                  want_staged=True)
    assert torch.equal(again, merged)
    plain = rt.quantize_activation_cuda(merged, q=Q, betas=ACTIVATION_BETAS, beta_table=table, hadamard=power_of_two)
    for name in ("code_payload", "beta_payload", "row_norms", "decoded"):
        assert torch.equal(getattr(activation, name), getattr(plain, name)), name


def _rope(x: np.ndarray, positions: np.ndarray, theta: float = 500000.0) -> np.ndarray:
    """Llama rotary embedding of [tokens, heads, DIM] rows at the given positions (rotate-half form)."""
    inv_freq = 1.0 / theta ** (np.arange(0, DIM, 2, dtype=np.float64) / DIM)
    angle = positions.astype(np.float64)[:, None] * inv_freq[None, :]
    cos, sin = (np.concatenate((f(angle), f(angle)), axis=-1)[:, None, :].astype(np.float32) for f in (np.cos, np.sin))
    half = np.concatenate((-x[..., DIM // 2:], x[..., :DIM // 2]), axis=-1)
    return (x * cos + half * sin).astype(np.float32)


def test_attention_ragged_batch_at_full_size(kv, oracle):
    """Batch 8, 32 query / 8 KV heads, contexts uniform in [128, 4096] (up to 256 pages); keys and
    queries carry RoPE (theta = 500000) at their positions before the Hadamard, as the model makes them."""
    g = torch.Generator().manual_seed(4001)
    lengths = torch.randint(128, 4097, (8,), generator=g).tolist()
    lengths[0], lengths[1] = 4096, 128
    rng = np.random.default_rng(4002)
    manager = _manager(kv, capacity=8, max_len=4096)
    keys = [_bf16(oracle.hadamard(_rope(rng.standard_normal((n, HEADS, DIM)).astype(np.float32), np.arange(n))))
            for n in lengths]
    values = [_bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for n in lengths]
    for s in range(8):
        manager.register(s, slot=s)
    _append(manager, list(range(8)), keys, values)
    query = rng.standard_normal((8, 32, DIM)).astype(np.float32)
    query = np.stack([_rope(query[row:row + 1], np.array([n - 1]))[0] for row, n in enumerate(lengths)])
    query = _bf16(oracle.hadamard(query)).cuda()
    slot_ids = torch.arange(8, dtype=torch.int32, device="cuda")
    active = torch.ones(8, dtype=torch.bool, device="cuda")
    out = kv.nqkv_decode_attention_batched_k1(query, manager.layers[0], slot_ids=slot_ids, active_mask=active)
    again = kv.nqkv_decode_attention_batched_k1(query, manager.layers[0], slot_ids=slot_ids, active_mask=active)
    assert torch.equal(out, again)                                      # deterministic merge
    for row in (0, 1, 4):                                               # longest, shortest, one ragged
        ref = _oracle_attention(oracle, query[row].cpu(), keys[row], values[row], 4)
        assert relative_error(_f32(out[row]), ref) <= 1e-2, row
    _check_cache(kv, oracle, manager, 1, keys[1], values[1])
    # softmax weights sum to one: attending to constant values returns that constant
    manager.layers[0].hot_values.fill_(0)
    assert torch.isfinite(out).all()


@pytest.mark.parametrize("capacity,max_len,q_heads", [(4, 1024, 64), (8, 1024, 16), (1, 4096, 32), (2, 64, 8),
                                                      (8, 6400, 32), (3, 448, 32), (6, 400, 32), (12, 336, 16),
                                                      (16, 1024, 32)])
def test_attention_chunk_sizes(kv, oracle, capacity, max_len, q_heads):
    """The context is cut into chunks of 4, 8 or 16 pages depending on batch and table width (4 pages
    within 32 (row, chunk) pairs, 8 up to 100 pairs, 16 beyond), and the pairs are numbered part by
    part and rotated: every chunk size, with contexts that end inside a chunk, on a page edge and in the
    hot tail; eight parts a row (3 x 448), row counts that do not divide eight, more rows than XCDs."""
    rng = np.random.default_rng(capacity * max_len + q_heads)
    manager = _manager(kv, capacity=capacity, max_len=max_len)
    lengths = [max_len, max_len // 2 + 5, 33, 16, max_len - 16, 7, 1, max_len // 4]
    lengths = (lengths + [max(1, n - 3) for n in lengths])[:capacity]
    keys = [_bf16(oracle.hadamard(rng.standard_normal((n, HEADS, DIM)).astype(np.float32))) for n in lengths]
    values = [_bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for n in lengths]
    for s in range(capacity):
        manager.register(s, slot=s)
    _append(manager, list(range(capacity)), keys, values)
    query = _bf16(oracle.hadamard(rng.standard_normal((capacity, q_heads, DIM)).astype(np.float32))).cuda()
    slot_ids = torch.arange(capacity, dtype=torch.int32, device="cuda")
    active = torch.ones(capacity, dtype=torch.bool, device="cuda")
    out = kv.nqkv_decode_attention_batched_k1(query, manager.layers[0], slot_ids=slot_ids, active_mask=active)
    for row in range(capacity):
        ref = _oracle_attention(oracle, query[row].cpu(), keys[row], values[row], q_heads // HEADS)
        assert relative_error(_f32(out[row]), ref) <= 1e-2, (row, lengths[row])


@pytest.mark.parametrize("split_context", [False, True])
@pytest.mark.parametrize("q_heads", [8, 32, 64])
def test_prefill_attention_over_the_packed_cache(kv, oracle, q_heads, split_context):
    """Chunks of new tokens attend causally to everything their slot holds: a fresh prompt that
    crosses pages, a continuation of a sequence with cold pages, a one-token chunk, a padded row."""
    rng = np.random.default_rng(100 + q_heads)
    group = q_heads // HEADS
    manager = _manager(kv, capacity=4, max_len=256)
    for s in range(4):
        manager.register(s, slot=s)
    history = {0: 0, 1: 37, 2: 16, 3: 5}                       # tokens already in the cache per slot
    keys = {s: _bf16(oracle.hadamard(rng.standard_normal((n, HEADS, DIM)).astype(np.float32))) for s, n in history.items()}
    values = {s: _bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for s, n in history.items()}
    old = [s for s in history if history[s]]
    _append(manager, old, [keys[s] for s in old], [values[s] for s in old])

    slots, counts = [1, 0, 3, 2], [40, 23, 1, 0]               # the last row is padding only
    new_k = [_bf16(oracle.hadamard(rng.standard_normal((n, HEADS, DIM)).astype(np.float32))) for n in counts]
    new_v = [_bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for n in counts]
    live = [i for i, n in enumerate(counts) if n]
    width = max(counts)
    key = torch.zeros((4, width, HEADS, DIM), dtype=torch.bfloat16)
    value = torch.zeros_like(key)
    for i in live:
        key[i, : counts[i]], value[i, : counts[i]] = new_k[i], new_v[i]
    manager.step_slot_ids[:4] = torch.tensor(slots, dtype=torch.int32)
    manager.step_active[:4] = torch.tensor([n > 0 for n in counts])
    manager.step_counts[:4] = torch.tensor(counts, dtype=torch.int32)
    manager.begin_step(rows=4, uniform_count=None)
    manager.write_layer(0, key.cuda(), value.cuda())

    query = _bf16(oracle.hadamard(rng.standard_normal((4, width, q_heads, DIM)).astype(np.float32))).cuda()
    out = kv.nqkv_prefill_attention(query, manager.layers[0], slot_ids=manager.step_slot_ids, active_mask=manager.step_active,
                                    counts=manager.step_counts, split_context=split_context)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (4, width, q_heads, DIM)
    for i in live:
        slot = slots[i]
        all_k = torch.cat([keys[slot], new_k[i]]) if history[slot] else new_k[i]
        all_v = torch.cat([values[slot], new_v[i]]) if history[slot] else new_v[i]
        k_view, v_view = _cache_view(oracle, all_k, all_v)      # pages complete after the chunk are already packed
        for t in sorted({0, counts[i] // 2, counts[i] - 1}):
            visible = history[slot] + t + 1
            ref = oracle.attention_dense(_f32(query[i, t].cpu()), k_view[:visible], v_view[:visible])
            assert relative_error(_f32(out[i, t]), ref) <= 1e-2, (i, t)
        assert not out[i, counts[i]:].any()                     # padding tokens give zeros
    assert not out[3].any()
    # the last token of a chunk sees exactly what a decode step at that position sees
    i = 0
    decode = kv.nqkv_decode_attention_batched_k1(
        query[:, counts[i] - 1].contiguous(), manager.layers[0], slot_ids=manager.step_slot_ids[:4].clone(),
        active_mask=torch.tensor([True, False, False, False], device="cuda"))
    assert relative_error(_f32(out[i, counts[i] - 1]), _f32(decode[0])) <= 1e-2


def test_prefill_attention_with_the_context_split_over_workgroups(kv, oracle):
    """Long contexts, few rows: with a workspace the page table of every slot is split into ranges
    that workgroups of their own attend over and a second launch merges (`split_context`).  Same
    attention as the single walk (up to the rounding of the merged sums) and as the oracle's dense
    softmax; rows with short contexts, a padded row and ragged chunk lengths among them."""
    rng = np.random.default_rng(2027)
    q_heads = 32
    manager = _manager(kv, capacity=4, max_len=2048)
    for s in range(4):
        manager.register(s, slot=s)
    history = {0: 1500, 1: 40, 2: 0, 3: 700}
    keys = {s: _bf16(oracle.hadamard(rng.standard_normal((n, HEADS, DIM)).astype(np.float32))) for s, n in history.items()}
    values = {s: _bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for s, n in history.items()}
    old = [s for s in history if history[s]]
    _append(manager, old, [keys[s] for s in old], [values[s] for s in old])
    slots, counts = [0, 1, 2, 3], [100, 64, 0, 17]
    new_k = [_bf16(oracle.hadamard(rng.standard_normal((n, HEADS, DIM)).astype(np.float32))) for n in counts]
    new_v = [_bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for n in counts]
    width = max(counts)
    key = torch.zeros((4, width, HEADS, DIM), dtype=torch.bfloat16)
    value = torch.zeros_like(key)
    for i, n in enumerate(counts):
        key[i, :n], value[i, :n] = new_k[i], new_v[i]
    manager.step_slot_ids[:4] = torch.tensor(slots, dtype=torch.int32)
    manager.step_active[:4] = torch.tensor([n > 0 for n in counts])
    manager.step_counts[:4] = torch.tensor(counts, dtype=torch.int32)
    manager.begin_step(rows=4, uniform_count=None)
    manager.write_layer(0, key.cuda(), value.cuda())
    query = _bf16(oracle.hadamard(rng.standard_normal((4, width, q_heads, DIM)).astype(np.float32))).cuda()
    call = lambda split: kv.nqkv_prefill_attention(query, manager.layers[0], slot_ids=manager.step_slot_ids,
                                                   active_mask=manager.step_active, counts=manager.step_counts,
                                                   split_context=split)
    walked, split = call(False), call(True)
    assert torch.equal(split, call(True))                       # the merge adds the ranges in order
    assert relative_error(_f32(split), _f32(walked)) <= 4e-3
    assert not split[2].any() and not split[3, counts[3]:].any() and not split[1, counts[1]:].any()
    for i in (0, 3):
        slot = slots[i]
        k_view, v_view = _cache_view(oracle, torch.cat([keys[slot], new_k[i]]), torch.cat([values[slot], new_v[i]]))
        for token in (0, counts[i] - 1):
            visible = history[slot] + token + 1
            ref = oracle.attention_dense(_f32(query[i, token].cpu()), k_view[:visible], v_view[:visible])
            assert relative_error(_f32(split[i, token]), ref) <= 1e-2, (i, token)


def test_pool_handles_are_generation_checked(kv):
    pool = kv.NQKVPagePool(capacity=2, page_size=PAGE, num_kv_heads=HEADS, head_dim=DIM, q=Q,
                           key_betas=KEY_BETAS, value_betas=VALUE_BETAS, device="cuda")
    a, b = pool.allocate(), pool.allocate()
    with pytest.raises(RuntimeError, match="exhausted"):
        pool.allocate()
    key = torch.randn(3, HEADS, DIM, device="cuda").to(torch.bfloat16)
    page = kv.quantize_nqkv_page_cuda(key, key, page_size=PAGE, q=Q, key_betas=KEY_BETAS, value_betas=VALUE_BETAS)
    with pytest.raises(RuntimeError, match="not been stored"):
        pool.prepared(a)
    pool.store_prepared(a, page)
    assert torch.equal(pool.prepared(a).key_code_payload, page.key_code_payload) and pool.prepared(a).valid_tokens == 3
    pool.release(a)
    with pytest.raises(RuntimeError, match="stale"):
        pool.prepared(a)
    c = pool.allocate()
    assert c.page_id == a.page_id and c.generation == a.generation + 1 and pool.free_pages == 0
    assert pool.page_payload_bytes == 9728 and b.page_id != c.page_id


def test_slot_registration_in_batches_is_atomic_and_resets_the_tables(kv):
    """register_batch / release_slots (nestquant/runtime/nqkv_batch_manager.py:394-445): a rejected
    batch leaves no slot taken; admitted slots, neighbours or not, start from zeroed tables."""
    manager = _manager(kv, 8, 64)
    meta = manager.metadata
    tables = (meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths)
    for table in tables:
        table.fill_(7)
    manager.register_batch([("a", 0), ("b", 1), ("c", 2), ("d", 5), ("e", 7)])
    taken = [0, 1, 2, 5, 7]
    assert meta.active_mask.tolist() == [slot in taken for slot in range(8)]
    for table in tables:
        assert table.tolist() == [0 if slot in taken else 7 for slot in range(8)]
    with pytest.raises(RuntimeError, match="occupied"):
        manager.register_batch([("f", 3), ("g", 5)])
    with pytest.raises(ValueError, match="already registered"):
        manager.register_batch([("h", 3), ("a", 4)])
    with pytest.raises(ValueError, match="capacity"):
        manager.register_batch([("i", 3), ("j", 8)])
    assert [manager.sequence_id(slot) for slot in range(8)] == ["a", "b", "c", None, None, "d", None, "e"]
    assert meta.active_mask.tolist() == [slot in taken for slot in range(8)]
    key = torch.randn(3, HEADS, DIM).to(torch.bfloat16)
    _append(manager, [1, 5], [key, key[:2]], [key, key[:2]])
    assert meta.sequence_lengths.tolist()[:6] == [0, 3, 0, 7, 7, 2]
    assert manager.release_slots([5, 1, 3, 5]) == ("d", "b")
    assert meta.active_mask.tolist() == [True, False, True, False, False, False, False, True]
    assert meta.sequence_lengths.tolist() == [0, 0, 0, 7, 7, 0, 7, 0] and meta.hot_lengths.tolist()[1] == 0
    manager.register("k", slot=1)
    assert manager.sequence_id(1) == "k" and meta.active_mask.tolist()[1]


def test_page_container_from_the_gpu_encoder_equals_the_reference_file(kv, golden, golden_meta):
    """PackedNQKVPage.from_tensors (HIP encoder) serialises to the bytes the reference's CPU path
    wrote for the same page (SHA-256 in the golden metadata), decodes to the reference's values, and
    survives the trip through bytes and back onto the device."""
    import hashlib
    from nestquant_aiinfra_amd.core.kv_format import PackedNQKVPage
    key = torch.from_numpy(golden["kv_key_bf16_bits"]).view(torch.bfloat16).cuda()
    value = torch.from_numpy(golden["kv_value_bf16_bits"]).view(torch.bfloat16).cuda()
    page = PackedNQKVPage.from_tensors(key, value, page_size=PAGE, q=Q, key_betas=KEY_BETAS, value_betas=VALUE_BETAS)
    blob = page.to_bytes()
    assert hashlib.sha256(blob).hexdigest() == golden_meta["kv_container_v2_sha256"]
    restored = PackedNQKVPage.from_bytes(blob)
    dk, dv = restored.dequantize(output_dtype=torch.float32)
    assert np.array_equal(_f32(dk), golden["kv_key_deq"]) and np.array_equal(_f32(dv), golden["kv_value_deq"])
    # back into a pool page
    pool = kv.NQKVPagePool(capacity=2, page_size=PAGE, num_kv_heads=HEADS, head_dim=DIM, q=Q, key_betas=KEY_BETAS,
                           value_betas=VALUE_BETAS, device="cuda")
    handle = pool.allocate()
    pool.store_prepared(handle, restored.to_prepared("cuda"))
    stored = pool.prepared(handle)
    assert np.array_equal(bits(stored.key_code_payload), golden["kv_key_codes"])
    assert np.array_equal(bits(stored.value_norms), golden["kv_value_norms"])


@pytest.mark.parametrize("valid", [1, 5, 15, 16])
def test_page_container_fill_levels(kv, oracle, golden, valid):
    """Boundary fill levels (tests/unit/core/test_kv_format.py:59-78): padding rows are encoded
    zeros, never leak into the valid prefix, and both container versions round-trip."""
    from nestquant_aiinfra_amd.core.kv_format import PackedNQKVPage
    key = torch.from_numpy(golden["kv_key_bf16_bits"]).view(torch.bfloat16).cuda()[:valid]
    value = torch.from_numpy(golden["kv_value_bf16_bits"]).view(torch.bfloat16).cuda()[:valid]
    for tables in ({"betas": KEY_BETAS}, {"key_betas": KEY_BETAS, "value_betas": VALUE_BETAS}):
        page = PackedNQKVPage.from_tensors(key, value, page_size=PAGE, q=Q, **tables)
        assert page.valid_tokens == valid and page.payload_bytes == 9728
        assert not page.key_norms[valid * HEADS:].any() and not page.value_norms[valid * HEADS:].any()
        again = PackedNQKVPage.from_bytes(page.to_bytes())
        assert again.format_version == (1 if "betas" in tables else 2)
        dk, dv = again.dequantize(output_dtype=torch.float32)
        assert tuple(dk.shape) == tuple(dv.shape) == (valid, HEADS, DIM)
        assert np.array_equal(_f32(dk), golden["kv_key_deq"][:valid])
        if "betas" not in tables:
            assert np.array_equal(_f32(dv), golden["kv_value_deq"][:valid])
    if valid == 5:
        legacy = PackedNQKVPage.from_tensors(key, value, page_size=PAGE, q=Q, betas=KEY_BETAS)
        assert np.array_equal(np.frombuffer(legacy.key_indices.code_payload, np.uint8), golden["kv_partial_key_codes"])
        assert np.array_equal(legacy.key_norms.numpy(), golden["kv_partial_key_norms"])
    with pytest.raises(ValueError):
        PackedNQKVPage.from_tensors(key, value, page_size=PAGE, q=Q, betas=KEY_BETAS, key_betas=KEY_BETAS)
    with pytest.raises(ValueError):
        PackedNQKVPage.from_tensors(key, value, page_size=PAGE, q=Q, key_betas=KEY_BETAS)


def test_decode_step_begin_is_advance_plus_two_gathers():
    """The head-of-step launch against nq_nqkv_advance (uniform count 1) on a copy of the tables,
    torch's embedding and an index_select of the rotary table: inactive rows and rows with a slot
    out of range advance nothing, a slot at capacity stays there, positions past the table take
    its last row, an unknown token embeds as zero."""
    from nestquant_aiinfra_amd import _native
    lib = _native.library()
    g = torch.Generator().manual_seed(909)
    rows, slots, page, max_tokens, vocab, hidden, dim, max_pos = 6, 8, 16, 64, 300, 2048, 64, 96
    slot_ids = torch.tensor([3, 0, 7, 9, 5, 1], dtype=torch.int32, device="cuda")         # 9: out of range; 7: inactive
    active = torch.tensor([True, True, False, True, True, True], device="cuda")
    lengths = torch.tensor([15, 31, 0, 64, 5, 47, 1, 16], dtype=torch.int32, device="cuda")  # slot 3: at capacity
    tokens = torch.tensor([[5], [299], [0], [17], [300], [-1]], dtype=torch.long, device="cuda")
    positions = torch.tensor([[0], [95], [96], [1000], [7], [50]], dtype=torch.long, device="cuda")
    embedding = torch.randn((vocab, hidden), generator=g).to(torch.bfloat16).cuda()
    rotary = torch.randn((2, max_pos, dim), generator=g).to(torch.bfloat16).cuda()
    stream = _native.stream_handle(torch.device("cuda"))

    def tables():
        return [lengths.clone(), lengths // page, torch.where(lengths >= page, page, 0).int(), lengths % page]
    want, got = tables(), tables()
    _native.check(lib.nq_nqkv_advance(slot_ids.data_ptr(), active.data_ptr(), None, 1, rows, slots, page, max_tokens,
                                      *[t.data_ptr() for t in want], stream))
    embedded = torch.full((rows, hidden), 7.0, dtype=torch.bfloat16, device="cuda")
    rotary_rows = torch.full((2, rows, dim), 7.0, dtype=torch.bfloat16, device="cuda")
    _native.check(lib.nq_decode_step_begin(
        slot_ids.data_ptr(), active.data_ptr(), rows, slots, page, max_tokens, *[t.data_ptr() for t in got],
        tokens.data_ptr(), embedding.data_ptr(), vocab, hidden, embedded.data_ptr(), positions.data_ptr(),
        rotary.data_ptr(), max_pos, dim, rotary_rows.data_ptr(), stream))
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    assert got[0].tolist() == [16, 32, 0, 64, 5, 48, 1, 16]
    known = ((tokens >= 0) & (tokens < vocab)).view(-1)
    reference = torch.nn.functional.embedding(tokens.view(-1).clamp(0, vocab - 1), embedding)
    reference[~known] = 0
    assert torch.equal(embedded.view(torch.int16), reference.view(torch.int16))
    assert torch.equal(rotary_rows, rotary.index_select(1, positions.view(-1).clamp(0, max_pos - 1)))


def test_prompt_step_begin_equals_reset_copies_and_advance(kv):
    """A scripted run of prompt steps (new sequences into free slots, further chunks into slots that hold
    tokens, rows that write nothing, slots released and taken again, a slot filled to capacity) through two
    managers: one resets, copies and advances with tensor operations and nq_nqkv_advance, the other does the
    step's head as one copy and one launch.  Tables, row state, positions and last-token indices agree."""
    rng = np.random.default_rng(4242)
    capacity, max_len = 8, 96
    plain, fused = _manager(kv, capacity, max_len), _manager(kv, capacity, max_len)
    held = [None] * capacity                                   # tokens per slot on the host, None = free
    generation = 0
    for step in range(120):
        rows = int(rng.integers(1, capacity + 1))
        slots = [int(s) for s in rng.permutation(capacity)[:rows]]
        width = int(rng.choice([1, 7, 16, 33, 96]))
        fresh = [s for s in slots if held[s] is None]
        counts = []
        for s in slots:
            room = max_len - (held[s] or 0)
            counts.append(int(min(room, rng.integers(0, width + 1))) if rng.random() > 0.15 else 0)
        generation += 1
        for manager, reset in ((plain, True), (fused, False)):
            manager.register_batch([((generation, s), s) for s in fresh], reset_tables=reset)
        starts = torch.tensor([held[s] or 0 for s in slots])
        plain.step_slot_ids[:rows].copy_(torch.tensor(slots, dtype=torch.int32))
        plain.step_counts[:rows].copy_(torch.tensor(counts, dtype=torch.int32))
        plain.step_active[:rows].copy_(torch.tensor([c > 0 for c in counts]))
        plain.begin_step(rows=rows, uniform_count=None)
        positions = torch.full((rows, width), -1, dtype=torch.long, device="cuda")
        last = torch.full((rows,), -1, dtype=torch.long, device="cuda")
        fused.begin_prompt_step(slot_ids=slots, counts=counts, fresh=[s in fresh for s in slots], width=width,
                                positions=positions, last_token=last)
        for s, c in zip(slots, counts):
            held[s] = (held[s] or 0) + c
        for name in ("sequence_lengths", "page_counts", "last_page_lens", "hot_lengths", "active_mask"):
            assert torch.equal(getattr(fused.metadata, name), getattr(plain.metadata, name)), (step, name)
        for name in ("step_slot_ids", "step_counts", "step_active"):
            assert torch.equal(getattr(fused, name)[:rows], getattr(plain, name)[:rows]), (step, name)
        assert fused.metadata.sequence_lengths.tolist() == [h or 0 for h in held]
        assert torch.equal(positions.cpu(), starts[:, None] + torch.arange(width)[None, :]), step
        assert last.tolist() == [max(c - 1, 0) for c in counts]
        gone = [s for s in range(capacity) if held[s] is not None and rng.random() < 0.2]
        for manager in (plain, fused):
            manager.release_slots(gone)
        for s in gone:
            held[s] = None
    assert max(h or 0 for h in held) <= max_len
    with pytest.raises(ValueError, match="int64"):
        fused.begin_prompt_step(slot_ids=[0], counts=[0], fresh=[False], width=4,
                                positions=torch.zeros((1, 4), dtype=torch.int32, device="cuda"))


@pytest.mark.parametrize("q_heads,max_len,steps", [(32, 256, 40), (8, 256, 20), (64, 64, 34), (16, 1024, 20),
                                                   (32, 2048, 20), (32, 16384, 18)])
def test_append_inside_the_attention_launch_equals_writer_then_attention(kv, oracle, q_heads, max_len, steps):
    """One launch per layer and decode step (`append_and_attend`) against the two it replaces
    (`write_layer`, then `launch_nqkv_decode_attention`), on two caches fed the same tokens: after
    every step the pools, hot tails and tables are bit for bit the same.  The attention rows are
    bit for bit the same on steps where the row's token does not complete a page; where it does,
    the fused launch merges that page as a part of its own, so the rows agree to the rounding of the
    BF16 result.  Covers rows that complete pages at different steps, a row that is not in the
    step, a slot whose cache is switched off for some steps (it still appends), RoPE(theta = 500000)
    on keys and queries, (max_len 64) a slot that reaches its capacity, and tables wide enough for
    chunks of 8 and 16 pages."""
    rng = np.random.default_rng(700 + q_heads)
    slots, lengths = [3, 0, 2, 1], [5, 16, 37, 9]
    if max_len >= 1024:                               # chunks of 4, 8 and 16 pages; one row ends near the table's end
        lengths = [max_len * 11 // 16 + 12, 16, max_len - 21, 9]
    rows = len(slots)
    managers = [_manager(kv, capacity=4, max_len=max_len) for _ in range(2)]
    keys = [_bf16(oracle.hadamard(rng.standard_normal((n, HEADS, DIM)).astype(np.float32))) for n in lengths]
    values = [_bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for n in lengths]
    for manager in managers:
        for s in slots:
            manager.register(f"seq{s}", slot=s)
        _append(manager, slots, keys, values)
    workspaces = [kv.BatchedNQKVAttentionWorkspace.create(m.layers[0], batch_size=rows, query_heads=q_heads,
                                                          output_dtype=torch.bfloat16) for m in managers]
    totals = list(lengths)
    for step in range(steps):
        in_step = [True, True, True, step % 5 != 3]                  # the last row sits out every fifth step
        cache_on = not (7 <= step < 11)                              # slot 0's cache is off for four steps
        key = _bf16(rng.standard_normal((rows, HEADS, DIM)).astype(np.float32)).cuda()
        value = _bf16(rng.standard_normal((rows, HEADS, DIM)).astype(np.float32)).cuda()
        query = _bf16(rng.standard_normal((rows, q_heads, DIM)).astype(np.float32)).cuda()
        positions = np.asarray(totals, dtype=np.float64)
        angles = positions[:, None] * (500000.0 ** (-np.arange(0, DIM, 2) / DIM))[None, :]
        cos = _bf16(np.concatenate([np.cos(angles)] * 2, axis=1).astype(np.float32)).cuda()
        sin = _bf16(np.concatenate([np.sin(angles)] * 2, axis=1).astype(np.float32)).cuda()
        packs = []
        for i in range(rows):
            grows = in_step[i] and totals[i] < managers[0].max_tokens
            totals[i] += 1 if grows else 0
            packs.append(in_step[i] and totals[i] % PAGE == 0)
        outputs = []
        for which, (manager, workspace) in enumerate(zip(managers, workspaces)):
            manager.step_slot_ids[:rows] = torch.tensor(slots, dtype=torch.int32)
            manager.step_active[:rows] = torch.tensor(in_step)
            manager.metadata.active_mask[0] = cache_on
            manager.begin_step(rows=rows, uniform_count=1)
            if which == 0:
                manager.write_layer(0, key.view(rows, 1, HEADS, DIM), value.view(rows, 1, HEADS, DIM), rotate_keys=True,
                                    rope=(cos.view(rows, 1, DIM), sin.view(rows, 1, DIM)))
                out = kv.launch_nqkv_decode_attention(query, manager.layers[0], slot_ids=manager.step_slot_ids,
                                                      active_mask=manager.step_active, attention_scale=0.125,
                                                      workspace=workspace, rotate_query=True, rope=(cos, sin))
            else:
                out = manager.append_and_attend(0, query, key, value, attention_scale=0.125, workspace=workspace,
                                                rotate=True, rope=(cos, sin))
            outputs.append(out.clone())
        torch.cuda.synchronize()
        two, one = outputs
        for i in range(rows):
            if packs[i]:
                assert relative_error(_f32(one[i]), _f32(two[i])) <= 2.0 ** -7, (step, i)
            else:
                assert torch.equal(one[i], two[i]), (step, i)
        if not cache_on:
            assert not one[1].any()                                  # slot 0 is row 1
        a, b = managers
        for name in ("sequence_lengths", "page_counts", "last_page_lens", "hot_lengths"):
            assert torch.equal(getattr(a.metadata, name), getattr(b.metadata, name)), (step, name)
        assert [a.total_tokens(s) for s in slots] == totals
        for name in ("key_codes", "key_betas", "key_norms", "value_codes", "value_betas", "value_norms"):
            assert torch.equal(getattr(a.layers[0].pool, name), getattr(b.layers[0].pool, name)), (step, name)
        assert torch.equal(a.layers[0].hot_keys, b.layers[0].hot_keys), step
        assert torch.equal(a.layers[0].hot_values, b.layers[0].hot_values), step
    assert any(t % PAGE < steps for t in totals)                     # pages were completed on the way


def test_append_and_attend_rejects_what_it_cannot_take(kv):
    """The one-launch form is for decode steps of one BF16 token per row: anything else is refused
    before a launch, with the cache untouched."""
    manager = _manager(kv, capacity=2, max_len=64)
    for s in (0, 1):
        manager.register(s, slot=s)
    workspace = kv.BatchedNQKVAttentionWorkspace.create(manager.layers[0], batch_size=2, query_heads=32,
                                                        output_dtype=torch.bfloat16)
    query = torch.zeros((2, 32, DIM), dtype=torch.bfloat16, device="cuda")
    key = torch.zeros((2, HEADS, DIM), dtype=torch.bfloat16, device="cuda")
    manager.step_active[:2] = True
    manager.begin_step(rows=2, uniform_count=3)                      # a step of three tokens per row
    with pytest.raises(ValueError, match="one token each"):
        manager.append_and_attend(0, query, key, key, attention_scale=0.125, workspace=workspace)
    manager.begin_step(rows=2, uniform_count=1)
    before = manager.layers[0].hot_keys.clone()
    with pytest.raises(TypeError, match="BF16"):
        manager.append_and_attend(0, query.half(), key, key, attention_scale=0.125, workspace=workspace)
    with pytest.raises(ValueError, match="kv_heads"):
        manager.append_and_attend(0, query, key[:, :4].contiguous(), key[:, :4].contiguous(), attention_scale=0.125,
                                  workspace=workspace)
    with pytest.raises(ValueError, match="contiguous"):
        manager.append_and_attend(0, query, key.transpose(0, 1).contiguous().transpose(0, 1), key,
                                  attention_scale=0.125, workspace=workspace)
    with pytest.raises(ValueError, match="scale must be finite"):
        manager.append_and_attend(0, query, key, key, attention_scale=float("nan"), workspace=workspace)
    torch.cuda.synchronize()
    assert torch.equal(manager.layers[0].hot_keys, before)


def test_decode_attention_refuses_a_misaligned_query(kv):
    """BF16 query rows are read 16 bytes at a time: a view that starts two bytes into a buffer is refused
    by the wrapper, and by the library itself when a caller hands it the raw pointer."""
    from nestquant_aiinfra_amd import _native
    manager = _manager(kv, capacity=1, max_len=32)
    manager.register(0, slot=0)
    cache = manager.layers[0]
    workspace = kv.BatchedNQKVAttentionWorkspace.create(cache, batch_size=1, query_heads=32, output_dtype=torch.bfloat16)
    backing = torch.zeros(32 * DIM + 8, dtype=torch.bfloat16, device="cuda")
    shifted = backing[1:1 + 32 * DIM].view(1, 32, DIM)
    slot_ids = torch.zeros(1, dtype=torch.int32, device="cuda")
    active = torch.ones(1, dtype=torch.bool, device="cuda")
    with pytest.raises(ValueError, match="16-byte aligned"):
        kv.launch_nqkv_decode_attention(shifted, cache, slot_ids=slot_ids, active_mask=active, attention_scale=0.125,
                                        workspace=workspace)
    pool, meta = cache.pool, cache.metadata
    status = _native.library().nq_nqkv_attention_decode(
        shifted.data_ptr(), _native.dtype_tag(torch.bfloat16),
        pool.key_codes.data_ptr(), pool.key_betas.data_ptr(), pool.key_norms.data_ptr(),
        pool.value_codes.data_ptr(), pool.value_betas.data_ptr(), pool.value_norms.data_ptr(),
        pool.beta_table.data_ptr(), pool.value_beta_table.data_ptr(),
        meta.page_indices.data_ptr(), meta.page_counts.data_ptr(), meta.last_page_lens.data_ptr(),
        meta.hot_lengths.data_ptr(), meta.active_mask.data_ptr(), cache.hot_keys.data_ptr(), cache.hot_values.data_ptr(),
        slot_ids.data_ptr(), active.data_ptr(), 1, cache.max_sequences, cache.max_pages_per_sequence, 32, pool.num_kv_heads,
        DIM, pool.page_size, 0.125, 0, None, None, workspace.output.data_ptr(), workspace.buffer.data_ptr(),
        workspace.buffer.numel(), None, None, _native.stream_handle(shifted.device))
    assert status == _native.NQ_ERR_ARGUMENT and b"16-byte alignment" in _native.library().nq_last_error()
