"""The one-sequence names of the reference's cache (PagedNQKVCache, NQKVHotColdCache over it,
nqkv_decode_attention_k1, NQKVLlamaCache, install_nqkv_llama_backend: nestquant/runtime/
paged_nqkv_cache.py:98-332, nqkv_attention_k1.py:669-760, nqkv_hf_backend.py:24-232) are adapters
over the batched kernels: what they store and compute must equal the batched objects' results on
the same tokens, which the other GPU tests pin against the oracle."""

import pytest
import torch

from conftest import KEY_BETAS, Q, VALUE_BETAS

pytestmark = pytest.mark.gpu

HEADS, KV_HEADS, DIM, PAGE = 8, 2, 64, 16


def _tokens(count, seed):
    g = torch.Generator().manual_seed(seed)
    key = torch.randn(count, KV_HEADS, DIM, generator=g).to(torch.bfloat16).cuda()
    value = torch.randn(count, KV_HEADS, DIM, generator=g).to(torch.bfloat16).cuda()
    return key, value


def _sequence_cache(pages=6, sequences=3):
    from nestquant_aiinfra_amd.runtime import NQKVHotColdCache, NQKVPagePool, PagedNQKVCache
    pool = NQKVPagePool(capacity=pages, page_size=PAGE, num_kv_heads=KV_HEADS, head_dim=DIM, q=Q, key_betas=KEY_BETAS,
                        value_betas=VALUE_BETAS, device="cuda")
    logical = PagedNQKVCache(pool, max_sequences=sequences, max_pages_per_sequence=4)
    return pool, logical, NQKVHotColdCache(logical)


def test_sequence_appends_equal_the_batched_manager_and_attention_equals_its_row():
    from nestquant_aiinfra_amd.runtime import (BatchedNQKVCacheManager, NQKVAttentionWorkspace, nqkv_decode_attention_batched_k1,
                                               nqkv_decode_attention_k1)
    pool, logical, cache = _sequence_cache()
    assert cache.register("first") == 0 and cache.register("second", slot=2) == 2
    assert logical.active_sequences == 2 and logical.sequence_id(2) == "second"
    manager = BatchedNQKVCacheManager(capacity=3, num_layers=1, num_kv_heads=KV_HEADS, head_dim=DIM, max_cache_len=64,
                                      page_size=PAGE, q=Q, key_betas=KEY_BETAS, value_betas=VALUE_BETAS,
                                      dtype=torch.bfloat16, device="cuda")
    manager.register("second", slot=2)
    key, value = _tokens(44, 7)
    at = 0
    for count in (5, 20, 16, 3):                       # tail only; a page and a tail; exactly a page; tail
        cache.append("second", key[at:at + count], value[at:at + count])
        manager.step_slot_ids[:1] = 2
        manager.step_active[:1] = True
        manager.step_counts[:1] = count
        manager.begin_step(rows=1, uniform_count=None)
        manager.write_layer(0, key[None, at:at + count].contiguous(), value[None, at:at + count].contiguous())
        at += count
    assert cache.total_tokens("second") == 44 and logical.total_tokens("second") == 32 and cache.hot_length(2) == 12
    handles = logical.handles("second")
    assert len(handles) == 2 and pool.allocated_pages == 2 and logical.reserved_handles("second") == ()
    other = manager.layers[0]
    for name in ("sequence_lengths", "page_counts", "last_page_lens", "hot_lengths"):
        assert getattr(cache.metadata, name)[2].item() == getattr(other.metadata, name)[2].item()
    for ordinal, handle in enumerate(handles):          # the same page bytes, wherever the pool put them
        mine, theirs = handle.page_id, int(other.metadata.page_indices[2, ordinal])
        for name in ("key_codes", "key_betas", "key_norms", "value_codes", "value_betas", "value_norms"):
            assert torch.equal(getattr(pool, name)[mine], getattr(other.pool, name)[theirs])
    assert torch.equal(cache.hot_keys[2, :12], other.hot_keys[2, :12])
    hot_key, hot_value = cache.hot_view("second")
    assert tuple(hot_key.shape) == (12, KV_HEADS, DIM) and torch.equal(hot_value, value[32:44])
    whole_key, whole_value = cache.materialize("second")
    assert tuple(whole_key.shape) == (44, KV_HEADS, DIM) and torch.equal(whole_key[32:], key[32:44])
    assert torch.nn.functional.cosine_similarity(whole_value[:32].float().flatten(), value[:32].float().flatten(), dim=0) > 0.98

    g = torch.Generator().manual_seed(8)
    query = torch.randn(HEADS, DIM, generator=g).to(torch.bfloat16).cuda()
    workspace = NQKVAttentionWorkspace.create(cache, query_heads=HEADS, output_dtype=torch.bfloat16)
    single = nqkv_decode_attention_k1(query, cache, "second", scale=0.125, workspace=workspace)
    batched = nqkv_decode_attention_batched_k1(
        query[None], other, slot_ids=torch.tensor([2], dtype=torch.int32, device="cuda"),
        active_mask=torch.ones(1, dtype=torch.bool, device="cuda"), scale=0.125)
    assert tuple(single.shape) == (HEADS, DIM) and torch.equal(single, batched[0])
    # against plain softmax attention over the materialised cache (what the reference's prefill computes)
    keys = whole_key.float().repeat_interleave(HEADS // KV_HEADS, dim=1)
    values = whole_value.float().repeat_interleave(HEADS // KV_HEADS, dim=1)
    weights = torch.softmax(torch.einsum("hd,thd->ht", query.float(), keys) * 0.125, dim=-1)
    dense = torch.einsum("ht,thd->hd", weights, values)
    assert float((single.float() - dense).abs().max() / dense.abs().max()) <= 1e-2
    with pytest.raises(ValueError, match="empty sequence"):
        nqkv_decode_attention_k1(query, cache, "first")

    # ownership: a released sequence gives its pages back and its handles go stale
    cache.release("second")
    assert pool.allocated_pages == 0 and logical.active_sequences == 1
    with pytest.raises(RuntimeError, match="stale or released"):
        pool.prepared(handles[0])
    with pytest.raises(KeyError):
        logical.slot("second")
    assert cache.metadata.sequence_lengths.tolist() == [0, 0, 0] and not bool(cache.metadata.active_mask[2])


def test_paged_cache_page_protocol():
    from nestquant_aiinfra_amd.core.kv_format import PackedNQKVPage
    from nestquant_aiinfra_amd.runtime import nqkv_decode_attention_k1, quantize_nqkv_page_cuda
    pool, logical, cache = _sequence_cache(pages=3, sequences=2)
    slot = logical.register("s")
    key, value = _tokens(16 + 9, 11)
    full = quantize_nqkv_page_cuda(key[:16], value[:16], page_size=PAGE, q=Q, key_betas=KEY_BETAS, value_betas=VALUE_BETAS)
    partial = quantize_nqkv_page_cuda(key[16:], value[16:], page_size=PAGE, q=Q, key_betas=KEY_BETAS, value_betas=VALUE_BETAS)
    reserved = logical.reserve_page("s")
    assert logical.reserved_handles("s") == (reserved,) and logical.handles("s") == () and pool.allocated_pages == 1
    assert int(logical.page_counts[slot]) == 0                       # not visible to the kernels yet
    logical.cancel_reserved_page("s", reserved)
    assert pool.allocated_pages == 0
    with pytest.raises(RuntimeError, match="not reserved"):
        logical.commit_prepared_page("s", reserved, full)
    first = logical.append_prepared_page("s", full)
    second = logical.append_page("s", PackedNQKVPage.from_prepared(partial, key_betas=KEY_BETAS, value_betas=VALUE_BETAS))
    assert logical.handles("s") == (first, second) and logical.total_tokens("s") == 25
    assert logical.page_indices[slot, :2].tolist() == [first.page_id, second.page_id]
    assert (int(logical.page_counts[slot]), int(logical.last_page_len[slot]), int(logical.sequence_lengths[slot])) == (2, 9, 25)
    with pytest.raises(RuntimeError, match="partial last page"):
        logical.reserve_page("s")
    with pytest.raises(RuntimeError, match="whole pages only"):
        cache.append("s", key[:1], value[:1])
    # attention reads both pages, the second up to its nine valid tokens
    g = torch.Generator().manual_seed(12)
    query = torch.randn(HEADS, DIM, generator=g).to(torch.bfloat16).cuda()
    out = nqkv_decode_attention_k1(query, cache, "s", scale=0.125)
    whole_key, whole_value = cache.materialize("s")
    assert tuple(whole_key.shape) == (25, KV_HEADS, DIM)
    keys = whole_key.float().repeat_interleave(HEADS // KV_HEADS, dim=1)
    values = whole_value.float().repeat_interleave(HEADS // KV_HEADS, dim=1)
    weights = torch.softmax(torch.einsum("hd,thd->ht", query.float(), keys) * 0.125, dim=-1)
    dense = torch.einsum("ht,thd->hd", weights, values)
    assert float((out.float() - dense).abs().max() / dense.abs().max()) <= 1e-2
    # the table is full of sequences: a third one is refused, a freed slot is taken again
    logical.register("t")
    with pytest.raises(RuntimeError, match="table is full"):
        logical.register("u")
    logical.release("s")
    assert logical.register("u") == slot and pool.allocated_pages == 0
    with pytest.raises(ValueError, match="already registered"):
        logical.register("u")


def test_one_sequence_llama_cache_tracks_the_batched_cache():
    """A tiny random-weight Llama driven through `model.forward` with the one-sequence cache: a prompt
    in two chunks, then greedy decode; the batched cache with one slot, fed the same tokens through the
    same module graph, gives the same logits (both attend to the packed cache with the same kernels)."""
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.runtime import (BatchedNQKVLlamaCache, BatchedNQKVLlamaRunner, NQKVLlamaCache,
                                               install_batched_nqkv_llama_backend, install_nqkv_llama_backend)

    torch.manual_seed(5021)
    config = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                         num_key_value_heads=2, head_dim=64, vocab_size=128, max_position_embeddings=512,
                         rope_theta=500000.0, tie_word_embeddings=True)
    model = LlamaForCausalLM(config).to(torch.bfloat16).cuda().eval()
    geometry = dict(num_layers=2, num_query_heads=4, num_kv_heads=2, head_dim=64, max_cache_len=96, page_size=PAGE, q=Q,
                    key_betas=KEY_BETAS, value_betas=VALUE_BETAS, dtype=torch.bfloat16, device="cuda")
    g = torch.Generator().manual_seed(5022)
    prompt = torch.randint(1, 128, (1, 37), generator=g).cuda()

    single = NQKVLlamaCache(**geometry)
    assert install_nqkv_llama_backend(model, single) == "nestquant_nqkv_k1"
    with torch.inference_mode():
        first = model(input_ids=prompt[:, :21], position_ids=torch.arange(21, device="cuda")[None], past_key_values=single,
                      use_cache=True).logits
        second = model(input_ids=prompt[:, 21:], position_ids=torch.arange(21, 37, device="cuda")[None],
                       past_key_values=single, use_cache=True).logits
        assert single.get_seq_length() == 37 and single.get_mask_sizes(1, 0) == (38, 0)
        token, single_logits = second[:, -1].argmax(-1).reshape(1, 1), [first, second]
        tokens = [int(token)]
        for step in range(14):                           # crosses the page boundary at 48 tokens
            out = model(input_ids=token, position_ids=torch.tensor([[37 + step]], device="cuda"), past_key_values=single,
                        use_cache=True).logits
            single_logits.append(out)
            token = out[:, -1].argmax(-1).reshape(1, 1)
            tokens.append(int(token))
    assert single.get_seq_length(1) == 51 and single.layer_caches[0].cold_cache.pool.allocated_pages == 3

    batched = BatchedNQKVLlamaCache(capacity=1, packed_prefill=True, **geometry)
    install_batched_nqkv_llama_backend(model, batched)
    runner = BatchedNQKVLlamaRunner(model, batched, fused_decode=False, fused_prefill=False)
    batched_logits = [runner.prefill_slots(prompt[:, :21], slots=[0], lengths=[21]),
                      runner.prefill_slots(prompt[:, 21:], slots=[0], lengths=[16])]
    for step in range(14):
        batched_logits.append(runner.decode_eager(torch.tensor([[tokens[step]]], device="cuda"), slots=[0],
                                                  positions=torch.tensor([[37 + step]], device="cuda")))
    for mine, theirs in zip(single_logits, batched_logits):
        assert torch.isfinite(mine).all() and mine.shape == theirs.shape
        assert torch.nn.functional.cosine_similarity(mine.float().flatten(), theirs.float().flatten(), dim=0) > 0.9999
        assert torch.equal(mine.argmax(-1), theirs.argmax(-1))
    for layer in range(2):                               # the same cache contents, layer by layer
        mine, theirs = single.layer_caches[layer], batched.manager.layers[layer]
        assert torch.equal(mine.hot_keys[0, :3], theirs.hot_keys[0, :3])
        for ordinal, handle in enumerate(mine.cold_cache.handles("batch0")):
            assert torch.equal(mine.pool.key_codes[handle.page_id], theirs.pool.key_codes[ordinal])
            assert torch.equal(mine.pool.value_codes[handle.page_id], theirs.pool.value_codes[ordinal])
    single.reset()
    assert single.get_seq_length() == 0 and single.layer_caches[1].cold_cache.pool.allocated_pages == 0
    with pytest.raises(NotImplementedError):
        single.reorder_cache(torch.zeros(1, dtype=torch.long))
    with pytest.raises(TypeError):
        install_nqkv_llama_backend(model, batched)
