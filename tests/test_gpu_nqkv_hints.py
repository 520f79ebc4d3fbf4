"""Decode hints of the NQKV4 pools (four bits per block beside the reference's six streams).

What is pinned here:
  * every one of the 14^8 code words decodes to the same eight floats with its hint as without
    (the library's own exhaustive check, run over the whole range);
  * the writers (ragged writer, the appending attention launch, a page stored from a container) leave
    exactly the hints of the code words they store (against the stand-alone hint kernel);
  * with hints the six streams of the pools, the hot tails and the tables stay bit for bit what they
    are without, and both attention kernels return bit-identical outputs;
  * a tiny model's runner gives the same logits with and without hints, captured and un-captured.
"""

import ctypes

import numpy as np
import pytest
import torch

from conftest import KEY_BETAS, Q, VALUE_BETAS

pytestmark = pytest.mark.gpu

HEADS, DIM, PAGE = 8, 64, 16
STREAMS = ("key_codes", "key_betas", "key_norms", "value_codes", "value_betas", "value_norms")


@pytest.fixture(scope="module")
def kv():
    from nestquant_aiinfra_amd.runtime import nqkv
    return nqkv


def _bf16(x: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(x).to(torch.bfloat16)


def _manager(kv, capacity, max_len, hints):
    return kv.BatchedNQKVCacheManager(capacity=capacity, num_layers=1, num_kv_heads=HEADS, head_dim=DIM,
                                      max_cache_len=max_len, page_size=PAGE, q=Q, key_betas=KEY_BETAS,
                                      value_betas=VALUE_BETAS, dtype=torch.bfloat16, device="cuda", hints=hints)


def _hints_of(codes: torch.Tensor) -> torch.Tensor:
    """The stand-alone hint kernel over a uint8 code stream [pages, bytes] (four bytes per block)."""
    from nestquant_aiinfra_amd import _native
    flat = codes.contiguous()
    out = torch.empty(flat.numel() // 8, dtype=torch.uint8, device=flat.device)
    _native.check(_native.library().nq_nqkv_page_hints(flat.data_ptr(), flat.numel() // 4, out.data_ptr(),
                                                        _native.stream_handle(flat.device)))
    return out.reshape(codes.shape[0], -1)


def test_every_code_word_decodes_the_same_with_its_hint():
    from nestquant_aiinfra_amd import _native
    lib = _native.library()
    mismatches = torch.zeros(1, dtype=torch.int64, device="cuda")
    total = 14 ** 8
    done = 0
    while done < total:                                  # a few launches, so that none runs for long
        count = min(1 << 28, total - done)
        _native.check(lib.nq_nqkv_verify_hints(done, count, mismatches.data_ptr(), _native.stream_handle(mismatches.device)))
        done += count
    assert int(mismatches.item()) == 0
    # the range is checked: one word past the last code word is refused
    assert lib.nq_nqkv_verify_hints(total, 1, mismatches.data_ptr(), None) == _native.NQ_ERR_SHAPE


def _append(manager, slots, keys, values):
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
    manager.begin_step(rows=rows, uniform_count=counts[0] if len(set(counts)) == 1 else None)
    manager.write_layer(0, key.cuda(), value.cuda())


@pytest.mark.parametrize("q_heads,max_len", [(32, 512), (8, 2048), (64, 4096)])
def test_hints_change_nothing_but_the_time(kv, oracle, q_heads, max_len):
    """Two caches fed the same tokens, one with hints: ragged prompts through the writer, a chunk of new
    tokens through the prefill attention, then decode steps through the appending attention launch (some
    complete pages) and the plain decode attention."""
    rng = np.random.default_rng(4100 + q_heads)
    slots = [2, 0, 3, 1]
    lengths = [max_len * 5 // 8 + 3, 16, max_len - 40, 9]
    rows = len(slots)
    plain, hinted = _manager(kv, 4, max_len, False), _manager(kv, 4, max_len, True)
    keys = [_bf16(oracle.hadamard(rng.standard_normal((n, HEADS, DIM)).astype(np.float32))) for n in lengths]
    values = [_bf16(rng.standard_normal((n, HEADS, DIM)).astype(np.float32)) for n in lengths]
    for manager in (plain, hinted):
        for s in slots:
            manager.register(f"seq{s}", slot=s)
        _append(manager, slots, keys, values)

    def same_state(where):
        for name in STREAMS:
            assert torch.equal(getattr(plain.layers[0].pool, name), getattr(hinted.layers[0].pool, name)), (where, name)
        assert torch.equal(plain.layers[0].hot_keys, hinted.layers[0].hot_keys), where
        assert torch.equal(plain.layers[0].hot_values, hinted.layers[0].hot_values), where
        for name in ("sequence_lengths", "page_counts", "last_page_lens", "hot_lengths"):
            assert torch.equal(getattr(plain.metadata, name), getattr(hinted.metadata, name)), (where, name)
        pool = hinted.layers[0].pool
        assert torch.equal(pool.key_hints, _hints_of(pool.key_codes)), where
        assert torch.equal(pool.value_hints, _hints_of(pool.value_codes)), where

    same_state("prompts")
    assert int(hinted.layers[0].pool.key_hints.count_nonzero()) > 0
    assert plain.layers[0].pool.key_hints is None

    # a chunk of 24 more tokens per row, attended causally over the packed cache
    chunk = 24
    more_k = [_bf16(oracle.hadamard(rng.standard_normal((chunk, HEADS, DIM)).astype(np.float32))) for _ in slots]
    more_v = [_bf16(rng.standard_normal((chunk, HEADS, DIM)).astype(np.float32)) for _ in slots]
    query = _bf16(rng.standard_normal((rows, chunk, q_heads, DIM)).astype(np.float32)).cuda()
    outs = []
    for manager in (plain, hinted):
        _append(manager, slots, more_k, more_v)
        for split in (False, True):
            outs.append(kv.nqkv_prefill_attention(query, manager.layers[0], slot_ids=manager.step_slot_ids[:rows],
                                                  active_mask=manager.step_active[:rows], uniform_count=chunk,
                                                  split_context=split))
    assert torch.equal(outs[0], outs[2]) and torch.equal(outs[1], outs[3])
    same_state("chunk")

    workspaces = [kv.BatchedNQKVAttentionWorkspace.create(m.layers[0], batch_size=rows, query_heads=q_heads,
                                                          output_dtype=torch.bfloat16) for m in (plain, hinted)]
    packed = 0
    for step in range(20):
        key = _bf16(rng.standard_normal((rows, HEADS, DIM)).astype(np.float32)).cuda()
        value = _bf16(rng.standard_normal((rows, HEADS, DIM)).astype(np.float32)).cuda()
        query = _bf16(rng.standard_normal((rows, q_heads, DIM)).astype(np.float32)).cuda()
        results = []
        for manager, workspace in zip((plain, hinted), workspaces):
            manager.step_slot_ids[:rows] = torch.tensor(slots, dtype=torch.int32)
            manager.step_active[:rows] = True
            manager.begin_step(rows=rows, uniform_count=1)
            appended = manager.append_and_attend(0, query, key, value, attention_scale=0.125, workspace=workspace,
                                                 rotate=True).clone()
            again = kv.launch_nqkv_decode_attention(query, manager.layers[0], slot_ids=manager.step_slot_ids,
                                                    active_mask=manager.step_active, attention_scale=0.125,
                                                    workspace=workspace, rotate_query=True).clone()
            results.append((appended, again))
        assert torch.equal(results[0][0], results[1][0]), step
        assert torch.equal(results[0][1], results[1][1]), step
        same_state(f"step {step}")
        packed += sum(1 for s in slots if plain.total_tokens(s) % PAGE == 0)
    assert packed >= 2                                   # the appending launch has packed pages on the way


def test_a_page_stored_from_a_container_gets_its_hints(kv, oracle):
    rng = np.random.default_rng(4200)
    key = _bf16(oracle.hadamard(rng.standard_normal((PAGE, HEADS, DIM)).astype(np.float32))).cuda()
    value = _bf16(rng.standard_normal((PAGE, HEADS, DIM)).astype(np.float32)).cuda()
    page = kv.quantize_nqkv_page_cuda(key, value, page_size=PAGE, q=Q, key_betas=KEY_BETAS, value_betas=VALUE_BETAS)
    pool = kv.NQKVPagePool(capacity=3, page_size=PAGE, num_kv_heads=HEADS, head_dim=DIM, q=Q, key_betas=KEY_BETAS,
                           value_betas=VALUE_BETAS, hints=True)
    pool.allocate()
    handle = pool.allocate()
    pool.store_prepared(handle, page)
    assert torch.equal(pool.key_hints, _hints_of(pool.key_codes))
    assert torch.equal(pool.value_hints, _hints_of(pool.value_codes))
    assert int(pool.key_hints[handle.page_id].count_nonzero()) > 0 and not pool.key_hints[0].any()
    assert pool.resident_bytes == kv.NQKVPagePool(
        capacity=3, page_size=PAGE, num_kv_heads=HEADS, head_dim=DIM, q=Q, key_betas=KEY_BETAS,
        value_betas=VALUE_BETAS).resident_bytes + 2 * 3 * PAGE * HEADS * DIM // 16


def test_hint_streams_come_in_pairs_and_sizes_are_checked(kv):
    from nestquant_aiinfra_amd import _native
    lib = _native.library()
    codes = torch.zeros(64, dtype=torch.uint8, device="cuda")
    hints = torch.zeros(8, dtype=torch.uint8, device="cuda")
    assert lib.nq_nqkv_page_hints(codes.data_ptr(), 15, hints.data_ptr(), None) == _native.NQ_ERR_SHAPE
    assert lib.nq_nqkv_page_hints(codes.data_ptr() + 4, 2, hints.data_ptr(), None) == _native.NQ_ERR_ARGUMENT
    assert lib.nq_nqkv_page_hints(None, 0, None, None) == _native.NQ_OK
    with pytest.raises(ValueError, match="decode hints need q = 14"):
        kv.NQKVPagePool(capacity=1, page_size=PAGE, num_kv_heads=HEADS, head_dim=DIM, q=16, key_betas=KEY_BETAS,
                        value_betas=VALUE_BETAS, hints=True)


def test_runner_gives_the_same_logits_with_and_without_hints(tmp_path):
    """A tiny Llama through the runner, once with a cache that keeps hints and once without: the prompt's
    logits, every decode step's logits (captured graph and un-captured, with pages completed on the way)
    and a chunk fed into slots that already hold tokens (prefill attention over the packed cache)."""
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm

    torch.manual_seed(5101)
    config = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                         num_key_value_heads=2, head_dim=64, vocab_size=128, max_position_embeddings=512,
                         rope_theta=500000.0, tie_word_embeddings=True)
    model = LlamaForCausalLM(config).to(torch.bfloat16).cuda().eval()
    path = tmp_path / "tiny.nqmc"
    asm.write_w4_checkpoint(model, path)
    asm.build_w4a4kv4_runner(model, path, capacity=2, max_cache_len=160, decode_hints=False)
    g = torch.Generator().manual_seed(5102)
    prompt = torch.randint(0, 128, (2, 41), generator=g).cuda()
    more = torch.randint(0, 128, (2, 19), generator=g).cuda()
    steps = torch.randint(0, 128, (30, 2, 1), generator=g).cuda()
    record = {}
    for hints in (False, True):
        runner = asm.attach_w4a4kv4_cache(model, capacity=2, max_cache_len=160, decode_hints=hints)
        pool = runner.cache.manager.layers[0].pool
        assert (pool.key_hints is not None) == hints
        outs = [runner.prefill_slots(prompt, slots=[0, 1], lengths=[41, 33]).float().clone()]
        outs.append(runner.prefill_slots(more, slots=[0, 1], lengths=[19, 7]).float().clone())
        held = [60, 40]
        for index, token in enumerate(steps):
            if index == 10:
                runner.capture()
            positions = torch.tensor(held, device="cuda").reshape(2, 1)
            call = runner.decode if index >= 10 else runner.decode_eager
            outs.append(call(token, slots=[0, 1], positions=positions).float().clone())
            held = [h + 1 for h in held]
        record[hints] = outs
        runner.release_slots([0, 1])
    for a, b in zip(record[False], record[True]):
        assert torch.equal(a, b)
