"""The packed W4A4KV4 path at the size its headline number is quoted on: the Llama-3.2-1B
architecture (16 layers, hidden 2048, 32 / 8 heads of 64, MLP 8192, vocabulary 128256, tied head,
RoPE theta 500000) with random weights, batch 8, ragged prompts, 24 decode steps that cross a page
boundary in every row.  The reference pins this level by invariants
(tests/unit/runtime/test_nqkv_batched_hf_backend.py:569-739): graph replay equals eager execution
bit for bit, logits and cache state; and the fused steps track the module graph.  The two differ
in the summation order of the RMSNorm mean only: most rows come out equal, and a row in which that
order moved one BF16 rounding sees the E8 codes behind it flip, a difference that every further
layer of random weights, and every further step on the cache that row has written, widens to the
size of the 4-bit noise itself.  Hence the bars over the 64 (step, row) logit vectors: median
cosine >= 0.9999, at least 75 % within the two-layer model's tolerance (cosine > 0.995), none
below 0.8, the same argmax in at least 85 %."""

import pytest
import torch

from gpu_util import bits, relative_error

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]

BATCH, STEPS, VOCAB = 8, 24, 128256
LENGTHS = [33, 9, 40, 16, 27, 31, 12, 38]           # hot tails of 1, 9, 8, 0, 11, 15, 12, 6 rows


@pytest.fixture(scope="module")
def llama_1b(tmp_path_factory):
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm

    torch.manual_seed(5101)
    config = LlamaConfig(hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32,
                         num_key_value_heads=8, head_dim=64, vocab_size=VOCAB, max_position_embeddings=4096,
                         rope_theta=500000.0, tie_word_embeddings=True)
    with torch.device("cuda"):
        model = LlamaForCausalLM(config).to(torch.bfloat16).eval()
    path = tmp_path_factory.mktemp("nqmc") / "llama_1b_random.nqmc"
    names = asm.write_w4_checkpoint(model, path)
    assert len(names) == 16 * 7
    runner = asm.build_w4a4kv4_runner(model, path, capacity=BATCH, max_cache_len=96)
    return model, runner


def _cache_tensors(cache):
    meta = cache.manager.metadata
    tensors = [meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths]
    for layer in cache.manager.layers:
        pool = layer.pool
        tensors += [layer.hot_keys, layer.hot_values, pool.key_codes, pool.key_betas, pool.key_norms,
                    pool.value_codes, pool.value_betas, pool.value_norms]
    return tensors


def test_graph_equals_eager_and_fused_tracks_modules_at_full_size(llama_1b):
    from nestquant_aiinfra_amd.runtime.nqkv_hf_backend import BatchedNQKVLlamaRunner
    model, runner = llama_1b
    cache = runner.cache
    slots = list(range(BATCH))
    g = torch.Generator().manual_seed(5102)
    ids = torch.randint(0, VOCAB, (BATCH, max(LENGTHS)), generator=g).cuda()
    logits = runner.prefill_slots(ids, slots=slots, lengths=LENGTHS)
    assert tuple(logits.shape) == (BATCH, max(LENGTHS), VOCAB)
    first = torch.stack([logits[row, n - 1].argmax() for row, n in enumerate(LENGTHS)]).reshape(BATCH, 1)
    assert all(torch.isfinite(logits[row, :n]).all() for row, n in enumerate(LENGTHS))
    del logits
    start = torch.tensor(LENGTHS, device="cuda").reshape(BATCH, 1)
    runner.capture()
    assert runner.graph_captured and cache.manager.metadata.sequence_lengths[:BATCH].tolist() == LENGTHS

    tensors = _cache_tensors(cache)
    saved, host = [t.clone() for t in tensors], list(cache._host_lengths)

    def restore():
        for tensor, value in zip(tensors, saved):
            tensor.copy_(value)
        cache._host_lengths[:] = host

    def generate(step_fn):
        token, position, tokens, last = first, start, [], None
        for _ in range(STEPS):
            last = step_fn(token, slots=slots, positions=position)
            token = last[:, 0].argmax(-1).reshape(BATCH, 1)
            tokens.append(token.clone())
            position = position + 1
        return torch.cat(tokens, dim=1), last.clone(), [t.clone() for t in tensors]

    graph_tokens, graph_last, graph_state = generate(runner.decode)
    assert runner.graph_replay_counts[BATCH] == STEPS and torch.isfinite(graph_last).all()
    meta = cache.manager.metadata
    assert meta.sequence_lengths[:BATCH].tolist() == [n + STEPS for n in LENGTHS]
    assert meta.page_counts[:BATCH].tolist() == [(n + STEPS) // 16 for n in LENGTHS]      # every row packed a page
    restore()
    eager_tokens, eager_last, eager_state = generate(runner.decode_eager)
    assert torch.equal(graph_tokens, eager_tokens) and torch.equal(graph_last, eager_last)   # bit for bit
    for a, b in zip(graph_state, eager_state):
        assert torch.equal(a, b)                                          # hot tails, packed pages, tables

    # fused steps against the module graph: the same inputs at every step, from the same cache state
    modular = BatchedNQKVLlamaRunner(model, cache, fused_decode=False)
    assert runner.fused_step is not None and modular.fused_step is None

    def teacher_forced(which, steps=8):
        outs, position = [], start
        for step in range(steps):
            outs.append(which.decode_eager(graph_tokens[:, step:step + 1].contiguous(), slots=slots,
                                           positions=position)[:, 0].float().clone())
            position = position + 1
        return torch.stack(outs)

    restore()
    fused = teacher_forced(runner)
    restore()
    reference = teacher_forced(modular)
    cosine = torch.nn.functional.cosine_similarity(fused.flatten(0, 1), reference.flatten(0, 1), dim=1)
    assert float(cosine.median()) >= 0.9999 and float((cosine > 0.995).float().mean()) >= 0.75, cosine
    assert float(cosine.min()) > 0.8, cosine
    assert (fused.argmax(-1) == reference.argmax(-1)).float().mean() >= 0.85
    runner.release_slots(slots)
