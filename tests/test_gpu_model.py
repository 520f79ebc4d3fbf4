"""End-to-end W4A4KV4 on a tiny random-init Llama (the reference's offline test route,
tests/unit/runtime/test_nqkv_batched_hf_backend.py:47-57): packed projections + NQKV4 cache
+ captured decode graph.  The reference pins this level by invariants, not vectors: graph
replay equals eager execution bit for bit across page boundaries and slot reuse
(:569-739); outputs are finite and shaped; dispatch counters move."""

import numpy as np
import pytest
import torch

from conftest import ACTIVATION_BETAS, Q
from gpu_util import bits, relative_error

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm

    torch.manual_seed(5001)
    config = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                         num_key_value_heads=2, head_dim=64, vocab_size=128, max_position_embeddings=512,
                         rope_theta=500000.0, tie_word_embeddings=True)
    model = LlamaForCausalLM(config).to(torch.bfloat16).cuda().eval()
    dense = {name: module.weight.detach().float().clone() for name, module in model.named_modules()
             if isinstance(module, torch.nn.Linear) and name.rsplit(".", 1)[-1] in asm.PROJECTIONS}
    path = tmp_path_factory.mktemp("nqmc") / "tiny.nqmc"
    names = asm.write_w4_checkpoint(model, path)
    runner = asm.build_w4a4kv4_runner(model, path, capacity=4, max_cache_len=128)
    return model, runner, names, dense, path


def test_checkpoint_and_conversion(tiny):
    from nestquant_aiinfra_amd.core.model_checkpoint import NQMCFileReader
    from nestquant_aiinfra_amd.models.fused_linear import FusedNQRTLinear
    model, runner, names, dense, path = tiny
    assert len(names) == 2 * 7
    reader = NQMCFileReader(path)
    entry = reader.get_entry("model.layers.0.mlp.down_proj.weight")
    assert entry.kind == "nestquant" and entry.shape == (256, 512)
    assert reader.get_entry("lm_head.weight").kind == "dense"          # tied alias resolves to the embeddings
    fused = [m for m in model.modules() if isinstance(m, FusedNQRTLinear)]
    assert len(fused) == 14 and all(m.input_hadamard for m in fused)
    # the stored record dequantises (rotated back) close to the original weight: ~4-bit error
    _, record = reader.read_named_record("model.layers.0.self_attn.q_proj.weight")
    from nestquant_aiinfra_amd.core.rotation import hadamard
    restored = hadamard(record.dequantize(device="cuda"))
    original = dense["model.layers.0.self_attn.q_proj"].cuda()
    assert float((restored - original).norm() / original.norm()) < 0.12


def _prompt(rows, width, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, 128, (rows, width), generator=g).cuda()


def test_prefill_then_graph_decode_equals_eager(tiny):
    model, runner, *_ = tiny
    cache = runner.cache
    lengths = [13, 30]                                   # one sub-page prompt, one crossing a page
    ids = _prompt(2, 30, 5002)
    logits = runner.prefill_slots(ids, slots=[2, 0], lengths=lengths)
    assert tuple(logits.shape) == (2, 30, 128) and torch.isfinite(logits[0, :13]).all() and torch.isfinite(logits[1]).all()
    runner.capture()
    assert runner.graph_captured and sorted(runner._graphs) == [1, 2, 4]
    assert cache.manager.total_tokens(2) == 13 and cache.manager.total_tokens(0) == 30       # capture left the cache alone

    # snapshot the cache, run 40 graph steps (two page boundaries per slot), restore, run eagerly
    meta = cache.manager.metadata
    def snapshot():
        tensors = [meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths]
        for layer in cache.manager.layers:
            pool = layer.pool
            tensors += [layer.hot_keys, layer.hot_values, pool.key_codes, pool.key_betas, pool.key_norms,
                        pool.value_codes, pool.value_betas, pool.value_norms]
        return tensors, [t.clone() for t in tensors], list(cache._host_lengths)
    tensors, saved, host = snapshot()

    def run(step_fn, steps=40):
        token = torch.stack([logits[0, 12].argmax(), logits[1, 29].argmax()]).reshape(2, 1)
        outs, position = [], torch.tensor([[13], [30]], device="cuda")
        for _ in range(steps):
            out = step_fn(token, slots=[2, 0], positions=position).clone()
            outs.append(out)
            token = out[:, 0].argmax(-1).reshape(2, 1)
            position = position + 1
        return torch.stack(outs), [t.clone() for t in tensors]

    graph_logits, graph_state = run(runner.decode)
    assert runner.graph_replay_counts[2] == 40 and torch.isfinite(graph_logits).all()
    assert cache.manager.total_tokens(2) == 53 and int(meta.page_counts[0]) == 70 // 16
    for tensor, value in zip(tensors, saved):
        tensor.copy_(value)
    cache._host_lengths[:] = host
    eager_logits, eager_state = run(runner.decode_eager)
    assert torch.equal(graph_logits, eager_logits)                       # bit for bit
    for a, b in zip(graph_state, eager_state):
        assert torch.equal(a, b)                                         # hot tails, packed pages, tables

    # slot reuse: release, prefill something else into the same slot, decode through the graph again
    runner.release_slots([2])
    assert cache.manager.total_tokens(2) == 0
    again = runner.prefill_slots(_prompt(1, 20, 5003), slots=[2], lengths=[20])
    out = runner.decode(again[:, 19].argmax(-1).reshape(1, 1), slots=[2], positions=torch.tensor([[20]], device="cuda"))
    assert tuple(out.shape) == (1, 1, 128) and torch.isfinite(out).all() and runner.graph_replay_counts[1] == 1
    runner.release_slots([0, 2])


def test_decode_logits_track_a_full_prefill(tiny):
    """Decoding token t on the quantised cache stays close to prefilling the same prefix in one
    shot (which attends to BF16 K/V): KV4 changes logits a little, never their shape."""
    model, runner, *_ = tiny
    ids = _prompt(1, 40, 5004)
    full = runner.prefill_slots(ids, slots=[1], lengths=[40])[0, 39].float()
    runner.release_slots([1])
    runner.prefill_slots(ids[:, :39], slots=[1], lengths=[39])
    step = runner.decode(ids[:, 39:40], slots=[1], positions=torch.tensor([[39]], device="cuda"))[0, 0].float()
    runner.release_slots([1])
    cosine = torch.nn.functional.cosine_similarity(full, step, dim=0)
    assert float(cosine) > 0.97


def test_chunked_prefill_attends_to_the_packed_cache(tiny):
    """A prompt fed in pieces: later pieces attend to what the cache already holds (packed pages
    and hot tail).  Logits stay close to the one-shot prefill (which attends to BF16 K/V), and
    decoding continues from either state."""
    model, runner, *_ = tiny
    ids = _prompt(1, 50, 5005)
    whole = runner.prefill_slots(ids, slots=[3], lengths=[50])[0, 49].float()
    runner.release_slots([3])
    first = runner.prefill_slots(ids[:, :21], slots=[3], lengths=[21])
    assert not runner.cache._continuation
    second = runner.prefill_slots(ids[:, 21:44], slots=[3], lengths=[23])
    assert runner.cache._continuation and runner.cache.manager.total_tokens(3) == 44
    third = runner.prefill_slots(ids[:, 44:], slots=[3], lengths=[6])[0, 5].float()
    assert torch.isfinite(first).all() and torch.isfinite(second).all()
    cosine = torch.nn.functional.cosine_similarity(whole, third, dim=0)
    assert float(cosine) > 0.97
    step = runner.decode(third.argmax().reshape(1, 1), slots=[3], positions=torch.tensor([[50]], device="cuda"))
    assert torch.isfinite(step).all() and runner.cache.manager.total_tokens(3) == 51
    runner.release_slots([3])
    # the same route for a whole prompt, on request
    runner.cache.packed_prefill = True
    try:
        packed = runner.prefill_slots(ids, slots=[3], lengths=[50])[0, 49].float()
    finally:
        runner.cache.packed_prefill = False
        runner.release_slots([3])
    assert float(torch.nn.functional.cosine_similarity(whole, packed, dim=0)) > 0.97


def test_dispatch_counters_and_m_routes(tiny):
    from nestquant_aiinfra_amd.models.fused_linear import FusedNQRTLinear
    model, runner, *_ = tiny
    layer = next(m for name, m in model.named_modules() if isinstance(m, FusedNQRTLinear) and name.endswith("o_proj"))
    base = (layer.w4a4_cuda_mma_m1_dispatch_count, layer.w4a4_cuda_mma_small_m_dispatch_count,
            layer.w4a4_cuda_mma_m16_dispatch_count, layer.w4a4_cuda_mma_large_m_staged_dispatch_count,
            layer.w4a4_cuda_mma_chunked_staged_dispatch_count)
    for m in (1, 4, 16, 64, 40):
        x = torch.randn(m, 256, device="cuda").to(torch.bfloat16)
        with torch.inference_mode():
            y = layer(x)
        assert tuple(y.shape) == (m, layer.out_features) and y.dtype == torch.bfloat16
    after = (layer.w4a4_cuda_mma_m1_dispatch_count, layer.w4a4_cuda_mma_small_m_dispatch_count,
             layer.w4a4_cuda_mma_m16_dispatch_count, layer.w4a4_cuda_mma_large_m_staged_dispatch_count,
             layer.w4a4_cuda_mma_chunked_staged_dispatch_count)
    assert tuple(b - a for a, b in zip(base, after)) == (1, 1, 1, 1, 1)
    assert layer.prepared and layer.packed_device_bytes > 0
    # a resolved weight keeps 6 bytes per block of eight weights, its row norms and the beta table on the
    # device: the NQRT4 streams it was derived from are not resident
    state = layer._prepared
    assert state.code_payload is None and state.beta_payload is None
    weights = layer.out_features * layer.in_features
    assert layer.packed_device_bytes == weights * 6 // 8 + 4 * layer.out_features + 16


def test_fused_rotation_matches_separate_rotation(oracle):
    """Encoding with the rotation fused equals rotating first with the stand-alone kernel,
    which equals the tensor-op Hadamard in the same dtype."""
    from nestquant_aiinfra_amd.core import rotation
    from nestquant_aiinfra_amd.runtime import w4a4_linear as rt

    def hadamard(x):
        # the butterfly network written with tensor operations (what rotation.hadamard runs for host
        # tensors), evaluated on the GPU: rotation.hadamard itself hands GPU tensors to the kernel
        n = x.shape[-1]
        return rotation._staged(x.reshape(-1, n).contiguous(), n).reshape(x.shape)

    assert torch.equal(rotation.hadamard(torch.ones(2, 64, device="cuda")), hadamard(torch.ones(2, 64, device="cuda")))
    for dtype in (torch.bfloat16, torch.float32):
        x = torch.randn(5, 2048, device="cuda").to(dtype)
        rotated = rt.hadamard_cuda(x)
        assert torch.equal(rotated, hadamard(x))
        fused = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS, hadamard=True)
        plain = rt.quantize_activation_cuda(rotated, q=Q, betas=ACTIVATION_BETAS)
        assert torch.equal(fused.code_payload, plain.code_payload) and torch.equal(fused.row_norms, plain.row_norms)
        assert torch.equal(fused.beta_payload, plain.beta_payload) and torch.equal(fused.decoded, plain.decoded)
    # every row length takes its own mix of register, lane and LDS stages
    for n in (2, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 4096, 8192, 16384, 32768):
        for dtype in (torch.bfloat16, torch.float16, torch.float32):
            x = torch.randn(3, n, device="cuda").to(dtype)
            assert torch.equal(rt.hadamard_cuda(x), hadamard(x)), (n, dtype)
    # float32 butterflies over a 64-wide head, rounded to BF16 once (the key / query rotation)
    k = torch.randn(3, 2, 7, 64, device="cuda").to(torch.bfloat16)
    assert torch.equal(rt.hadamard_cuda(k, compute_dtype=torch.float32), hadamard(k.float()).to(torch.bfloat16))
    assert relative_error(bits(rt.hadamard_cuda(k.float())), oracle.hadamard(bits(k.float()))) < 1e-6


def test_captured_prefill_equals_the_uncaptured_one(tiny):
    """`capture_prefill(rows, width)` replays the fused prefill as one graph: the same last-token logits and
    the same cache (pools, hot tails, tables) as the un-captured call, for ragged lengths that change from
    call to call; other shapes and continuation chunks keep the un-captured path."""
    model, runner, *_ = tiny
    cache = runner.cache
    pools = [layer.pool for layer in cache.manager.layers]
    meta = cache.manager.metadata

    def state():
        tensors = [getattr(pool, name).clone() for pool in pools
                   for name in ("key_codes", "key_betas", "key_norms", "value_codes", "value_betas", "value_norms")]
        tensors += [t.clone() for layer in cache.manager.layers for t in (layer.hot_keys, layer.hot_values)]
        tensors += [t.clone() for t in (meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths)]
        return tensors

    def wipe():                                          # pages of released slots keep their bytes: start both passes from zeros
        for pool in pools:
            for name in ("key_codes", "key_betas", "key_norms", "value_codes", "value_betas", "value_norms", "key_hints",
                         "value_hints"):
                if getattr(pool, name) is not None:
                    getattr(pool, name).zero_()
        for layer in cache.manager.layers:
            layer.hot_keys.zero_()
            layer.hot_values.zero_()

    runner.release_slots([s for s in range(4) if cache.manager.sequence_id(s) is not None])
    cases = [([1, 3], [40, 23]), ([0, 2], [17, 48]), ([2, 1], [48, 1])]
    eager = []
    wipe()
    for seed, (slots, lengths) in enumerate(cases):
        ids = _prompt(2, 48, 6100 + seed)
        logits = runner.prefill_slots(ids, slots=slots, lengths=lengths, last_token_logits=True).clone()
        eager.append((logits, state()))
        runner.release_slots(slots)
    before = state()
    runner.capture_prefill(rows=2, width=48)
    assert all(torch.equal(a, b) for a, b in zip(before, state()))          # capturing leaves the cache alone
    wipe()
    for seed, (slots, lengths) in enumerate(cases):
        ids = _prompt(2, 48, 6100 + seed)
        logits = runner.prefill_slots(ids, slots=slots, lengths=lengths, last_token_logits=True)
        want_logits, want_state = eager[seed]
        assert torch.equal(logits, want_logits), seed
        assert all(torch.equal(a, b) for a, b in zip(state(), want_state)), seed
        runner.release_slots(slots)
    assert runner.prefill_graph_replay_counts[(2, 48)] == 3
    # another width, all-position logits and a chunk into slots that hold tokens do not take the graph
    ids = _prompt(2, 40, 6200)
    runner.prefill_slots(ids, slots=[0, 1], lengths=[40, 12], last_token_logits=True)
    runner.prefill_slots(_prompt(2, 48, 6201), slots=[0, 1], lengths=[30, 48], last_token_logits=True)   # continuation
    runner.release_slots([0, 1])
    runner.prefill_slots(_prompt(2, 48, 6202), slots=[0, 1], lengths=[30, 48])
    runner.release_slots([0, 1])
    assert runner.prefill_graph_replay_counts[(2, 48)] == 3
    with pytest.raises(ValueError, match="rows must be in"):
        runner.capture_prefill(rows=9, width=16)
