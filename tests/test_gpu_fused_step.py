"""GPU checks of the fused decode-step pieces, through the C ABI:
  * nq_fused_input_stage against the BF16 tensor operations it replaces (LlamaRMSNorm with a
    residual add, SiLU-and-multiply) followed by the plain encoder;
  * nq_w4a4_gemv_grouped against one nq_w4a4_gemv call per weight (bit for bit);
  * the rotary embedding inside nq_nqkv_write / nq_nqkv_attention_decode against the same
    BF16 tensor arithmetic done beforehand (bit for bit);
  * nq_rope_hadamard against the BF16 rotary embedding and float32 Hadamard it replaces;
  * FusedLlamaDecodeStep and FusedLlamaPrefillStep against the module graph of the same tiny
    model (tolerance: the row reductions of the norm run in a different order).
"""

import numpy as np
import pytest
import torch

from conftest import ACTIVATION_BETAS, Q, WEIGHT_BETAS
from gpu_util import bits, oracle_weight, relative_error

pytestmark = pytest.mark.gpu

KEY_BETAS = tuple(v / 14 for v in (3.50, 4.58, 6.47, 17.06))
VALUE_BETAS = tuple(v / 14 for v in (3.53, 5.59, 9.62, 29.03))


@pytest.fixture(scope="module")
def rt():
    from nestquant_aiinfra_amd.runtime import w4a4_linear
    return w4a4_linear


def _table():
    return torch.tensor(ACTIVATION_BETAS, dtype=torch.float32, device="cuda")


def _same_activation(a, b):
    return (torch.equal(a.code_payload, b.code_payload) and torch.equal(a.beta_payload, b.beta_payload)
            and torch.equal(a.row_norms, b.row_norms) and torch.equal(a.decoded, b.decoded))


def _rms_norm(h, weight, eps):
    x = h.float()
    x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return weight * x.to(h.dtype)


@pytest.mark.parametrize("rows,n", [(1, 2048), (8, 2048), (3, 256), (5, 8192), (40, 512), (1100, 2048), (4200, 512),
                                    (64, 2048), (150, 4096), (128, 8192), (300, 2048), (500, 8192)])   # prefill chunks
@pytest.mark.parametrize("with_residual", [False, True])
def test_residual_rmsnorm_stage(rt, rows, n, with_residual):
    g = torch.Generator().manual_seed(rows * n + with_residual)
    x = torch.randn(rows, n, generator=g).to(torch.bfloat16).cuda()
    residual = (3 * torch.randn(rows, n, generator=g)).to(torch.bfloat16).cuda() if with_residual else None
    weight = (1 + 0.1 * torch.randn(n, generator=g)).to(torch.bfloat16).cuda()
    eps = 1e-5
    activation, h, staged = rt.fused_input_stage(x, mode="rmsnorm", residual=residual, norm_weight=weight, eps=eps,
                                                 beta_table=_table(), want_residual=True, want_staged=True)
    expect_h = x + residual if with_residual else x
    assert torch.equal(h, expect_h)
    expect = _rms_norm(expect_h, weight, eps)
    # only where the differently ordered mean moved a rounding: one BF16 step, or (a few values per
    # million) two when the step of the normalised value is stretched by a weight above one
    difference = (staged.float() - expect.float()).abs()
    assert bool((difference <= expect.float().abs() * 2.0 ** -6 + 1e-30).all())
    assert int((difference > expect.float().abs() * 2.0 ** -7 + 1e-30).sum()) <= rows * n // 100000
    assert int((staged != expect).sum()) <= max(2, rows * n // 200)
    # the encode that follows is the plain encoder on the staged rows
    plain = rt.quantize_activation_cuda(staged, q=Q, betas=ACTIVATION_BETAS, hadamard=True)
    assert _same_activation(activation, plain)
    # element-wise stage alone
    none, _, staged_only = rt.fused_input_stage(x, mode="rmsnorm", residual=residual, norm_weight=weight, eps=eps,
                                                encode=False, want_staged=True)
    assert none is None and torch.equal(staged_only, staged)


@pytest.mark.parametrize("rows,n", [(1, 8192), (8, 8192), (2, 512), (300, 8192), (40, 2048), (100, 8192), (192, 4096)])
def test_swiglu_stage(rt, rows, n):
    g = torch.Generator().manual_seed(rows + n)
    gate = (2 * torch.randn(rows, n, generator=g)).to(torch.bfloat16).cuda()
    up = torch.randn(rows, n, generator=g).to(torch.bfloat16).cuda()
    activation, _, staged = rt.fused_input_stage(up, mode="swiglu", gate=gate, beta_table=_table(), want_staged=True)
    expect = torch.nn.functional.silu(gate) * up
    difference = (staged.float() - expect.float()).abs()
    assert bool((difference <= expect.float().abs() * 2.0 ** -6 + 1e-30).all())      # exp differs in the last place
    assert int((staged != expect).sum()) <= max(2, rows * n // 100)
    plain = rt.quantize_activation_cuda(staged, q=Q, betas=ACTIVATION_BETAS, hadamard=True)
    assert _same_activation(activation, plain)


def test_fused_stage_argument_checks(rt):
    x = torch.zeros(2, 256, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        rt.fused_input_stage(x, mode="layernorm", beta_table=_table())
    with pytest.raises(ValueError):
        rt.fused_input_stage(x, mode="rmsnorm", beta_table=_table())                 # no norm weight
    with pytest.raises(ValueError):
        rt.fused_input_stage(x, mode="swiglu", beta_table=_table())                  # no gate
    with pytest.raises(TypeError):
        rt.fused_input_stage(x.float(), mode="swiglu", gate=x.float(), beta_table=_table())


@pytest.mark.parametrize("m", [1, 3, 8])
def test_grouped_gemv_equals_single_launches(rt, oracle, m):
    from test_gpu_gemv import _record
    from gpu_util import student_t_rows
    k = 2048
    weights = []
    for index, n_out in enumerate((512, 136, 2050)):
        seed = 20261101 + index
        _, wc, wb, wn = oracle_weight(oracle, n_out, k, seed=900 + index, dither_seed=seed)
        weights.append(rt.prepare_fused_linear(_record(rt, wc, wb, wn, k, seed), device="cuda"))
    x = torch.from_numpy(oracle.hadamard(student_t_rows(m, k, seed=31 + m).numpy())).to(torch.bfloat16).cuda()
    activation = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS)
    for dtype, view in ((torch.float32, torch.int32), (torch.bfloat16, torch.int16)):
        grouped = rt.linear_packed_w4a4_gemv_grouped(activation, weights, output_dtype=dtype)
        for out, weight in zip(grouped, weights):
            single = rt._gemv(activation, weight, split_k=1, output_dtype=dtype)
            if m < 5:
                assert torch.equal(out.view(view), single.view(view))
            else:       # on the matrix cores the tile shape, and with it the summation order, follows the channel count
                assert relative_error(bits(out.float()), bits(single.float())) < (1e-5 if dtype == torch.float32 else 1e-2)
    with pytest.raises(ValueError):
        rt.linear_packed_w4a4_gemv_grouped(activation, weights * 2)


@pytest.mark.parametrize("m", [5, 8, 11, 16])
def test_grouped_gemv_on_the_matrix_cores(rt, oracle, m):
    """From five rows on, weights that together fill the chip in tiles of 16 channels (here
    3568 channels, one tile ragged) multiply on the matrix cores; above eight rows every
    weight does.  Same decoded operands as the vector-unit kernel, another summation order."""
    from test_gpu_gemv import _record, _references, TOLERANCE, BF16_TOLERANCE
    from gpu_util import student_t_rows
    k = 2048
    weights, streams = [], []
    for index, n_out in enumerate((2048, 520, 1000)):
        seed = 20261201 + index
        _, wc, wb, wn = oracle_weight(oracle, n_out, k, seed=700 + index, dither_seed=seed)
        weights.append(rt.prepare_fused_linear(_record(rt, wc, wb, wn, k, seed), device="cuda"))
        streams.append((wc, wb, wn, seed))
    x = torch.from_numpy(oracle.hadamard(student_t_rows(m, k, seed=41 + m).numpy())).to(torch.bfloat16).cuda()
    activation = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS)
    grouped = rt.linear_packed_w4a4_gemv_grouped(activation, weights, output_dtype=torch.float32)
    again = rt.linear_packed_w4a4_gemv_grouped(activation, weights, output_dtype=torch.float32)
    for out, twin, weight, (wc, wb, wn, seed) in zip(grouped, again, weights, streams):
        assert torch.equal(out, twin)                                            # deterministic
        ref32, ref16 = _references(oracle, activation, rt, wc, wb, wn, seed)
        assert relative_error(bits(out), ref32) <= TOLERANCE
        assert relative_error(bits(out), ref16) <= BF16_TOLERANCE
        single = rt._gemv(activation, weight, split_k=0, output_dtype=torch.float32)
        assert relative_error(bits(single), bits(out)) < 1e-5                    # narrower tiles, another order
    half = rt.linear_packed_w4a4_gemv_grouped(activation, weights[:1], output_dtype=torch.bfloat16)[0]
    assert relative_error(bits(half.float()), bits(grouped[0])) < 1e-2


@pytest.mark.parametrize("k", [256, 1024, 2048, 16384])
def test_matrix_core_gemv_gives_the_same_bits_alone_and_in_a_group(rt, k):
    """A narrow weight alone runs in tiles of 8 channels x 2 interleaved K ranges, the same weight
    inside a group that fills the chip in tiles of 16 channels x 1 range; the two-range launch takes
    half the wavefronts of the one-range launch, so the same 128-wide pieces of K meet in the same
    accumulators in the same order: bit for bit, also at the K where the wavefront count is clamped."""
    g = torch.Generator().manual_seed(77 + k)
    weights = []
    for index, n_out in enumerate((264, 3072)):
        rotated = rt.hadamard_cuda((0.02 * torch.randn(n_out, k, generator=g)).cuda(), compute_dtype=torch.float32)
        record = rt.quantize_weight_nqrt4(rotated, q=Q, betas=WEIGHT_BETAS, dither_seed=20261301 + index,
                                          tensor_name=f"w{index}")
        weights.append(rt.prepare_fused_linear(record, device="cuda"))
    x = torch.randn(8, k, generator=g).to(torch.bfloat16).cuda()
    activation = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS, hadamard=True)
    for dtype in (torch.float32, torch.bfloat16):
        grouped = rt.linear_packed_w4a4_gemv_grouped(activation, weights, output_dtype=dtype)
        for out, weight in zip(grouped, weights):
            alone = rt._gemv(activation, weight, split_k=1, output_dtype=dtype)
            assert torch.equal(out, alone)


def _rope_tables(rows, tokens, dim, seed):
    g = torch.Generator().manual_seed(seed)
    angle = 6.0 * torch.rand(rows, tokens, dim // 2, generator=g)
    angle = torch.cat([angle, angle], dim=-1)
    return angle.cos().to(torch.bfloat16).cuda(), angle.sin().to(torch.bfloat16).cuda()


def _apply_rope(x, cos, sin):
    half = x.shape[-1] // 2
    rotated = torch.cat([-x[..., half:], x[..., :half]], dim=-1)
    return (x * cos) + (rotated * sin)


def test_rotary_embedding_inside_writer_and_attention():
    from nestquant_aiinfra_amd.runtime import nqkv as kv
    heads, q_heads, dim, page = 2, 8, 64, 16
    def manager():
        return kv.BatchedNQKVCacheManager(capacity=2, num_layers=1, num_kv_heads=heads, head_dim=dim,
                                          max_cache_len=96, page_size=page, q=Q, key_betas=KEY_BETAS,
                                          value_betas=VALUE_BETAS, dtype=torch.bfloat16, device="cuda")
    fused, plain = manager(), manager()
    for m in (fused, plain):
        m.register("a", slot=0)
        m.register("b", slot=1)
    g = torch.Generator().manual_seed(77)
    for step, tokens in enumerate((21, 1, 1, 11, 1)):                       # crosses pages in both slots
        key = torch.randn(2, tokens, heads, dim, generator=g).to(torch.bfloat16).cuda()
        value = torch.randn(2, tokens, heads, dim, generator=g).to(torch.bfloat16).cuda()
        cos, sin = _rope_tables(2, tokens, dim, seed=100 + step)
        for m in (fused, plain):
            m.step_slot_ids[:2] = torch.tensor([1, 0], dtype=torch.int32)
            m.step_active[:2] = True
            m.begin_step(rows=2, uniform_count=tokens)
        fused.write_layer(0, key, value, rotate_keys=True, rope=(cos, sin))
        plain.write_layer(0, _apply_rope(key, cos[:, :, None, :], sin[:, :, None, :]).contiguous(), value,
                          rotate_keys=True)
    a, b = fused.layers[0], plain.layers[0]
    for name in ("key_codes", "key_betas", "key_norms", "value_codes", "value_betas", "value_norms"):
        assert torch.equal(getattr(a.pool, name), getattr(b.pool, name)), name
    assert torch.equal(a.hot_keys, b.hot_keys) and torch.equal(a.hot_values, b.hot_values)

    query = torch.randn(2, q_heads, dim, generator=g).to(torch.bfloat16).cuda()
    cos, sin = _rope_tables(2, 1, dim, seed=999)
    workspace = kv.BatchedNQKVAttentionWorkspace.create(a, batch_size=2, query_heads=q_heads,
                                                        output_dtype=torch.bfloat16)
    common = dict(slot_ids=fused.step_slot_ids[:2], active_mask=fused.step_active[:2], attention_scale=0.125,
                  workspace=workspace, rotate_query=True)
    inside = kv.launch_nqkv_decode_attention(query, a, rope=(cos.view(2, dim), sin.view(2, dim)), **common).clone()
    before = kv.launch_nqkv_decode_attention(_apply_rope(query, cos, sin).contiguous(), a, **common).clone()
    assert torch.equal(inside, before) and bool(inside.float().abs().sum() > 0)


@pytest.mark.parametrize("heads,dim", [(8, 64), (3, 128)])
def test_rope_and_rotation_of_head_vectors_in_one_launch(rt, heads, dim):
    from nestquant_aiinfra_amd.core.rotation import _staged

    def hadamard(x):            # the tensor-operation butterflies, on the GPU (not the stand-alone kernel)
        return _staged(x.reshape(-1, x.shape[-1]).contiguous(), x.shape[-1]).reshape(x.shape)

    rows = 37
    g = torch.Generator().manual_seed(heads * dim)
    x = torch.randn(rows, heads, dim, generator=g).to(torch.bfloat16).cuda()
    cos, sin = _rope_tables(rows, 1, dim, seed=5)
    cos, sin = cos.view(rows, dim), sin.view(rows, dim)
    embedded = _apply_rope(x, cos[:, None, :], sin[:, None, :])
    assert torch.equal(rt.rope_hadamard_cuda(x, rope=(cos, sin), hadamard=False), embedded)
    assert torch.equal(rt.rope_hadamard_cuda(x, hadamard=True), hadamard(x.float()).to(torch.bfloat16))
    assert torch.equal(rt.rope_hadamard_cuda(x, rope=(cos, sin)), hadamard(embedded.float()).to(torch.bfloat16))
    # queries and keys of the same rows in one launch: each as its own launch gives it
    keys = torch.randn(rows, max(1, heads // 4), dim, generator=g).to(torch.bfloat16).cuda()
    for tables, rotate in (((cos, sin), True), (None, True), ((cos, sin), False)):
        q_out, k_out = rt.rope_hadamard_pair_cuda(x, keys, rope=tables, hadamard=rotate)
        assert torch.equal(q_out, rt.rope_hadamard_cuda(x, rope=tables, hadamard=rotate))
        assert torch.equal(k_out, rt.rope_hadamard_cuda(keys, rope=tables, hadamard=rotate))
    with pytest.raises(ValueError):
        rt.rope_hadamard_pair_cuda(x, keys[:5].contiguous(), rope=(cos, sin))
    with pytest.raises(ValueError):
        rt.rope_hadamard_cuda(x, rope=(cos[:5], sin[:5]))
    with pytest.raises(ValueError):
        rt.rope_hadamard_cuda(torch.zeros(2, 2, 32, dtype=torch.bfloat16, device="cuda"))


def _tiny_runners(tmp_path, seed, capacity, max_cache_len):
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm

    runners = []
    for fused in (True, False):
        torch.manual_seed(seed)
        config = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                             num_key_value_heads=2, head_dim=64, vocab_size=128, max_position_embeddings=512,
                             rope_theta=500000.0, tie_word_embeddings=True)
        model = LlamaForCausalLM(config).to(torch.bfloat16).cuda().eval()
        path = tmp_path / f"tiny{int(fused)}.nqmc"
        asm.write_w4_checkpoint(model, path)
        runners.append(asm.build_w4a4kv4_runner(model, path, capacity=capacity, max_cache_len=max_cache_len,
                                                fused_prefill=fused, fused_decode=fused))
    return runners


def test_fused_prefill_step_tracks_the_module_graph(tmp_path):
    """A ragged prompt batch, then a continuation chunk over the packed cache, then decode steps:
    the fused prefill step against the module graph of an identical model (tolerance: the
    row reductions of the norm run in a different order, so activations differ in the last place
    and a few codes with them)."""
    fused, modular = _tiny_runners(tmp_path, 5005, capacity=3, max_cache_len=160)
    assert fused.fused_prefill is not None and modular.fused_prefill is None
    g = torch.Generator().manual_seed(5006)
    ids = torch.randint(0, 128, (3, 70), generator=g).cuda()
    lengths = [70, 33, 1]
    more = torch.randint(0, 128, (3, 40), generator=g).cuda()
    more_lengths = [40, 17, 5]

    def run(runner):
        first = runner.prefill_slots(ids, slots=[0, 1, 2], lengths=lengths).float()
        second = runner.prefill_slots(more, slots=[0, 1, 2], lengths=more_lengths).float()     # continuation
        token = torch.stack([second[i, n - 1].argmax() for i, n in enumerate(more_lengths)]).reshape(3, 1)
        position = torch.tensor([[a + b] for a, b in zip(lengths, more_lengths)], device="cuda")
        step = runner.decode_eager(token * 0 + 7, slots=[0, 1, 2], positions=position).float()
        return first, second, step
    a, b = run(fused), run(modular)
    for i, (n, m) in enumerate(zip(lengths, more_lengths)):
        for got, want, count in ((a[0][i], b[0][i], n), (a[1][i], b[1][i], m)):
            got, want = got[:count], want[:count]
            assert torch.isfinite(got).all()
            cosine = torch.nn.functional.cosine_similarity(got, want, dim=-1)
            assert float(cosine.min()) > 0.99, (i, float(cosine.min()))
            assert relative_error(bits(got), bits(want)) < 0.08
    cosine = torch.nn.functional.cosine_similarity(a[2].flatten(1), b[2].flatten(1), dim=1)
    assert float(cosine.min()) > 0.99
    lengths_a = fused.cache.manager.metadata.sequence_lengths[:3].tolist()
    assert lengths_a == modular.cache.manager.metadata.sequence_lengths[:3].tolist() == [111, 51, 7]


def test_fused_decode_step_tracks_the_module_graph(tmp_path):
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm
    from nestquant_aiinfra_amd.runtime.nqkv_hf_backend import BatchedNQKVLlamaRunner

    torch.manual_seed(5001)
    config = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                         num_key_value_heads=2, head_dim=64, vocab_size=128, max_position_embeddings=512,
                         rope_theta=500000.0, tie_word_embeddings=True)
    model = LlamaForCausalLM(config).to(torch.bfloat16).cuda().eval()
    path = tmp_path / "tiny.nqmc"
    asm.write_w4_checkpoint(model, path)
    runner = asm.build_w4a4kv4_runner(model, path, capacity=2, max_cache_len=96)
    assert runner.fused_step is not None
    modular = BatchedNQKVLlamaRunner(model, runner.cache, fused_decode=False)
    assert modular.fused_step is None

    g = torch.Generator().manual_seed(5002)
    ids = torch.randint(0, 128, (2, 20), generator=g).cuda()
    logits = runner.prefill_slots(ids, slots=[0, 1], lengths=[20, 9])
    cache = runner.cache
    meta = cache.manager.metadata
    tensors = [meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths]
    for layer in cache.manager.layers:
        pool = layer.pool
        tensors += [layer.hot_keys, layer.hot_values, pool.key_codes, pool.key_betas, pool.key_norms,
                    pool.value_codes, pool.value_betas, pool.value_norms]
    saved, host = [t.clone() for t in tensors], list(cache._host_lengths)

    token = torch.stack([logits[0, 19].argmax(), logits[1, 8].argmax()]).reshape(2, 1)
    position = torch.tensor([[20], [9]], device="cuda")
    def run(which, steps=12):
        outs, tok, pos = [], token, position
        for _ in range(steps):
            out = which.decode_eager(tok, slots=[0, 1], positions=pos).float().clone()
            outs.append(out)
            tok = token                                   # same inputs for both paths at every step
            pos = pos + 1
        return torch.stack(outs)
    fused = run(runner)
    for tensor, value in zip(tensors, saved):
        tensor.copy_(value)
    cache._host_lengths[:] = host
    reference = run(modular)
    assert torch.isfinite(fused).all()
    cosine = torch.nn.functional.cosine_similarity(fused.flatten(1), reference.flatten(1), dim=1)
    assert float(cosine.min()) > 0.995
    assert relative_error(bits(fused), bits(reference)) < 0.08
    # the first step starts from identical state: only reduction order separates the two
    assert relative_error(bits(fused[0]), bits(reference[0])) < 0.03


def test_fused_decode_step_with_more_than_eight_rows(tmp_path):
    """Above eight rows the step's linears run on the MFMA kernel instead of the grouped GEMV."""
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm
    from nestquant_aiinfra_amd.runtime.nqkv_hf_backend import BatchedNQKVLlamaRunner

    torch.manual_seed(5003)
    config = LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                         num_key_value_heads=2, head_dim=64, vocab_size=128, max_position_embeddings=512,
                         rope_theta=500000.0, tie_word_embeddings=True)
    model = LlamaForCausalLM(config).to(torch.bfloat16).cuda().eval()
    path = tmp_path / "tiny.nqmc"
    asm.write_w4_checkpoint(model, path)
    rows = 12
    runner = asm.build_w4a4kv4_runner(model, path, capacity=rows, max_cache_len=64)
    modular = BatchedNQKVLlamaRunner(model, runner.cache, fused_decode=False)
    g = torch.Generator().manual_seed(5004)
    ids = torch.randint(0, 128, (rows, 18), generator=g).cuda()
    lengths = [18 - (i % 5) for i in range(rows)]
    logits = runner.prefill_slots(ids, slots=list(range(rows)), lengths=lengths)
    token = torch.stack([logits[i, n - 1].argmax() for i, n in enumerate(lengths)]).reshape(rows, 1)
    position = torch.tensor(lengths, device="cuda").reshape(rows, 1)
    cache = runner.cache
    meta = cache.manager.metadata
    tensors = [meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths]
    for layer in cache.manager.layers:
        tensors += [layer.hot_keys, layer.hot_values]
    saved, host = [t.clone() for t in tensors], list(cache._host_lengths)
    fused = runner.decode_eager(token, slots=list(range(rows)), positions=position).float().clone()
    for tensor, value in zip(tensors, saved):
        tensor.copy_(value)
    cache._host_lengths[:] = host
    reference = modular.decode_eager(token, slots=list(range(rows)), positions=position).float()
    assert torch.isfinite(fused).all() and tuple(fused.shape) == (rows, 1, 128)
    assert relative_error(bits(fused), bits(reference)) < 0.03
    # and through the captured graph of that width
    for tensor, value in zip(tensors, saved):
        tensor.copy_(value)
    cache._host_lengths[:] = host
    runner.capture(widths=[rows])
    replayed = runner.decode(token, slots=list(range(rows)), positions=position).float()
    assert torch.equal(replayed, fused)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_greedy_sampler_is_the_first_argmax(dtype):
    """The device sampler against torch.argmax: ties (BF16 logits repeat values) go to the lowest
    index, NaN counts as the largest value, rows may be strided slices, a vocabulary that is not a
    whole number of 16-byte vectors takes the element loop; inactive rows keep token and position."""
    from nestquant_aiinfra_amd.runtime.nqkv_hf_backend import greedy_sample_
    g = torch.Generator().manual_seed(77)
    for rows, vocab, stride in ((8, 128256, 128256), (3, 1000, 1024), (5, 777, 777), (1, 5, 8), (2, 70001, 70001)):
        storage = torch.randn((rows, stride), generator=g).to(dtype).cuda()
        storage[0, :vocab] = storage[0, :vocab].round()                    # many equal maxima
        if rows > 1:
            storage[1, vocab // 2] = float("nan")
            storage[1, vocab - 1] = float("nan")
        if stride > vocab:
            storage[:, vocab:] = 1e4                                      # beyond the vocabulary: never chosen
        logits = storage[:, :vocab]
        want = logits.float().argmax(-1)
        if rows > 1:
            want[1] = vocab // 2                                          # the first NaN
        tokens = torch.full((rows, 1), -1, dtype=torch.long, device="cuda")
        positions = torch.arange(rows, dtype=torch.long, device="cuda").reshape(rows, 1) * 10
        active = torch.ones(rows, dtype=torch.bool, device="cuda")
        if rows > 2:
            active[2] = False
        history = torch.full((4, rows), -1, dtype=torch.long, device="cuda")
        cursors = torch.zeros(rows, dtype=torch.int32, device="cuda")
        for step in range(6):                                             # the history is a ring of four steps
            greedy_sample_(logits, tokens, positions=positions, active_mask=active, history=history, cursors=cursors)
        live = active.cpu()
        assert torch.equal(tokens.view(-1).cpu()[live], want.cpu()[live]), (rows, vocab)
        assert (tokens.view(-1).cpu()[~live] == -1).all()
        assert torch.equal(positions.view(-1).cpu(), torch.arange(rows) * 10 + 6 * live.long())
        assert torch.equal(cursors.cpu(), 6 * live.int())
        assert (history.cpu()[:, live] == want.cpu()[live]).all() and (history.cpu()[:, ~live] == -1).all()
        plain = torch.zeros(rows, dtype=torch.long, device="cuda")
        assert torch.equal(greedy_sample_(logits, plain), want)


@pytest.mark.parametrize("fused", [True, False])
def test_many_greedy_steps_without_a_host_read(tmp_path, fused):
    """decode_greedy replays the captured step with the sampler's token fed back on the device:
    the same tokens as decode + argmax on the host, step by step, and the same cache state."""
    runner = _tiny_runners(tmp_path, 5010, capacity=4, max_cache_len=200)[0 if fused else 1]
    g = torch.Generator().manual_seed(5011)
    ids = torch.randint(0, 128, (3, 40), generator=g).cuda()
    lengths, slots, steps = [40, 21, 5], [2, 0, 3], 37

    def start():
        logits = runner.prefill_slots(ids, slots=slots, lengths=lengths)
        token = torch.stack([logits[i, n - 1].argmax() for i, n in enumerate(lengths)]).reshape(3, 1)
        return token, torch.tensor(lengths, device="cuda").reshape(3, 1)

    token, position = start()
    runner.capture()
    by_host = []
    for _ in range(steps):
        token = runner.decode(token, slots=slots, positions=position)[:, 0].argmax(-1).reshape(3, 1)
        by_host.append(token.view(-1).clone())
        position = position + 1
    lengths_by_host = runner.cache.manager.metadata.sequence_lengths.clone()
    runner.release_slots(slots)

    token, position = start()
    on_device = runner.decode_greedy(token, slots=slots, positions=position, steps=steps)
    assert torch.equal(on_device, torch.stack(by_host))
    assert torch.equal(runner.cache.manager.metadata.sequence_lengths, lengths_by_host)
    assert [runner.cache._host_lengths[s] for s in slots] == [n + steps for n in lengths]
    # a second run continues from the device's own tokens
    more = runner.decode_greedy(on_device[-1].reshape(3, 1), slots=slots, positions=position + steps, steps=5)
    assert more.shape == (5, 3)
    with pytest.raises(ValueError):
        runner.decode_greedy(token, slots=slots, positions=position, steps=500)


def test_decode_refuses_to_run_past_the_cache_length(tmp_path):
    """The host mirror of the lengths stops a step that would not fit (the device tables clamp at
    capacity, they never write out of bounds): decode, decode_eager, decode_greedy and prefill."""
    runner = _tiny_runners(tmp_path, 5020, capacity=2, max_cache_len=48)[0]
    ids = torch.randint(0, 128, (1, 40), generator=torch.Generator().manual_seed(1)).cuda()
    logits = runner.prefill_slots(ids, slots=[1], lengths=[40])
    token = logits[:, -1].argmax(-1).reshape(1, 1)
    position = torch.tensor([[40]], device="cuda")
    runner.capture()
    with pytest.raises(RuntimeError, match="max_cache_len"):
        runner.decode_greedy(token, slots=[1], positions=position, steps=9)
    tokens = runner.decode_greedy(token, slots=[1], positions=position, steps=8)          # fills the cache exactly
    assert runner.cache.manager.total_tokens(1) == 48
    for step in (runner.decode, runner.decode_eager):
        with pytest.raises(RuntimeError, match="max_cache_len"):
            step(tokens[-1].reshape(1, 1), slots=[1], positions=position + 8)
    with pytest.raises(RuntimeError, match="max_cache_len"):
        runner.prefill_slots(ids[:, :1], slots=[1], lengths=[1])
    assert runner.cache.manager.total_tokens(1) == 48


def test_bf16_rows_linear_against_float64():
    """The LM-head stream kernel: small-integer operands make every sum exact, so the result must
    equal the float64 product bit for bit whatever the order of accumulation (a wrong row, token
    or k pairing cannot pass); Gaussian operands must agree with the float64 product to one BF16
    rounding (2**-8 relative) plus the FP32 accumulation error.  Ragged N, every row count class,
    both K."""
    from nestquant_aiinfra_amd.runtime.w4a4_linear import bf16_rows_linear, can_use_bf16_rows_linear
    g = torch.Generator().manual_seed(4242)
    for rows, n, k in ((1, 128256, 2048), (8, 4099, 2048), (16, 1000, 4096), (5, 77, 2048), (13, 16, 4096), (3, 1, 2048),
                       (8, 2048, 8192), (16, 77, 8192), (5, 1000, 4096), (1, 4099, 8192)):
        act = torch.randint(-3, 4, (rows, k), generator=g).to(torch.bfloat16).cuda()
        weight = torch.randint(-3, 4, (n, k), generator=g).to(torch.bfloat16).cuda()
        assert can_use_bf16_rows_linear(act, weight)
        want = (act.double() @ weight.double().T).to(torch.bfloat16)
        assert torch.equal(bf16_rows_linear(act, weight), want), (rows, n, k)
        act = torch.randn((rows, k), generator=g).to(torch.bfloat16).cuda()
        weight = (0.05 * torch.randn((n, k), generator=g)).to(torch.bfloat16).cuda()
        exact = act.double() @ weight.double().T
        got = bf16_rows_linear(act, weight).double()
        bound = exact.abs() * 2.0 ** -8 + (act.double().abs() @ weight.double().abs().T) * k * 2.0 ** -24
        assert bool(((got - exact).abs() <= bound).all()), (rows, n, k, float(((got - exact).abs() / bound).max()))
    # one weight, three outputs: the rows of q, k and v one after the other, ragged on purpose
    from nestquant_aiinfra_amd.runtime.w4a4_linear import bf16_rows_linear_grouped
    for rows, k, sizes in ((8, 2048, [2048, 512, 512]), (3, 8192, [40, 9]), (16, 4096, [5, 1, 30])):
        act = torch.randn((rows, k), generator=g).to(torch.bfloat16).cuda()
        weight = (0.05 * torch.randn((sum(sizes), k), generator=g)).to(torch.bfloat16).cuda()
        outs = bf16_rows_linear_grouped(act, weight, sizes)
        whole = bf16_rows_linear(act, weight)
        assert [tuple(out.shape) for out in outs] == [(rows, size) for size in sizes]
        assert torch.equal(torch.cat(outs, 1), whole)
    with pytest.raises(ValueError, match="add up"):
        bf16_rows_linear_grouped(act, weight, [5, 1])
    for bad_rows, bad_weight in ((torch.zeros((17, 2048)), torch.zeros((32, 2048))), (torch.zeros((4, 1024)), torch.zeros((32, 1024)))):
        assert not can_use_bf16_rows_linear(bad_rows.to(torch.bfloat16).cuda(), bad_weight.to(torch.bfloat16).cuda())
        with pytest.raises(ValueError):
            bf16_rows_linear(bad_rows.to(torch.bfloat16).cuda(), bad_weight.to(torch.bfloat16).cuda())


def test_last_token_logits_and_the_lm_head_stream(tmp_path, monkeypatch):
    """A model as wide as the stream kernel's K (2048): `last_token_logits` returns the logits of
    every row's last prompt token (against the full prefill of the same prompt: the same hidden
    state, the head through the library there and through the stream kernel here, so equal to a
    BF16 rounding), and a decode step's logits are the same through either head."""
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm
    from nestquant_aiinfra_amd.runtime import llama_decode_step

    torch.manual_seed(6001)
    config = LlamaConfig(hidden_size=2048, intermediate_size=1024, num_hidden_layers=1, num_attention_heads=32,
                         num_key_value_heads=8, head_dim=64, vocab_size=1000, max_position_embeddings=256,
                         rope_theta=500000.0, tie_word_embeddings=True)
    model = LlamaForCausalLM(config).to(torch.bfloat16).cuda().eval()
    path = tmp_path / "wide.nqmc"
    asm.write_w4_checkpoint(model, path)
    runner = asm.build_w4a4kv4_runner(model, path, capacity=2, max_cache_len=96)
    assert runner.fused_step is not None and runner.fused_prefill is not None
    calls = []
    stream_kernel = llama_decode_step.bf16_rows_linear
    monkeypatch.setattr(llama_decode_step, "bf16_rows_linear", lambda *a: calls.append(1) or stream_kernel(*a))

    ids = torch.randint(0, 1000, (2, 20), generator=torch.Generator().manual_seed(6002)).cuda()
    lengths = [20, 9]
    full = runner.prefill_slots(ids, slots=[0, 1], lengths=lengths).float()
    assert not calls                                   # all positions: the library's GEMM
    runner.release_slots([0, 1])
    last = runner.prefill_slots(ids, slots=[0, 1], lengths=lengths, last_token_logits=True).float()
    assert len(calls) == 1 and last.shape == (2, 1, 1000)
    for row, length in enumerate(lengths):
        want = full[row, length - 1]
        assert float((last[row, 0] - want).abs().max()) <= 2.0 ** -7 * float(want.abs().max())
    with pytest.raises(ValueError, match="at least one token"):
        runner.prefill_slots(ids, slots=[0, 1], lengths=[0, 3], last_token_logits=True)

    # the same prompt in both slots: slot 0 decodes through the stream kernel, slot 1 through the library
    runner.release_slots([0, 1])
    same = ids[:1].repeat(2, 1)
    runner.prefill_slots(same, slots=[0, 1], lengths=[20, 20], last_token_logits=True)
    token, position = torch.tensor([[7]], device="cuda"), torch.tensor([[20]], device="cuda")
    calls.clear()
    streamed = runner.decode_eager(token, slots=[0], positions=position).float()
    assert len(calls) == 1
    monkeypatch.setattr(llama_decode_step, "can_use_bf16_rows_linear", lambda *a: False)
    library = runner.decode_eager(token, slots=[1], positions=position).float()
    assert len(calls) == 1
    assert float((streamed - library).abs().max()) <= 2.0 ** -7 * float(library.abs().max())
    assert int(streamed.argmax()) == int(library.argmax())


def test_expanded_weights_step_tracks_the_packed_step(tmp_path):
    """`expand_weights`: the decode step that streams BF16 copies of the weights (the values the
    packed kernels decode, multiplied in another order) against the packed step on the same
    prompt in another slot, eager and captured; K = 2048 and 4096 projections.  Every linear agrees
    with its packed form to a BF16 step of a few outputs (the kernel tests hold that); a step or
    two of difference moves some activation codes, which a random-init network amplifies from
    layer to layer, hence the loose bound on the logits."""
    from transformers import LlamaConfig, LlamaForCausalLM
    from nestquant_aiinfra_amd.models import llama_w4a4kv4 as asm
    from nestquant_aiinfra_amd.runtime.llama_decode_step import FusedLlamaDecodeStep

    torch.manual_seed(7001)
    config = LlamaConfig(hidden_size=2048, intermediate_size=4096, num_hidden_layers=2, num_attention_heads=32,
                         num_key_value_heads=8, head_dim=64, vocab_size=1000, max_position_embeddings=256,
                         rope_theta=500000.0, tie_word_embeddings=True)
    model = LlamaForCausalLM(config).to(torch.bfloat16).cuda().eval()
    path = tmp_path / "wide.nqmc"
    asm.write_w4_checkpoint(model, path)
    runner = asm.build_w4a4kv4_runner(model, path, capacity=2, max_cache_len=96, expand_weights=True)
    streamed_step = runner.fused_step
    assert streamed_step.expand_weights
    packed_step = FusedLlamaDecodeStep(model, runner.cache)
    ids = torch.randint(0, 1000, (1, 20), generator=torch.Generator().manual_seed(7002)).cuda().repeat(2, 1)
    runner.prefill_slots(ids, slots=[0, 1], lengths=[20, 20], last_token_logits=True)
    token, position = torch.tensor([[7]], device="cuda"), torch.tensor([[20]], device="cuda")
    streamed = runner.decode_eager(token, slots=[0], positions=position).float()
    assert streamed_step._expanded and all(entry is not None for entry in streamed_step._expanded.values())
    runner.fused_step = packed_step
    packed = runner.decode_eager(token, slots=[1], positions=position).float()
    runner.fused_step = streamed_step
    cosine = torch.nn.functional.cosine_similarity(streamed.flatten(), packed.flatten(), dim=0)
    assert float(cosine) > 0.95, float(cosine)
    runner.capture()
    chosen = runner.decode_greedy(token, slots=[0], positions=position + 1, steps=4)
    assert chosen.shape == (4, 1) and bool(((chosen >= 0) & (chosen < 1000)).all())
