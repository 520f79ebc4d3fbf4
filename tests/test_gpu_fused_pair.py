"""A decode step's input stage and the linear(s) behind it as one launch (nq_fused_stage_linear): the
same bits as the two launches it replaces (nq_fused_input_stage / nq_attention_output_stage, then
nq_w4a4_gemv_grouped), for every stage, row count and kernel form the 1B decode step meets; and the
failure path: consumers whose bounded wait runs out set the status word, store nothing and exit.
Reference of the arithmetic being fused: nestquant/models/fused_linear.py:287-306, 316-407."""

import pytest
import torch

from conftest import ACTIVATION_BETAS, Q, WEIGHT_BETAS

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    from nestquant_aiinfra_amd.runtime import w4a4_linear
    return w4a4_linear


_WEIGHTS = {}


def _weights(rt, k, sizes, seed):
    key = (k, tuple(sizes), seed)
    if key not in _WEIGHTS:
        g = torch.Generator().manual_seed(seed)
        made = []
        for index, n_out in enumerate(sizes):
            rotated = rt.hadamard_cuda((0.02 * torch.randn(n_out, k, generator=g)).cuda(), compute_dtype=torch.float32)
            record = rt.quantize_weight_nqrt4(rotated, q=Q, betas=WEIGHT_BETAS, dither_seed=20261401 + 7 * seed + index,
                                              tensor_name=f"w{seed}_{index}")
            made.append(rt.prepare_fused_linear(record, device="cuda"))
        _WEIGHTS[key] = made
    return _WEIGHTS[key]


def _table():
    return torch.tensor(ACTIVATION_BETAS, dtype=torch.float32, device="cuda")


def _same_activation(a, b):
    return (torch.equal(a.code_payload, b.code_payload) and torch.equal(a.beta_payload, b.beta_payload)
            and torch.equal(a.row_norms, b.row_norms) and torch.equal(a.decoded, b.decoded))


# (name, K, the channel counts of the weights that share the rows): the four pairs of a 1B decode step and two ragged ones
PAIRS = [("qkv", 2048, (2048, 512, 512)), ("o_proj", 2048, (2048,)), ("gate_up", 2048, (8192, 8192)),
         ("down_proj", 8192, (2048,)), ("ragged", 2048, (136, 2050)), ("ragged_long", 8192, (520,))]


@pytest.mark.parametrize("rows", [1, 2, 3, 4, 5, 8, 9, 13, 16])
@pytest.mark.parametrize("name,k,sizes", PAIRS)
def test_stage_and_linear_in_one_launch_equal_two_launches(rt, name, k, sizes, rows):
    weights = _weights(rt, k, sizes, seed=len(name))
    sync = rt.StageLinearSync(torch.device("cuda"))
    g = torch.Generator().manual_seed(100 * rows + k % 97)
    x = torch.randn(rows, k, generator=g).to(torch.bfloat16).cuda()
    other = torch.randn(rows, k, generator=g).to(torch.bfloat16).cuda()
    norm_weight = (1.0 + 0.1 * torch.randn(k, generator=g)).to(torch.bfloat16).cuda()
    for mode, kwargs in (("rmsnorm", dict(residual=other, norm_weight=norm_weight, eps=1e-5)), ("swiglu", dict(gate=other))):
        for dtype in (torch.bfloat16, torch.float32):
            for repeat in range(3):                      # successive launches walk the ring of flag words
                outs, activation, residual, staged = rt.fused_stage_linear(
                    x, weights, sync, mode=mode, beta_table=_table(), want_residual=True, want_staged=True,
                    output_dtype=dtype, **kwargs)
                expect_activation, expect_residual, expect_staged = rt.fused_input_stage(
                    x, mode=mode, beta_table=_table(), want_residual=True, want_staged=True, **kwargs)
                expect = rt.linear_packed_w4a4_gemv_grouped(expect_activation, weights, output_dtype=dtype)
                assert _same_activation(activation, expect_activation)
                assert torch.equal(staged, expect_staged)
                assert torch.equal(residual, expect_residual) if mode == "rmsnorm" else residual is None
                for out, want in zip(outs, expect):
                    assert out.shape == want.shape and torch.equal(out, want)
    assert not sync.timed_out


@pytest.mark.parametrize("rows", [1, 2, 5, 8, 16])
@pytest.mark.parametrize("name,k,sizes", PAIRS)
def test_encoder_and_linear_in_one_launch_equal_two_launches(rt, name, k, sizes, rows):
    """The rows themselves as the input stage (what a packed linear module does with its input: rotate,
    encode, multiply): modes "rows" and "rotated_rows" against `quantize_activation_cuda` with and without
    the rotation followed by the grouped linear, bit for bit."""
    if k == 8192 and rows == 5:
        rows = 11                                        # slices of 1024 values from nine rows on
    weights = _weights(rt, k, sizes, seed=len(name))
    sync = rt.StageLinearSync(torch.device("cuda"))
    g = torch.Generator().manual_seed(300 * rows + k % 89)
    x = (torch.randn(rows, k, generator=g) * (1.0 + 3.0 * (torch.rand(rows, 1, generator=g) > 0.5))).to(torch.bfloat16).cuda()
    for mode, rotate in (("rows", True), ("rotated_rows", False)):
        expect_activation = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS, beta_table=_table(), hadamard=rotate)
        for dtype in (torch.bfloat16, torch.float32):
            expect = rt.linear_packed_w4a4_gemv_grouped(expect_activation, weights, output_dtype=dtype)
            for repeat in range(2):
                outs, activation, residual, staged = rt.fused_stage_linear(x, weights, sync, mode=mode, beta_table=_table(),
                                                                            output_dtype=dtype)
                assert residual is None and staged is None
                assert _same_activation(activation, expect_activation), (mode, dtype)
                for out, want in zip(outs, expect):
                    assert out.shape == want.shape and torch.equal(out, want), (mode, dtype)
    assert not sync.timed_out
    with pytest.raises(ValueError, match="staged"):
        rt.fused_stage_linear(x, weights, sync, mode="rows", beta_table=_table(), want_staged=True)


@pytest.mark.parametrize("rows", [1, 4, 8])
def test_attention_merge_and_o_proj_in_one_launch(rt, rows):
    from nestquant_aiinfra_amd.runtime import nqkv
    from conftest import KEY_BETAS, VALUE_BETAS
    heads, kv_heads, dim = 32, 8, 64
    manager = nqkv.BatchedNQKVCacheManager(capacity=rows, num_layers=1, num_kv_heads=kv_heads, head_dim=dim, max_cache_len=160,
                                           page_size=16, q=Q, key_betas=KEY_BETAS, value_betas=VALUE_BETAS,
                                           dtype=torch.bfloat16, device="cuda")
    g = torch.Generator().manual_seed(900 + rows)
    lengths = [int(n) for n in torch.randint(20, 150, (rows,), generator=g)]
    for slot, length in enumerate(lengths):
        manager.register(slot, slot=slot)
    width = max(lengths)
    key = torch.randn(rows, width, kv_heads, dim, generator=g).to(torch.bfloat16).cuda()
    value = torch.randn(rows, width, kv_heads, dim, generator=g).to(torch.bfloat16).cuda()
    manager.step_slot_ids[:rows] = torch.arange(rows, dtype=torch.int32)
    manager.step_active[:rows] = True
    manager.step_counts[:rows] = torch.tensor(lengths, dtype=torch.int32)
    manager.begin_step(rows=rows, uniform_count=None)
    manager.write_layer(0, key, value)
    cache = manager.layers[0]
    workspace = nqkv.BatchedNQKVAttentionWorkspace.create(cache, batch_size=rows, query_heads=heads, output_dtype=torch.bfloat16)
    query = torch.randn(rows, heads, dim, generator=g).to(torch.bfloat16).cuda()
    nqkv.launch_nqkv_decode_attention(query, cache, slot_ids=manager.step_slot_ids[:rows], active_mask=manager.step_active[:rows],
                                      attention_scale=0.125, workspace=workspace, merge=False)
    weights = _weights(rt, heads * dim, (2048,), seed=5)
    sync = rt.StageLinearSync(torch.device("cuda"))
    expect_activation, expect_staged = nqkv.attention_output_stage(workspace, beta_table=_table(), want_staged=True)
    expect = rt.linear_packed_w4a4_gemv_grouped(expect_activation, weights, output_dtype=torch.bfloat16)
    for _ in range(2):
        outs, activation, _, staged = rt.fused_stage_linear(None, weights, sync, mode="attention", beta_table=_table(),
                                                            attention_workspace=workspace, want_staged=True)
        assert _same_activation(activation, expect_activation) and torch.equal(staged, expect_staged)
        assert torch.equal(outs[0], expect[0])
    assert not sync.timed_out


def test_a_wait_that_runs_out_sets_the_status_and_stores_nothing(rt):
    """The consumers' wait is bounded.  A limit of zero polls makes every consumer that looks before the
    encoder is done give up: the status word is set, those workgroups leave their outputs untouched, the
    launch ends, and after `reset` the same objects work again."""
    weights = _weights(rt, 8192, (2048,), seed=9)
    sync = rt.StageLinearSync(torch.device("cuda"), spin_limit=0)
    g = torch.Generator().manual_seed(77)
    x = torch.randn(1, 8192, generator=g).to(torch.bfloat16).cuda()
    gate = torch.randn(1, 8192, generator=g).to(torch.bfloat16).cuda()
    outs, activation, _, _ = rt.fused_stage_linear(x, weights, sync, mode="swiglu", beta_table=_table(), gate=gate)
    torch.cuda.synchronize()
    assert sync.timed_out                                     # the encoder of an 8192-value row takes about 10 us
    expect_activation, _, _ = rt.fused_input_stage(x, mode="swiglu", beta_table=_table(), gate=gate)
    assert _same_activation(activation, expect_activation)   # the producers are not affected
    sync.reset()
    sync.spin_limit = 400_000
    outs, activation, _, _ = rt.fused_stage_linear(x, weights, sync, mode="swiglu", beta_table=_table(), gate=gate)
    expect = rt.linear_packed_w4a4_gemv_grouped(expect_activation, weights, output_dtype=torch.bfloat16)
    assert torch.equal(outs[0], expect[0]) and not sync.timed_out


def test_fused_pair_argument_checks(rt):
    weights = _weights(rt, 2048, (136, 2050), seed=6)
    sync = rt.StageLinearSync(torch.device("cuda"))
    x = torch.zeros(2, 2048, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="mode"):
        rt.fused_stage_linear(x, weights, sync, mode="layernorm", beta_table=_table())
    with pytest.raises(ValueError, match="norm weight"):
        rt.fused_stage_linear(x, weights, sync, mode="rmsnorm", beta_table=_table())
    with pytest.raises(ValueError, match="gate"):
        rt.fused_stage_linear(x, weights, sync, mode="swiglu", beta_table=_table())
    with pytest.raises(ValueError, match="outside what the fused"):
        rt.fused_stage_linear(torch.zeros(2, 4096, dtype=torch.bfloat16, device="cuda"), weights, sync, mode="swiglu",
                              beta_table=_table(), gate=torch.zeros(2, 4096, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(TypeError):
        rt.fused_stage_linear(x.float(), weights, sync, mode="swiglu", beta_table=_table(), gate=x.float())
    assert rt.can_use_fused_stage_linear(9, 8192, _weights(rt, 8192, (520,), seed=11))
    assert not rt.can_use_fused_stage_linear(17, 8192, _weights(rt, 8192, (520,), seed=11))
    assert rt.can_use_fused_stage_linear(16, 2048, weights)
