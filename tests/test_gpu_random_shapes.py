"""Seeded sweeps over random shapes, dtypes and data kinds: the encoder bit for bit against the
oracle, the decode and prefill linears, the KV writer page by page, and both attention kernels.
The fixed cases of the other files pin the shapes the model uses; these pin what lies between them
(ragged row counts, short and long rows, every route's thresholds, slots in any order).

Bars: codes, beta ids, norms and the BF16 decode of the encoder bit-exact; linears <= 1e-2 against
the oracle's FP32 product and <= 2e-3 against its product of BF16-rounded operands (5e-3 for
K <= 256, where a single weight that rounds to the neighbouring BF16 value weighs that much);
decode and prefill attention <= 1e-2 (the prefill kernel's products run on the matrix cores with BF16
operands: its scores take each decoded key as two BF16 parts, without which a head whose value terms
cancel reached 1.3e-2)."""

import numpy as np
import pytest
import torch

from conftest import ACTIVATION_BETAS, KEY_BETAS, Q
from gpu_util import bits, oracle_weight, outlier_rows, relative_error, student_t_rows
import test_gpu_gemv as gemv_cases
import test_gpu_nqkv as nqkv_cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    from nestquant_aiinfra_amd.runtime import w4a4_linear
    return w4a4_linear


@pytest.fixture(scope="module")
def kv():
    from nestquant_aiinfra_amd.runtime import nqkv
    return nqkv


def _rows_of(kind: str, rows: int, n: int, seed: int) -> np.ndarray:
    r = np.random.default_rng(seed)
    if kind == "normal":
        return r.standard_normal((rows, n)).astype(np.float32)
    if kind == "t4":
        return student_t_rows(rows, n, seed).numpy()
    if kind == "outlier":
        return outlier_rows(rows, n, seed).numpy()
    if kind == "scaled":                                    # every row at a scale of its own, 1e-6 .. 1e6
        return (r.standard_normal((rows, n)) * 10.0 ** r.uniform(-6, 6, size=(rows, 1))).astype(np.float32)
    if kind == "sparse":                                    # nine zeros in ten, and one row of zeros
        x = r.standard_normal((rows, n)).astype(np.float32)
        x[r.random((rows, n)) < 0.9] = 0.0
        if rows > 1:
            x[r.integers(rows)] = 0.0
        return x
    return np.round(r.standard_normal((rows, n)) * 3).astype(np.float32) * 0.5        # half-integers: many exact ties


@pytest.mark.parametrize("sweep_seed", [7, 23])
def test_encoder_over_random_shapes_is_bit_exact(rt, oracle, sweep_seed):
    rng = np.random.default_rng(sweep_seed)
    for _ in range(400):
        rows = int(rng.choice([1, 2, 3, 5, 8, 13, 16, 17, 40, 100, 190, 200, 300, 513, 700]))
        n = int(rng.choice([32, 64, 96, 160, 256, 512, 1024, 1536, 2048, 3072, 4096, 8192]))
        rows = min(rows, max(1, 700 * 2048 // n))
        kind = str(rng.choice(["normal", "t4", "outlier", "scaled", "sparse", "ties"]))
        dtype = [torch.float32, torch.bfloat16, torch.float16][rng.integers(3)]
        rotate = bool(rng.integers(2)) and n & (n - 1) == 0
        betas = [ACTIVATION_BETAS, KEY_BETAS, ACTIVATION_BETAS[:3]][rng.integers(3)]
        seed = int(rng.integers(1 << 30))
        case = (rows, n, kind, dtype, rotate, len(betas), seed)
        x = torch.from_numpy(_rows_of(kind, rows, n, seed)).to(dtype)
        if dtype == torch.float16 and float(x.abs().max()) >= 100.0:        # keep the float16 butterflies finite
            x = x.clamp(-60000, 60000) * (100.0 / float(x.abs().max()))
        x_dev = x.cuda()
        table = torch.tensor(betas, dtype=torch.float32, device="cuda")
        decoded = torch.empty((rows, n), dtype=torch.bfloat16, device="cuda") if len(betas) == 4 else None
        codes, ids, norms = rt.quantize_rows_packed(x_dev, q=Q, beta_table=table, hadamard=rotate, decoded=decoded)
        # the rotation itself is pinned elsewhere; here the stand-alone kernel gives the rows the encoder saw
        seen = rt.hadamard_cuda(x_dev, compute_dtype=dtype, output_dtype=torch.float32).cpu().numpy() if rotate \
            else x.float().numpy()
        want_codes, want_ids, want_norms = oracle.quantize_rows(seen, Q, betas)
        assert np.array_equal(bits(norms), want_norms), case
        assert np.array_equal(bits(codes), oracle.pack_unsigned(want_codes, 4)), case
        assert np.array_equal(bits(ids), oracle.pack_unsigned(want_ids, 2)), case
        if decoded is not None:
            want = oracle.bf16_round(oracle.dequantize_rows(want_codes, want_ids, want_norms, betas, Q))
            assert np.array_equal(decoded.float().cpu().numpy(), want), case


@pytest.mark.parametrize("sweep_seed", [11, 31])
def test_linears_over_random_shapes_match_oracle(rt, oracle, sweep_seed):
    rng = np.random.default_rng(sweep_seed)
    for _ in range(300):
        k = int(rng.choice([128, 256, 512, 1024, 2048, 4096, 8192]))
        n_out = int(rng.choice([16, 23, 32, 40, 64, 96, 136, 256, 512, 1000]))
        n_out = min(n_out, max(16, 2048 * 512 // k // 8 * 8))
        if rng.integers(2):
            m = int(rng.integers(1, 17))                     # the decode kernels
        else:                                                # both prefill routes and their thresholds
            m = int(rng.choice([17, 31, 32, 33, 64, 100, 128, 200, 256, 257, 300, 513, 600]))
        seed = int(rng.integers(1 << 31))
        case = (m, k, n_out, seed)
        _, wc, wb, wn = oracle_weight(oracle, n_out, k, seed=seed % 100000, dither_seed=seed)
        weight = rt.prepare_fused_linear(gemv_cases._record(rt, wc, wb, wn, k, seed), device="cuda")
        x = student_t_rows(m, k, seed=seed % 9973).to(torch.bfloat16).cuda()
        activation = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS, hadamard=True)
        ref32, ref16 = gemv_cases._references(oracle, activation, rt, wc, wb, wn, seed)
        tight = 2e-3 if k > 256 else 5e-3
        if m <= 8 or (m <= 16 and k % 128 == 0):
            y = rt._gemv(activation, weight, split_k=0, output_dtype=torch.float32)
            assert relative_error(bits(y), ref16) <= tight, ("gemv", case)
        y = rt._gemm(activation, weight, output_dtype=torch.bfloat16)
        assert relative_error(bits(y.float()), ref32) <= 1e-2, ("gemm, BF16 out", case)
        y = rt._gemm(activation, weight, output_dtype=torch.float32)
        assert relative_error(bits(y), ref16) <= tight, ("gemm, FP32 out", case)


@pytest.mark.parametrize("sweep_seed", [5, 77])
def test_kv_writer_and_attention_over_random_batches(kv, oracle, sweep_seed):
    heads, dim = nqkv_cases.HEADS, nqkv_cases.DIM
    _bf16, _f32 = nqkv_cases._bf16, nqkv_cases._f32
    rng = np.random.default_rng(sweep_seed)
    for _ in range(150):
        capacity = int(rng.choice([1, 2, 3, 4, 8]))
        max_len = int(rng.choice([64, 256, 512, 1024]))
        q_heads = int(rng.choice([8, 16, 32, 64]))
        batch = int(rng.integers(1, capacity + 1))
        slots = [int(s) for s in rng.permutation(capacity)[:batch]]
        rounds = int(rng.integers(1, 4))
        seed = int(rng.integers(1 << 30))
        case = (capacity, max_len, q_heads, slots, rounds, seed)
        r = np.random.default_rng(seed)
        manager = nqkv_cases._manager(kv, capacity=capacity, max_len=max_len)
        for s in slots:
            manager.register(f"s{s}", slot=s)
        history = {s: (torch.zeros((0, heads, dim), dtype=torch.bfloat16),) * 2 for s in slots}
        for _ in range(rounds):                              # ragged appends, some rows sitting a round out
            counts = []
            for s in slots:
                room = max_len - 2 - history[s][0].shape[0]
                top = max(1, min(room, int(r.choice([1, 3, 16, 40, 200, 600]))))
                counts.append(int(r.integers(1, top + 1)) if room > 0 else 0)
            live = [(s, c) for s, c in zip(slots, counts) if c > 0]
            if not live:
                break
            keys = [_bf16(oracle.hadamard(r.standard_normal((c, heads, dim)).astype(np.float32))) for _, c in live]
            values = [_bf16(r.standard_normal((c, heads, dim)).astype(np.float32) * float(r.choice([0.1, 1.0, 8.0])))
                      for _, c in live]
            nqkv_cases._append(manager, [s for s, _ in live], keys, values)
            for (s, _), k, v in zip(live, keys, values):
                history[s] = (torch.cat([history[s][0], k]), torch.cat([history[s][1], v]))
        torch.cuda.synchronize()
        for s in slots:
            nqkv_cases._check_cache(kv, oracle, manager, s, history[s][0], history[s][1])
        views = {s: nqkv_cases._cache_view(oracle, history[s][0], history[s][1]) for s in slots}
        slot_ids = torch.tensor(slots, dtype=torch.int32, device="cuda")
        active = torch.ones(batch, dtype=torch.bool, device="cuda")
        query = _bf16(oracle.hadamard(r.standard_normal((batch, q_heads, dim)).astype(np.float32))).cuda()
        out = kv.nqkv_decode_attention_batched_k1(query, manager.layers[0], slot_ids=slot_ids, active_mask=active)
        for row, s in enumerate(slots):
            ref = oracle.attention_dense(_f32(query[row].cpu()), *views[s])
            assert relative_error(_f32(out[row]), ref) <= 1e-2, ("decode attention", row, case)
        # the last `tokens` tokens of every row taken as a prefill chunk: token t sees the tokens up to its own
        tokens = int(r.choice([1, 5, 16, 33]))
        lengths = [history[s][0].shape[0] for s in slots]
        if min(lengths) < tokens:
            continue
        queries = _bf16(oracle.hadamard(r.standard_normal((batch, tokens, q_heads, dim)).astype(np.float32))).cuda()
        counts = torch.full((batch,), tokens, dtype=torch.int32, device="cuda")
        for split in (False, True):
            got = kv.nqkv_prefill_attention(queries, manager.layers[0], slot_ids=slot_ids, active_mask=active,
                                            counts=counts, split_context=split)
            for row, s in enumerate(slots):
                for t in (0, tokens - 1):
                    visible = lengths[row] - tokens + t + 1
                    ref = oracle.attention_dense(_f32(queries[row, t].cpu()), views[s][0][:visible], views[s][1][:visible])
                    assert relative_error(_f32(got[row, t]), ref) <= 1e-2, ("prefill attention", split, row, t, case)


@pytest.mark.parametrize("sweep_seed", [3, 41])
def test_appending_attention_over_random_steps(kv, oracle, sweep_seed):
    """The decode step's one-launch form (`append_and_attend`) against writer + attention on a second
    cache fed the same tokens, as in test_gpu_nqkv.py, but with the rows in a step, the slots whose
    cache is switched off, the slot order, the starting lengths and the head counts drawn at random."""
    heads, dim, page = nqkv_cases.HEADS, nqkv_cases.DIM, nqkv_cases.PAGE
    _bf16, _f32 = nqkv_cases._bf16, nqkv_cases._f32
    rng = np.random.default_rng(sweep_seed)
    for _ in range(30):
        capacity = int(rng.choice([1, 2, 4, 8]))
        max_len = int(rng.choice([64, 256, 1024, 2048]))
        q_heads = int(rng.choice([8, 16, 32, 64]))
        rows = int(rng.integers(1, capacity + 1))
        slots = [int(s) for s in rng.permutation(capacity)[:rows]]
        lengths = [int(rng.integers(1, max_len - 8)) if rng.integers(3) else int(rng.choice([1, 15, 16, 17, max_len - 20]))
                   for _ in slots]
        steps = int(rng.integers(18, 36))
        case = (capacity, max_len, q_heads, slots, lengths, steps)
        managers = [nqkv_cases._manager(kv, capacity=capacity, max_len=max_len) for _ in range(2)]
        keys = [_bf16(oracle.hadamard(rng.standard_normal((n, heads, dim)).astype(np.float32))) for n in lengths]
        values = [_bf16(rng.standard_normal((n, heads, dim)).astype(np.float32)) for n in lengths]
        for manager in managers:
            for s in slots:
                manager.register(f"seq{s}", slot=s)
            nqkv_cases._append(manager, slots, keys, values)
        workspaces = [kv.BatchedNQKVAttentionWorkspace.create(m.layers[0], batch_size=rows, query_heads=q_heads,
                                                              output_dtype=torch.bfloat16) for m in managers]
        totals = list(lengths)
        for step in range(steps):
            in_step = [bool(rng.random() < 0.85) for _ in slots]
            cache_on = [bool(rng.random() < 0.9) for _ in range(capacity)]
            key = _bf16(rng.standard_normal((rows, heads, dim)).astype(np.float32)).cuda()
            value = _bf16(rng.standard_normal((rows, heads, dim)).astype(np.float32)).cuda()
            query = _bf16(rng.standard_normal((rows, q_heads, dim)).astype(np.float32)).cuda()
            angles = np.asarray(totals, dtype=np.float64)[:, None] * (500000.0 ** (-np.arange(0, dim, 2) / dim))[None, :]
            cos = _bf16(np.concatenate([np.cos(angles)] * 2, axis=1).astype(np.float32)).cuda()
            sin = _bf16(np.concatenate([np.sin(angles)] * 2, axis=1).astype(np.float32)).cuda()
            packs = []
            for i in range(rows):
                grows = in_step[i] and totals[i] < managers[0].max_tokens
                totals[i] += 1 if grows else 0
                packs.append(in_step[i] and totals[i] % page == 0)
            outputs = []
            for which, (manager, workspace) in enumerate(zip(managers, workspaces)):
                manager.step_slot_ids[:rows] = torch.tensor(slots, dtype=torch.int32)
                manager.step_active[:rows] = torch.tensor(in_step)
                manager.metadata.active_mask[:capacity] = torch.tensor(cache_on)
                manager.begin_step(rows=rows, uniform_count=1)
                if which == 0:
                    manager.write_layer(0, key.view(rows, 1, heads, dim), value.view(rows, 1, heads, dim), rotate_keys=True,
                                        rope=(cos.view(rows, 1, dim), sin.view(rows, 1, dim)))
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
                    assert relative_error(_f32(one[i]), _f32(two[i])) <= 2.0 ** -7, (step, i, case)
                else:
                    assert torch.equal(one[i], two[i]), (step, i, case)
                if not cache_on[slots[i]] or not in_step[i]:
                    assert not one[i].any(), (step, i, case)
            a, b = managers
            for name in ("sequence_lengths", "page_counts", "last_page_lens", "hot_lengths"):
                assert torch.equal(getattr(a.metadata, name), getattr(b.metadata, name)), (step, name, case)
            assert [a.total_tokens(s) for s in slots] == totals, (step, case)
            for name in ("key_codes", "key_betas", "key_norms", "value_codes", "value_betas", "value_norms"):
                assert torch.equal(getattr(a.layers[0].pool, name), getattr(b.layers[0].pool, name)), (step, name, case)
            assert torch.equal(a.layers[0].hot_keys, b.layers[0].hot_keys), (step, case)
            assert torch.equal(a.layers[0].hot_values, b.layers[0].hot_values), (step, case)


from test_gpu_model import tiny  # noqa: E402,F401  (the two-layer model and its runner, one instance for this file)


@pytest.mark.parametrize("sweep_seed", [9, 58])
def test_runner_graph_equals_eager_under_slot_churn(tiny, sweep_seed):
    """A scripted engine on the tiny model: prompts of random lengths enter free slots, live slots take
    further prompt chunks, random subsets of the live slots decode in random row order, slots are
    released and reused.  Every decode step runs twice from the same cache state, through the
    captured graph and un-captured, and must give the same logits, tables, hot tails and pages bit
    for bit; bursts on the device sampler must choose the tokens that step-by-step argmax chooses."""
    _, runner, *_ = tiny
    cache, meta = runner.cache, runner.cache.manager.metadata
    runner.release_slots([s for s in range(runner.batch_size) if cache.manager.sequence_id(s) is not None])
    if not runner.graph_captured:
        runner.capture()
    rng = np.random.default_rng(sweep_seed)
    generator = torch.Generator().manual_seed(sweep_seed)
    tensors = [meta.sequence_lengths, meta.page_counts, meta.last_page_lens, meta.hot_lengths]
    for layer in cache.manager.layers:
        pool = layer.pool
        tensors += [layer.hot_keys, layer.hot_values, pool.key_codes, pool.key_betas, pool.key_norms,
                    pool.value_codes, pool.value_betas, pool.value_norms]

    def snapshot():
        return [t.clone() for t in tensors], list(cache._host_lengths)

    def restore(saved):
        for tensor, value in zip(tensors, saved[0]):
            tensor.copy_(value)
        cache._host_lengths[:] = saved[1]

    live: dict[int, list[int]] = {}                          # slot -> [tokens held, next token]
    limit = runner.max_cache_len
    decoded = 0
    for event in range(50):
        free = [s for s in range(runner.batch_size) if s not in live]
        choice = rng.random()
        if free and (not live or choice < 0.25):             # new prompts into free slots
            slots = [int(s) for s in rng.permutation(free)[: int(rng.integers(1, len(free) + 1))]]
            lengths = [int(rng.integers(1, 41)) for _ in slots]
            ids = torch.randint(0, 128, (len(slots), max(lengths)), generator=generator).cuda()
            logits = runner.prefill_slots(ids, slots=slots, lengths=lengths, last_token_logits=True)
            for row, (slot, length) in enumerate(zip(slots, lengths)):
                live[slot] = [length, int(logits[row, 0].argmax())]
        elif live and choice < 0.35:                         # a further chunk of a live slot's prompt
            slot = int(rng.choice(sorted(live)))
            length = int(rng.integers(1, 21))
            if live[slot][0] + length < limit - 8:
                ids = torch.randint(0, 128, (1, length), generator=generator).cuda()
                logits = runner.prefill_slots(ids, slots=[slot], lengths=[length], last_token_logits=True)
                live[slot] = [live[slot][0] + length, int(logits[0, 0].argmax())]
        elif live and choice < 0.45:                         # a sequence ends
            slot = int(rng.choice(sorted(live)))
            runner.release_slots([slot])
            del live[slot]
            assert cache.manager.total_tokens(slot) == 0
        elif live:                                           # decode steps of a subset, in any row order
            slots = [int(s) for s in rng.permutation(sorted(live))[: int(rng.integers(1, len(live) + 1))]]
            steps = int(rng.integers(1, 7))
            if any(live[s][0] + steps >= limit - 1 for s in slots):
                for s in slots:
                    runner.release_slots([s])
                    del live[s]
                continue
            tokens = torch.tensor([[live[s][1]] for s in slots], device="cuda")
            positions = torch.tensor([[live[s][0]] for s in slots], device="cuda")
            case = (event, slots, steps, {s: tuple(v) for s, v in live.items()})
            if rng.random() < 0.3:                           # a burst on the device sampler against single steps
                saved = snapshot()
                chosen = runner.decode_greedy(tokens, slots=slots, positions=positions, steps=steps)
                burst_state = [t.clone() for t in tensors]
                restore(saved)
                runner._decode_state = None
            else:
                chosen = None
            for step in range(steps):
                saved = snapshot()
                by_graph = runner.decode(tokens, slots=slots, positions=positions).clone()
                graph_state = [t.clone() for t in tensors]
                restore(saved)
                runner._decode_state = None
                eager = runner.decode_eager(tokens, slots=slots, positions=positions)
                assert torch.equal(by_graph, eager), ("logits", step, case)
                for a, b in zip(graph_state, tensors):
                    assert torch.equal(a, b), ("cache state", step, case)
                tokens = eager[:, 0].argmax(-1).reshape(-1, 1)
                positions = positions + 1
                if chosen is not None:
                    assert torch.equal(chosen[step], tokens[:, 0]), ("device sampler", step, case)
                decoded += 1
            if chosen is not None:
                for a, b in zip(burst_state, tensors):
                    assert torch.equal(a, b), ("cache state after the burst", case)
            for row, s in enumerate(slots):
                live[s] = [live[s][0] + steps, int(tokens[row, 0])]
                assert cache.manager.total_tokens(s) == live[s][0], case
    assert decoded >= 20
    runner.release_slots(sorted(live))


@pytest.mark.parametrize("sweep_seed", [13, 87])
def test_fused_input_stages_over_random_shapes(rt, sweep_seed):
    """Residual + RMSNorm and SwiGLU in front of the encoder, over every kernel form's row counts: the
    residual stream exact, the staged rows within one BF16 step of the tensor operations (two where a
    norm weight above one stretches the step), and the codes those of the plain encoder on the staged rows."""
    import test_gpu_fused_step as stage_cases
    rng = np.random.default_rng(sweep_seed)
    table = torch.tensor(ACTIVATION_BETAS, dtype=torch.float32, device="cuda")
    for _ in range(120):
        rows = int(rng.choice([1, 2, 5, 8, 16, 17, 40, 100, 192, 193, 300, 512, 513, 700, 1100]))
        n = int(rng.choice([256, 512, 1024, 2048, 4096, 8192]))
        rows = min(rows, max(1, (1 << 22) // n))
        mode = str(rng.choice(["rmsnorm", "rmsnorm+residual", "swiglu"]))
        scale = float(rng.choice([0.05, 1.0, 30.0]))
        case = (rows, n, mode, scale)
        g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
        x = (scale * torch.randn(rows, n, generator=g)).to(torch.bfloat16).cuda()
        if mode == "swiglu":
            gate = (2 * torch.randn(rows, n, generator=g)).to(torch.bfloat16).cuda()
            activation, _, staged = rt.fused_input_stage(x, mode="swiglu", gate=gate, beta_table=table, want_staged=True)
            expect = torch.nn.functional.silu(gate) * x
        else:
            residual = (3 * scale * torch.randn(rows, n, generator=g)).to(torch.bfloat16).cuda() if "+" in mode else None
            weight = (1 + 0.1 * torch.randn(n, generator=g)).to(torch.bfloat16).cuda()
            activation, h, staged = rt.fused_input_stage(x, mode="rmsnorm", residual=residual, norm_weight=weight, eps=1e-5,
                                                         beta_table=table, want_residual=True, want_staged=True)
            expect_h = x if residual is None else x + residual
            assert torch.equal(h, expect_h), case
            expect = stage_cases._rms_norm(expect_h, weight, 1e-5)
        difference = (staged.float() - expect.float()).abs()
        assert bool((difference <= expect.float().abs() * 2.0 ** -6 + 1e-30).all()), case
        # a mean summed in another order moves a row's scale by a unit in the last place now and then, and with
        # it the rounding of a few of the row's values: counted loosely, bounded tightly above
        assert int((staged != expect).sum()) <= max(16, rows * n // 50), case
        plain = rt.quantize_activation_cuda(staged, q=Q, betas=ACTIVATION_BETAS, hadamard=True)
        assert stage_cases._same_activation(activation, plain), case


@pytest.mark.parametrize("sweep_seed", [17, 63])
def test_dense_gemm_and_grouped_linears_over_random_shapes(rt, oracle, sweep_seed):
    """The dense BF16 product on every tile and K split over ragged M and N, and the grouped prefill
    linears (both routes) against one call per weight, bit for bit."""
    from conftest import WEIGHT_BETAS
    rng = np.random.default_rng(sweep_seed)
    for _ in range(25):
        m, n = int(rng.integers(1, 1200)), int(rng.integers(1, 700))
        k = 128 * int(rng.integers(1, 17))
        case = (m, n, k)
        g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
        a = torch.randn(m, k, generator=g).to(torch.bfloat16).cuda()
        b = torch.randn(n, k, generator=g).to(torch.bfloat16).cuda()
        ref = bits(a.float() @ b.float().t())
        for tile in [-1] + [int(t) for t in rng.permutation(10)[:4]]:
            split = int(rng.choice([0, 1, 2, 4, 8]))
            if split > 1 and k % (128 * split):
                split = 0
            c = rt.bf16_gemm(a, b, tile=tile, split_k=split)
            assert relative_error(bits(c.float()), ref) <= 2.0 ** -8, (tile, split, case)
    for _ in range(12):
        k = int(rng.choice([256, 512, 1024, 2048]))
        m = int(rng.choice([17, 40, 100, 128, 256, 257, 300, 600]))
        count = int(rng.integers(2, 5 if m < rt.DECODE_ONCE_ROWS else 4))
        unit = 32 if m < rt.DECODE_ONCE_ROWS else 256
        sizes = [unit * int(rng.integers(1, 4)) for _ in range(count)]
        case = (m, k, sizes)
        weights = []
        for i, n_out in enumerate(sizes):
            g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
            w = torch.from_numpy(oracle.hadamard((0.02 * torch.randn(n_out, k, generator=g)).numpy()))
            record = rt.quantize_weight_nqrt4(w.cuda(), q=Q, betas=WEIGHT_BETAS, dither_seed=int(rng.integers(1 << 31)),
                                              tensor_name=f"w{i}")
            weights.append(rt.prepare_fused_linear(record, device="cuda"))
        x = student_t_rows(m, k, seed=int(rng.integers(1 << 20))).to(torch.bfloat16).cuda()
        activation = rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS, hadamard=True)
        assert rt.can_use_w4a4_gemm_grouped(activation, weights), case
        grouped = rt.linear_packed_w4a4_gemm_grouped(activation, weights)
        split, tiles = 1, sum(sizes) // 32
        while split < 16 and tiles * split < 256 and (k // (split * 2)) % 128 == 0:
            split *= 2
        for out, weight in zip(grouped, weights):
            alone = (rt._gemm(activation, weight, output_dtype=torch.bfloat16, split_k=split) if m < rt.DECODE_ONCE_ROWS
                     else rt.linear_packed_w4a4_mma_chunked_staged(activation, weight))
            assert torch.equal(out, alone), case


@pytest.mark.parametrize("sweep_seed", [19, 71])
def test_greedy_sampler_over_random_logits(sweep_seed):
    """The device sampler against torch.argmax over random row counts, vocabulary sizes (odd ones
    take the element loop), dtypes, strided rows, repeated maxima, infinities and NaN (the first NaN
    of a row wins, as in torch.argmax)."""
    from nestquant_aiinfra_amd.runtime.nqkv_hf_backend import greedy_sample_
    rng = np.random.default_rng(sweep_seed)
    g = torch.Generator().manual_seed(sweep_seed)
    for _ in range(60):
        rows = int(rng.integers(1, 33))
        vocab = int(rng.choice([1, 5, 8, 777, 1000, 4096, 32000, 70001, 128256]))
        stride = vocab + int(rng.choice([0, 0, 8, 13]))
        dtype = [torch.bfloat16, torch.float32, torch.float16][rng.integers(3)]
        case = (rows, vocab, stride, dtype)
        storage = torch.randn((rows, stride), generator=g).to(dtype)
        for row in range(rows):
            kind = rng.integers(5)
            if kind == 0:
                storage[row, :vocab] = storage[row, :vocab].round()             # many equal maxima
            elif kind == 1:
                storage[row, int(rng.integers(vocab))] = float("inf")
                storage[row, int(rng.integers(vocab))] = float("inf")
            elif kind == 2:
                storage[row, int(rng.integers(vocab))] = float("nan")
                storage[row, int(rng.integers(vocab))] = float("nan")
            elif kind == 3:
                storage[row, :vocab] = float("-inf")                            # nothing to prefer: index 0
        storage[:, vocab:] = 1e4                                                # beyond the vocabulary: never chosen
        logits = storage.cuda()[:, :vocab]
        values = logits.float().cpu()
        want = values.argmax(-1)
        for row in range(rows):                                                 # NaN is the largest, the first one wins
            nans = torch.isnan(values[row]).nonzero()
            if len(nans):
                want[row] = int(nans[0])
        plain = torch.zeros(rows, dtype=torch.long, device="cuda")
        assert torch.equal(greedy_sample_(logits, plain).cpu(), want), case
