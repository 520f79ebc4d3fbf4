"""Seeded sweeps over random shapes, dtypes and data kinds: the encoder bit for bit against the
oracle, the decode and prefill linears, the KV writer page by page, and both attention kernels.
The fixed cases of the other files pin the shapes the model uses; these pin what lies between them
(ragged row counts, short and long rows, every route's thresholds, slots in any order).

Bars: codes, beta ids, norms and the BF16 decode of the encoder bit-exact; linears <= 1e-2 against
the oracle's FP32 product and <= 2e-3 against its product of BF16-rounded operands (5e-3 for
K <= 256, where a single weight that rounds to the neighbouring BF16 value weighs that much);
decode attention <= 1e-2; prefill attention <= 2e-2 (its products run on the matrix cores with BF16
weights and values, and a head whose value terms cancel loses that much of the result)."""

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
            m = int(rng.choice([17, 31, 32, 33, 64, 100, 128, 200, 287, 288, 300, 513, 600]))
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
                    assert relative_error(_f32(got[row, t]), ref) <= 2e-2, ("prefill attention", split, row, t, case)
