"""GPU parity of the packed W4A4 prefill linear (MFMA), through the C ABI.

Bar: max |y - y_ref| / max |y_ref| <= 1e-2 against the oracle's decode-then-FP32 matmul;
<= 2e-3 against the same product on BF16-rounded operands (what the matrix cores multiply).
"""

import dataclasses

import numpy as np
import pytest
import torch

from conftest import ACTIVATION_BETAS, Q, WEIGHT_BETAS
from gpu_util import bits, oracle_weight, outlier_rows, relative_error
from test_gpu_gemv import BF16_TOLERANCE, TOLERANCE, _record, _references

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    from nestquant_aiinfra_amd.runtime import w4a4_linear
    return w4a4_linear


def _activation(rt, oracle, m, k, seed):
    x = torch.from_numpy(oracle.hadamard(outlier_rows(m, k, seed=seed).numpy())).to(torch.bfloat16).cuda()
    return rt.quantize_activation_cuda(x, q=Q, betas=ACTIVATION_BETAS)


@pytest.mark.parametrize("m", [1, 9, 16, 33, 40, 64, 128, 300])
@pytest.mark.parametrize("k,n_out", [(128, 32), (512, 72), (2048, 96)])
def test_small_shapes_match_oracle(rt, oracle, m, k, n_out):
    seed = 20261201 + m
    _, wc, wb, wn = oracle_weight(oracle, n_out, k, seed=4000 + k + n_out, dither_seed=seed)
    weight = rt.prepare_fused_linear(_record(rt, wc, wb, wn, k, seed), device="cuda")
    activation = _activation(rt, oracle, m, k, seed=3001 + m)
    ref32, ref16 = _references(oracle, activation, rt, wc, wb, wn, seed)
    y = rt._gemm(activation, weight, output_dtype=torch.float32)
    assert relative_error(bits(y), ref32) <= TOLERANCE
    assert relative_error(bits(y), ref16) <= BF16_TOLERANCE
    for split in (1, 2, 4):
        if (k // split) % 128:
            continue
        ys = rt._gemm(activation, weight, output_dtype=torch.float32, split_k=split)
        assert relative_error(bits(ys), ref16) <= BF16_TOLERANCE
        assert torch.equal(ys, rt._gemm(activation, weight, output_dtype=torch.float32, split_k=split))
    # the packed-only path (kernel decodes the activation itself) gives identical bits
    packed_only = dataclasses.replace(activation, decoded=None)
    assert torch.equal(rt._gemm(packed_only, weight, output_dtype=torch.float32), y)
    y16 = rt.linear_packed_w4a4_mma_chunked_staged(activation, weight)
    assert y16.dtype == torch.bfloat16 and relative_error(bits(y16.float()), ref32) <= TOLERANCE


def test_gemm_agrees_with_gemv_rows(rt, oracle):
    """Each prefill row equals the decode kernel's result for that row (same operands)."""
    k, n_out, seed = 2048, 64, 20261301
    _, wc, wb, wn = oracle_weight(oracle, n_out, k, seed=5, dither_seed=seed)
    weight = rt.prepare_fused_linear(_record(rt, wc, wb, wn, k, seed), device="cuda")
    activation = _activation(rt, oracle, 8, k, seed=6)
    a = rt._gemm(activation, weight, output_dtype=torch.float32)
    b = rt._gemv(activation, weight, split_k=1, output_dtype=torch.float32)
    assert relative_error(bits(a), bits(b)) <= 1e-5


@pytest.mark.parametrize("name,k,n_out,wseed,dseed", [("gate_proj", 2048, 8192, 1003, 20261103),
                                                      ("down_proj", 8192, 2048, 1004, 20261104)])
def test_llama_1b_prefill_shapes(rt, oracle, name, k, n_out, wseed, dseed):
    """Full-size prefill shapes at ragged M; weights encoded on the GPU; the oracle checks a
    random subset of 256 output channels (its decode of all channels takes too long here)."""
    g = torch.Generator().manual_seed(wseed)
    w = torch.from_numpy(oracle.hadamard((0.02 * torch.randn(n_out, k, generator=g)).numpy()))
    record = rt.quantize_weight_nqrt4(w.cuda(), q=Q, betas=WEIGHT_BETAS, dither_seed=dseed, tensor_name=name)
    weight = rt.prepare_fused_linear(record, device="cuda")
    rows = np.sort(np.random.default_rng(1).choice(n_out, size=256, replace=False))
    codes = oracle.unpack_unsigned(np.frombuffer(record.indices.code_payload, np.uint8), n_out * k, 4).reshape(n_out, k)
    beta = oracle.unpack_unsigned(np.frombuffer(record.indices.beta_payload, np.uint8), n_out * k // 8, 2).reshape(n_out, k // 8)
    norms = record.row_norms.numpy()
    dither = oracle.dither_stateless(n_out * k // 8, dseed).reshape(n_out, k // 8, 8)[rows]
    w_hat = oracle.dequantize_rows(codes[rows], beta[rows], norms[rows], WEIGHT_BETAS, Q, dither=dither)
    for m in (9, 16, 40, 64, 128, 384):                  # up to 16 rows gate_proj decodes in registers
        activation = _activation(rt, oracle, m, k, seed=3001)
        a_codes = oracle.unpack_unsigned(bits(activation.code_payload), m * k, 4)
        a_beta = oracle.unpack_unsigned(bits(activation.beta_payload), m * k // 8, 2)
        a_hat = oracle.dequantize_rows(a_codes, a_beta, bits(activation.row_norms), ACTIVATION_BETAS, Q)
        ref32 = oracle.matmul_nt(a_hat, w_hat)
        y = rt.linear_packed_w4a4_mma_chunked_staged(activation, weight)
        assert y.dtype == torch.bfloat16 and tuple(y.shape) == (m, n_out)
        assert relative_error(bits(y.float())[:, rows], ref32) <= TOLERANCE, (name, m)
        if m == 384:
            # 384 rows take the decode-once route by default; an explicit single slice keeps the fused
            # kernel (the weight decoded inside the multiply): both must meet the oracle
            fused = rt._gemm(activation, weight, output_dtype=torch.bfloat16, split_k=1)
            assert relative_error(bits(fused.float())[:, rows], ref32) <= TOLERANCE, (name, m, "fused")


def test_slice_and_pad_matches_reference_chunking(rt, oracle):
    """Zero-norm padding rows decode to zeros; chunked results equal the one-launch result."""
    k, n_out, seed = 512, 48, 20261302
    _, wc, wb, wn = oracle_weight(oracle, n_out, k, seed=8, dither_seed=seed)
    weight = rt.prepare_fused_linear(_record(rt, wc, wb, wn, k, seed), device="cuda")
    activation = _activation(rt, oracle, 40, k, seed=9)
    whole = rt._gemm(activation, weight, output_dtype=torch.float32)
    chunk = rt.slice_pad_packed_activation_rows(activation, 32, 8, 32)
    part = rt._gemm(chunk, weight, output_dtype=torch.float32)
    assert torch.equal(part[:8], whole[32:40]) and not part[8:].any()
    # a 16-row chunk takes the decode-in-register kernel: same products, another summation order
    small = rt._gemm(rt.slice_pad_packed_activation_rows(activation, 32, 8, 16), weight, output_dtype=torch.float32)
    assert relative_error(bits(small[:8]), bits(whole[32:40])) < 1e-5 and not small[8:].any()
    packed_only = dataclasses.replace(chunk, decoded=None)
    assert torch.equal(rt._gemm(packed_only, weight, output_dtype=torch.float32), part)


@pytest.mark.parametrize("k,n_out", [(2048, 2048), (512, 200)])
def test_long_prefill_decodes_the_weight_once(rt, oracle, k, n_out):
    """From DECODE_ONCE_ROWS rows on, BF16 outputs come from nq_w4a4_decode_weight + the dense
    matrix-core GEMM inside nq_w4a4_gemm: the decoded weight equals the oracle's BF16-rounded weight (resolved form: but for
    rare one-step roundings) and the product stays within the bar; below the threshold and for
    FP32 outputs the fused kernel runs."""
    from test_gpu_gemv import _record
    seed = 20261150
    _, wc, wb, wn = oracle_weight(oracle, n_out, k, seed=4000 + k, dither_seed=seed)
    record = _record(rt, wc, wb, wn, k, seed)
    weight = rt.prepare_fused_linear(record, device="cuda")
    streams_only = rt.prepare_fused_linear(record, device="cuda", resolve=False)
    w_hat = oracle.bf16_round(oracle.dequantize_rows(wc, wb, wn, WEIGHT_BETAS, Q, seed=seed))
    # the kernels form beta * (norm / sqrt(K)) first (the oracle multiplies by beta, then by the
    # row scale): same lattice points, FP32 products that differ in the last place, hence rare
    # one-step differences after the BF16 rounding.  The resolved form takes the dither to 2^-17 lattice
    # units before the scale, which only shows on weights that are themselves almost zero.
    row_peak = np.abs(w_hat).max(axis=1, keepdims=True)
    for form, deviation, share in ((streams_only, 2.0 ** -22, 500), (weight, 2.0 ** -16, 50)):
        decoded = bits(rt.decode_weight_bf16(form).float())
        assert np.all(np.abs(decoded - w_hat) <= np.abs(w_hat) * 2.0 ** -7 + row_peak * deviation)
        assert np.count_nonzero(decoded != w_hat) <= decoded.size // share + 1
    from_streams, from_resolved = (bits(rt.decode_weight_bf16(form).float()) for form in (streams_only, weight))
    assert np.count_nonzero(from_streams != from_resolved) <= from_streams.size // 50 + 1

    m = rt.DECODE_ONCE_ROWS + 37
    activation = _activation(rt, oracle, m, k, seed=77)
    a_codes = oracle.unpack_unsigned(bits(activation.code_payload), m * k, 4)
    a_beta = oracle.unpack_unsigned(bits(activation.beta_payload), m * k // 8, 2)
    a_hat = oracle.dequantize_rows(a_codes, a_beta, bits(activation.row_norms), ACTIVATION_BETAS, Q)
    ref = oracle.matmul_nt(a_hat, oracle.dequantize_rows(wc, wb, wn, WEIGHT_BETAS, Q, seed=seed))
    y = rt.linear_packed_w4a4_mma_chunked_staged(activation, weight)
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (m, n_out)
    assert relative_error(bits(y.float()), ref) <= TOLERANCE
    fused = rt._gemm(activation, weight, output_dtype=torch.bfloat16, split_k=1)      # explicit split: fused kernel
    assert relative_error(bits(y.float()), bits(fused.float())) <= 5e-3


@pytest.mark.parametrize("m,n,k", [(300, 200, 128), (257, 520, 384), (64, 64, 128), (1000, 72, 256), (384, 8192, 2048),
                                   (384, 2048, 8192), (130, 136, 1024), (100, 36, 128), (70, 33, 256), (33, 12, 128)])
def test_dense_bf16_gemm_against_float32(rt, m, n, k):
    """nq_bf16_gemm (the multiply of the decode-once route) against the FP32 product of the same BF16
    operands: FP32 accumulation and one BF16 rounding of the result leave <= 2^-8 relative to the
    largest output; every workgroup tile shape on both kernels (7..9: the small tiles on the kernel
    with movers and multipliers), ragged edges included, and rows of C that are multiples of 16 bytes
    (stored by whole rows through LDS), of 8 bytes (four columns per lane) and of neither."""
    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).cuda()
    b = torch.randn(n, k, generator=g).to(torch.bfloat16).cuda()
    ref = bits(a.float() @ b.float().t())
    for tile in range(-1, 10):
        c = rt.bf16_gemm(a, b, tile=tile)
        assert c.dtype == torch.bfloat16 and tuple(c.shape) == (m, n)
        assert relative_error(bits(c.float()), ref) <= 2.0 ** -8, (tile,)
    # K split: slabs of float32 partial results added in ascending order by a second launch
    for split in (2, 4, 8):
        if k % (128 * split):
            with pytest.raises(RuntimeError, match="K split"):
                rt.bf16_gemm(a, b, split_k=split)
            continue
        for tile in (-1, 3, 6, 7, 9):
            c = rt.bf16_gemm(a, b, tile=tile, split_k=split)
            assert relative_error(bits(c.float()), ref) <= 2.0 ** -8, (tile, split)
    assert torch.equal(rt.bf16_gemm(a, b, split_k=1), rt.bf16_gemm(a, b, split_k=1))
    with pytest.raises(ValueError, match="multiple of 128"):
        rt.bf16_gemm(a[:, :64].contiguous(), b[:, :64].contiguous())


@pytest.mark.parametrize("m,k,sizes", [(300, 512, (512, 256, 256)), (1024, 2048, (2048, 512, 512)), (384, 1024, (768, 768))])
def test_grouped_prefill_linears_equal_one_call_per_weight(rt, oracle, m, k, sizes):
    """q, k and v (or gate and up) of one activation through one dense product over their stacked
    decoded weights (`linear_packed_w4a4_gemm_grouped`, `nq_bf16_gemm_split`): every output is bit
    for bit what the decode-once route gives for its weight alone (same decoded BF16 operands,
    same sum over K per element, whatever tile the product runs on)."""
    weights = []
    for i, n_out in enumerate(sizes):
        g = torch.Generator().manual_seed(7000 + i)
        w = torch.from_numpy(oracle.hadamard((0.02 * torch.randn(n_out, k, generator=g)).numpy()))
        record = rt.quantize_weight_nqrt4(w.cuda(), q=Q, betas=WEIGHT_BETAS, dither_seed=20270000 + i, tensor_name=f"w{i}")
        weights.append(rt.prepare_fused_linear(record, device="cuda"))
    activation = _activation(rt, oracle, m, k, seed=7100)
    assert rt.can_use_w4a4_gemm_grouped(activation, weights)
    grouped = rt.linear_packed_w4a4_gemm_grouped(activation, weights)
    for out, weight, n_out in zip(grouped, weights, sizes):
        alone = rt.linear_packed_w4a4_mma_chunked_staged(activation, weight)
        assert out.dtype == torch.bfloat16 and tuple(out.shape) == (m, n_out)
        assert torch.equal(out, alone), n_out
    # a decode step's rows (the grouped GEMV's), or a single weight: refused
    short = _activation(rt, oracle, 16, k, seed=7101)
    assert not rt.can_use_w4a4_gemm_grouped(short, weights)
    with pytest.raises(ValueError, match="grouped prefill linears"):
        rt.linear_packed_w4a4_gemm_grouped(short, weights)
    assert not rt.can_use_w4a4_gemm_grouped(activation, weights[:1])


@pytest.mark.parametrize("m,k,sizes", [(17, 512, (256, 64, 64)), (128, 2048, (2048, 512, 512)), (256, 1024, (512, 512)),
                                       (40, 256, (32, 64, 96, 32)), (128, 2048, (8192, 8192)), (100, 8192, (64, 32)),
                                       (96, 512, (8192, 8192)), (250, 256, (8192, 4096, 4160)), (95, 256, (8192, 8192))])
def test_grouped_short_prefill_linears_equal_one_launch_per_weight(rt, oracle, m, k, sizes):
    """Below the decode-once size one launch of the fused kernel walks the channels of all the
    weights (`nq_w4a4_gemm_grouped`): every output is bit for bit what the kernel gives for its
    weight alone with the K split the group runs with (the split follows the sum of the widths).  A
    group of 16384 channels or more at 96 to 256 rows runs with 64-channel tiles, a weight alone with
    32-channel ones: the same bits."""
    from nestquant_aiinfra_amd.runtime.w4a4_linear import _gemm
    weights = []
    for i, n_out in enumerate(sizes):
        g = torch.Generator().manual_seed(7200 + i)
        w = torch.from_numpy(oracle.hadamard((0.02 * torch.randn(n_out, k, generator=g)).numpy()))
        record = rt.quantize_weight_nqrt4(w.cuda(), q=Q, betas=WEIGHT_BETAS, dither_seed=20280000 + i, tensor_name=f"w{i}")
        weights.append(rt.prepare_fused_linear(record, device="cuda"))
    activation = _activation(rt, oracle, m, k, seed=7300)
    assert rt.can_use_w4a4_gemm_grouped(activation, weights)
    grouped = rt.linear_packed_w4a4_gemm_grouped(activation, weights)
    split, tiles = 1, sum(sizes) // 32
    while split < 16 and tiles * split < 256 and (k // (split * 2)) % 128 == 0:
        split *= 2
    for out, weight, n_out in zip(grouped, weights, sizes):
        alone = _gemm(activation, weight, output_dtype=torch.bfloat16, split_k=split)
        assert out.dtype == torch.bfloat16 and tuple(out.shape) == (m, n_out)
        assert torch.equal(out, alone), (n_out, split)
    # the same call twice gives the same bits (the slabs are added in order)
    again = rt.linear_packed_w4a4_gemm_grouped(activation, weights)
    assert all(torch.equal(a, b) for a, b in zip(grouped, again))


@pytest.mark.parametrize("m,k,n_out,split", [(128, 256, 16400, 0), (200, 128, 16417, 0), (96, 4096, 4100, 0), (130, 1024, 2050, 8)])
def test_wide_tiles_on_ragged_widths_match_oracle(rt, oracle, m, k, n_out, split):
    """The 64-channel tiles of the fused kernel (96 to 256 rows; 16384 channels and more, rows of 4096
    values and more with K slabs, or a split that leaves 256 workgroups) where the last workgroup holds
    a few channels only: against the oracle's product, FP32 and BF16 outputs."""
    seed = 20300000 + n_out
    _, wc, wb, wn = oracle_weight(oracle, n_out, k, seed=9100 + n_out % 97, dither_seed=seed)
    weight = rt.prepare_fused_linear(_record(rt, wc, wb, wn, k, seed), device="cuda")
    activation = _activation(rt, oracle, m, k, seed=9200 + m)
    ref32, ref16 = _references(oracle, activation, rt, wc, wb, wn, seed)
    y = rt._gemm(activation, weight, output_dtype=torch.float32, split_k=split)
    assert relative_error(bits(y), ref32) <= TOLERANCE
    assert relative_error(bits(y), ref16) <= BF16_TOLERANCE
    y16 = rt._gemm(activation, weight, output_dtype=torch.bfloat16, split_k=split)
    assert torch.equal(y16, y.to(torch.bfloat16))
