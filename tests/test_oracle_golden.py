"""The CPU oracle against vectors produced by the reference's own CPU core.

These pin what no closed form does: E8 decisions on exact Voronoi ties in torch's
CPU float order, undithered decodes, per-block beta choice, row-norm bits, and the
payload bytes of NQRT4 records and NQKV pages.
"""

import hashlib

import numpy as np

from conftest import ACTIVATION_BETAS, KEY_BETAS, Q, VALUE_BETAS, WEIGHT_BETAS


def test_nearest_e8_points_and_distances(oracle, golden):
    point, dist = oracle.nearest_e8(golden["e8_x"])
    assert np.array_equal(point, golden["e8_point"])
    assert np.array_equal(dist, golden["e8_dist"])


def test_undithered_decode_including_boundary_blocks(oracle, golden):
    out = oracle.decode_nested(golden["decode_codes"].astype(np.int32), Q)
    assert np.array_equal(out, golden["decode_out"])
    # the three blocks the reference's GPU test singles out as exact Voronoi ties
    assert golden["decode_codes"][:3].tolist() == [
        [5, 12, 3, 0, 7, 3, 9, 2], [5, 5, 2, 7, 2, 4, 10, 2], [3, 0, 2, 12, 4, 9, 7, 2]]


def test_stateless_dither(oracle, golden):
    for seed in (0, 20261025, 2**31 - 1):
        assert np.array_equal(oracle.dither_stateless(64, seed), golden[f"dither_{seed}"])
    assert np.array_equal(oracle.dither_stateless(16, 20261025, block_offset=1000),
                          golden["dither_offset_1000_seed_20261025"])


def test_quantize_rows_undithered(oracle, golden):
    for name in ("qr64", "qr2048"):
        codes, beta, norms = oracle.quantize_rows(golden[f"{name}_x"], Q, ACTIVATION_BETAS)
        assert np.array_equal(norms, golden[f"{name}_norms"]), name
        assert np.array_equal(codes, golden[f"{name}_codes"]), name
        assert np.array_equal(beta, golden[f"{name}_beta"]), name
        deq = oracle.dequantize_rows(codes, beta, norms, ACTIVATION_BETAS, Q)
        assert np.array_equal(deq, golden[f"{name}_deq"]), name
    assert not golden["qr64_deq"][5].any()          # the zero row stays zero


def test_quantize_rows_long_rows(oracle, golden_long_rows):
    """The eight-chain row norm and the scaling hold at the down_proj activation width."""
    for name in ("qr8192", "qr4096"):
        x = (golden_long_rows[f"{name}_x_bf16"].view(np.uint16).astype(np.uint32) << 16).view(np.float32)
        codes, beta, norms = oracle.quantize_rows(x, Q, ACTIVATION_BETAS)
        assert np.array_equal(norms, golden_long_rows[f"{name}_norms"]), name
        assert np.array_equal(codes.reshape(golden_long_rows[f"{name}_codes"].shape), golden_long_rows[f"{name}_codes"]), name
        assert np.array_equal(beta.reshape(golden_long_rows[f"{name}_beta"].shape), golden_long_rows[f"{name}_beta"]), name


def test_nqrt4_record_payloads_and_dequantize(oracle, golden, golden_meta):
    seed = golden_meta["nqrt_seed"]
    w = golden["nqrt_w"]
    dither = oracle.dither_stateless(32 * 16, seed).reshape(32, 16, 8)
    codes, beta, norms = oracle.quantize_rows(w, Q, WEIGHT_BETAS, dither=dither)
    assert np.array_equal(oracle.pack_unsigned(codes, 4), golden["nqrt_code_payload"])
    assert np.array_equal(oracle.pack_unsigned(beta, 2), golden["nqrt_beta_payload"])
    assert np.array_equal(norms, golden["nqrt_norms"])
    deq = oracle.dequantize_rows(codes, beta, norms, WEIGHT_BETAS, Q, seed=seed)
    assert np.array_equal(deq, golden["nqrt_deq"])


def _bf16_bits_to_f32(bits):
    return (bits.astype(np.uint16).astype(np.uint32) << 16).view(np.float32)


def test_nqkv_page_payload(oracle, golden, golden_meta):
    key = _bf16_bits_to_f32(golden["kv_key_bf16_bits"])
    value = _bf16_bits_to_f32(golden["kv_value_bf16_bits"])
    page = oracle.nqkv_page_payload(key, value, page_size=16, q=Q,
                                    key_betas=KEY_BETAS, value_betas=VALUE_BETAS)
    for stream in ("key_codes", "key_betas", "key_norms", "value_codes", "value_betas", "value_norms"):
        assert np.array_equal(page[stream], golden[f"kv_{stream}"]), stream
    assert sum(page[s].nbytes for s in page) == golden_meta["kv_payload_bytes"] == 9728
    # 4.75 bits per entry; the dual-table container is 18 bytes longer than the legacy one
    assert 9728 * 8 / (2 * 16 * 8 * 64) == 4.75
    assert golden_meta["kv_container_v2_bytes"] - golden_meta["kv_container_v1_bytes"] == 18
    # partially filled page: rows after the valid prefix are encoded zeros
    partial = oracle.nqkv_page_payload(key[:5], value[:5], page_size=16, q=Q,
                                       key_betas=KEY_BETAS, value_betas=KEY_BETAS)
    assert np.array_equal(partial["key_codes"], golden["kv_partial_key_codes"])
    assert np.array_equal(partial["key_norms"], golden["kv_partial_key_norms"])
    assert not partial["key_norms"][5 * 8:].any()


def test_config1_payload_hashes(oracle, golden, golden_meta):
    """2048 x 2048 plumbing case: payload SHA-256 of the reference's packed streams."""
    import torch

    ref = golden_meta["config1"]
    g = torch.Generator().manual_seed(58)
    x0 = torch.randn(2048, 2048, generator=g)
    signs = (2 * torch.randint(0, 2, (2048,), generator=g) - 1).float()
    xr = oracle.hadamard((x0 * signs).numpy())
    assert hashlib.sha256(xr.tobytes()).hexdigest() == ref["input_sha256"]

    def sha(a):
        return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()

    codes, beta, norms = oracle.quantize_rows(xr, Q, ACTIVATION_BETAS)
    assert sha(oracle.pack_unsigned(codes, 4)) == ref["A_code_sha256"]
    assert sha(oracle.pack_unsigned(beta, 2)) == ref["A_beta_sha256"]
    assert sha(norms) == ref["A_norm_sha256"]

    dither = oracle.dither_stateless(2048 * 256, ref["dither_seed"]).reshape(2048, 256, 8)
    wc, wb, wn = oracle.quantize_rows(xr, Q, WEIGHT_BETAS, dither=dither)
    assert sha(oracle.pack_unsigned(wc, 4)) == ref["B_code_sha256"]
    assert sha(oracle.pack_unsigned(wb, 2)) == ref["B_beta_sha256"]

    ac, ab, an = oracle.quantize_rows(golden["config1_act"], Q, ACTIVATION_BETAS)
    assert sha(oracle.pack_unsigned(ac, 4)) == ref["act_code_sha256"]
    w_hat = oracle.dequantize_rows(wc, wb, wn, WEIGHT_BETAS, Q, seed=ref["dither_seed"])
    a_hat = oracle.dequantize_rows(ac, ab, an, ACTIVATION_BETAS, Q)
    y = oracle.matmul_nt(a_hat, w_hat).reshape(-1)
    scale = np.abs(golden["config1_y"]).max()
    assert np.abs(y - golden["config1_y"]).max() <= 1e-5 * scale
