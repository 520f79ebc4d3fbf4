"""Host-side formats and containers, on the CPU: the fixed-width index packing, the NQKV page
container and the NQRT tensor record.  Expected values are the reference's own known answers
(tests/unit/core/test_packing.py:18-90, tests/unit/core/test_kv_format.py:35-47, 80-131) and the
container hash written from the reference (tests/golden/reference_vectors.json)."""

import hashlib

import numpy as np
import pytest
import torch

from conftest import KEY_BETAS, Q, VALUE_BETAS, WEIGHT_BETAS
from nestquant_aiinfra_amd.core.kv_format import PackedNQKVPage
from nestquant_aiinfra_amd.core.packing import PackedNestQuantIndices, pack_nestquant_indices
from nestquant_aiinfra_amd.core.tensor_checkpoint import PackedNestQuantTensor


def _bit_by_bit(values, width):
    out = bytearray((len(values) * width + 7) // 8)
    for i, v in enumerate(values):
        out[i * width // 8] |= int(v) << (i * width % 8)
    return bytes(out)


@pytest.mark.parametrize("cardinality", [2, 4, 14, 256])
def test_packing_is_little_endian_within_a_byte(cardinality):
    codes = torch.arange(24).remainder(cardinality).reshape(1, 3, 8)
    beta = torch.tensor([[0, 1 % cardinality, 2 % cardinality]])
    packed = pack_nestquant_indices(codes, beta, q=cardinality, beta_count=cardinality)
    width = packed.code_bit_width
    assert packed.code_payload == _bit_by_bit(codes.flatten().tolist(), width)
    assert packed.beta_payload == _bit_by_bit(beta.flatten().tolist(), width)
    back_codes, back_beta = packed.unpack()
    assert torch.equal(back_codes, codes) and torch.equal(back_beta, beta)


def test_q14_with_four_betas_known_bytes_and_container_round_trip():
    codes = torch.arange(16).remainder(14).reshape(1, 2, 8)
    beta = torch.tensor([[0, 3]])
    packed = pack_nestquant_indices(codes, beta, q=14, beta_count=4)
    assert (packed.code_bit_width, packed.beta_index_bit_width) == (4, 2)
    assert len(packed.code_payload) == 8 and packed.beta_payload == bytes([0b00001100])
    blob = packed.to_bytes()
    again = PackedNestQuantIndices.from_bytes(blob)
    assert again == packed and again.serialized_bytes == len(blob)
    back_codes, back_beta = again.unpack()
    assert torch.equal(back_codes, codes) and torch.equal(back_beta, beta)
    for damaged in (blob[:-1], blob + b"\0", b"XXXX" + blob[4:], blob[:10]):
        with pytest.raises(ValueError):
            PackedNestQuantIndices.from_bytes(damaged)


def test_row_ranges_unpack_without_reading_the_rest():
    codes = torch.arange(5 * 3 * 8).remainder(14).reshape(5, 3, 8)
    beta = torch.arange(15).remainder(4).reshape(5, 3)          # three 2-bit ids per row: rows start inside bytes
    packed = pack_nestquant_indices(codes, beta, q=14, beta_count=4)
    for start, end in ((0, 1), (1, 4), (4, 5), (2, 2), (0, 5)):
        got_codes, got_beta = packed.unpack_rows(start, end)
        assert torch.equal(got_codes, codes[start:end]) and torch.equal(got_beta, beta[start:end])
    with pytest.raises(ValueError, match="outside"):
        packed.unpack_rows(-1, 2)
    with pytest.raises(ValueError, match="outside"):
        packed.unpack_rows(3, 6)
    with pytest.raises(TypeError):
        packed.unpack_rows(True, 2)


def test_padding_bits_are_zero_and_bad_inputs_are_rejected():
    packed = pack_nestquant_indices(torch.tensor([[[1, 2, 3, 4, 5, 6, 7, 8]]]), torch.tensor([[2]]), q=14, beta_count=4)
    assert packed.beta_payload == bytes([2])
    with pytest.raises(ValueError):
        pack_nestquant_indices(torch.full((1, 1, 8), 14), torch.zeros((1, 1), dtype=torch.int64), q=14, beta_count=4)
    with pytest.raises(ValueError):
        pack_nestquant_indices(torch.zeros((1, 1, 8), dtype=torch.int64), torch.zeros((1, 2), dtype=torch.int64),
                               q=14, beta_count=4)
    with pytest.raises(TypeError):
        pack_nestquant_indices(torch.zeros((1, 1, 8)), torch.zeros((1, 1), dtype=torch.int64), q=14, beta_count=4)


def _golden_page(golden, *, dual=True):
    shape = (16 * 8, 8, 8)
    key = PackedNestQuantIndices(shape, Q, 4, golden["kv_key_codes"].tobytes(), golden["kv_key_betas"].tobytes())
    value = PackedNestQuantIndices(shape, Q, 4, golden["kv_value_codes"].tobytes(), golden["kv_value_betas"].tobytes())
    return PackedNQKVPage(16, 16, 8, 64, Q, KEY_BETAS, torch.bfloat16, key, torch.from_numpy(golden["kv_key_norms"].copy()),
                          value, torch.from_numpy(golden["kv_value_norms"].copy()),
                          value_betas=VALUE_BETAS if dual else None)


def test_nqkv_container_reproduces_the_reference_bytes(golden, golden_meta):
    page = _golden_page(golden)
    blob = page.to_bytes()
    assert len(blob) == page.serialized_bytes == golden_meta["kv_container_v2_bytes"] == 9932
    assert hashlib.sha256(blob).hexdigest() == golden_meta["kv_container_v2_sha256"]
    assert page.payload_bytes == golden_meta["kv_payload_bytes"] == 9728
    report = page.storage_report()
    assert report["format"] == "NQKV-v2" and report["payload_bits_per_entry"] == 4.75
    assert (report["code_bytes"], report["beta_bytes"], report["norm_bytes"]) == (8192, 512, 1024)
    again = PackedNQKVPage.from_bytes(blob)
    assert again.to_bytes() == blob and again.format_version == 2
    assert again.betas == tuple(np.float32(b).item() for b in KEY_BETAS)         # float32 on the wire
    assert torch.equal(again.key_norms, page.key_norms) and again.key_indices == page.key_indices
    # the one-table form omits the second float32 table and its 16-bit count: 18 bytes
    legacy = _golden_page(golden, dual=False)
    assert legacy.format_version == 1
    assert legacy.serialized_bytes == golden_meta["kv_container_v1_bytes"] == 9932 - 18
    assert PackedNQKVPage.from_bytes(legacy.to_bytes()).value_betas is None


def test_nqkv_container_rejects_damage(golden):
    blob = bytearray(_golden_page(golden).to_bytes())
    flipped = bytearray(blob)
    flipped[len(blob) // 2] ^= 1
    with pytest.raises(ValueError, match="checksum"):
        PackedNQKVPage.from_bytes(flipped)
    with pytest.raises(ValueError, match="magic"):
        PackedNQKVPage.from_bytes(b"NQKX" + bytes(blob[4:]))
    with pytest.raises(ValueError, match="version"):
        PackedNQKVPage.from_bytes(bytes(blob[:4]) + b"\x07" + bytes(blob[5:]))
    with pytest.raises(ValueError, match="lengths|shorter"):
        PackedNQKVPage.from_bytes(bytes(blob[:-1]))
    with pytest.raises(ValueError, match="shorter"):
        PackedNQKVPage.from_bytes(bytes(blob[:20]))


def test_nqkv_page_metadata_is_validated(golden):
    import dataclasses
    page = _golden_page(golden)
    for change in ({"valid_tokens": 0}, {"valid_tokens": 17}, {"head_dim": 60}, {"num_kv_heads": 4},
                   {"betas": KEY_BETAS[:3]}, {"betas": (1.0, -1.0, 2.0, 3.0)}, {"q": 13},
                   {"key_norms": page.key_norms[:5]}, {"key_norms": page.key_norms.double()},
                   {"codec_semantics": "something else"}):
        with pytest.raises((ValueError, TypeError)):
            dataclasses.replace(page, **change).to_bytes()
    bad = page.key_norms.clone()
    bad[3] = float("inf")
    with pytest.raises(ValueError, match="finite"):
        dataclasses.replace(page, key_norms=bad).to_bytes()


def test_nqrt_tensor_record_round_trip(golden, golden_meta):
    indices = PackedNestQuantIndices((32, 16, 8), Q, 4, golden["nqrt_code_payload"].tobytes(),
                                     golden["nqrt_beta_payload"].tobytes())
    record = PackedNestQuantTensor(tensor_name="layer.weight", indices=indices,
                                   row_norms=torch.from_numpy(golden["nqrt_norms"].copy()), betas=WEIGHT_BETAS,
                                   feature_count=128, output_dtype=torch.float32, dither_seed=golden_meta["nqrt_seed"],
                                   dither_algorithm="lcg31_mix_v1")
    blob = record.to_bytes()
    again = PackedNestQuantTensor.from_bytes(blob)
    assert again.to_bytes() == blob and again.serialized_bytes == len(blob)
    assert again.indices == indices and again.dither_seed == golden_meta["nqrt_seed"]
    assert torch.equal(again.row_norms, record.row_norms) and again.betas == tuple(WEIGHT_BETAS)
    with pytest.raises(ValueError):
        PackedNestQuantTensor.from_bytes(blob[:-3])
    with pytest.raises(ValueError):
        PackedNestQuantTensor.from_bytes(b"NOPE" + blob[4:])


def test_packages_export_the_operator_names_of_the_path():
    """Every exported name resolves, and the operators the reference's callers import for this path
    (nestquant/runtime/__init__.py, nestquant/models/fused_linear.py) are there under the same names."""
    import nestquant_aiinfra_amd.core as core
    import nestquant_aiinfra_amd.models as models
    import nestquant_aiinfra_amd.runtime as runtime
    for package in (core, models, runtime):
        for name in package.__all__:
            assert getattr(package, name) is not None
        with pytest.raises(AttributeError):
            package.no_such_operator
    wanted = {
        "quantize_activation_cuda", "prepare_fused_linear", "PreparedNQA4Activation", "PreparedNQRTLinear",
        "can_use_w4a4_gemv_m1", "can_use_w4a4_mma_small_m", "can_use_w4a4_mma_m16", "can_use_w4a4_mma_large_m_staged",
        "can_use_w4a4_mma_m128_staged", "can_use_w4a4_mma_chunked_staged", "linear_packed_w4a4_gemv_m1",
        "linear_packed_w4a4_mma_small_m", "linear_packed_w4a4_mma_m16", "linear_packed_w4a4_mma_large_m_staged",
        "linear_packed_w4a4_mma_chunked_staged", "linear_packed_w4a4_gemv_m1_splitk_probe",
        "quantize_nqkv_page_cuda", "dequantize_nqkv_page_triton", "nqkv_decode_attention_batched_k1",
        "NQKVPagePool", "BatchedNQKVMetadata", "NQKVHotColdCache", "BatchedNQKVCacheManager",
        "BatchedNQKVAttentionWorkspace", "BatchedNQKVLlamaCache", "install_batched_nqkv_llama_backend",
        "BatchedNQKVLlamaRunner",
    }
    assert wanted <= set(runtime.__all__)
    assert {"FusedNQRTLinear", "convert_linears_to_fused_nqrt_", "SharedPackedActivationCache"} <= set(models.__all__)
    assert {"PackedNestQuantIndices", "pack_nestquant_indices", "PackedNestQuantTensor", "PackedNQKVPage",
            "NQMCFileReader"} <= set(core.__all__)
