"""The C-ABI library loads without a GPU and exports exactly what include/nqhip.h declares."""

import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


def _declared():
    text = (ROOT / "include" / "nqhip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nq_[a-z0-9_]+)\s*\(", text)))


def test_header_bindings_and_exports_agree():
    from nestquant_aiinfra_amd import _native
    declared = _declared()
    assert declared, "no declarations found"
    assert sorted(_native.SIGNATURES) == declared
    if not _native.LIBRARY_PATH.exists():
        from nestquant_aiinfra_amd import build
        build.build()
    lib = ctypes.CDLL(str(_native.LIBRARY_PATH))
    for name in declared:
        assert hasattr(lib, name), name
    assert _native.library().nq_abi_version() >= 1
    assert _native.library().nq_last_error() is not None


def test_host_side_validation_needs_no_gpu():
    """Shape checks run before anything is launched and name the offending argument."""
    from nestquant_aiinfra_amd import _native
    lib = _native.library()
    status = lib.nq_quantize_rows(None, 0, 1, 40, 14, None, 4, 0, 0, 0, 0, None, None, None, None, None)
    assert status == _native.NQ_ERR_SHAPE and b"multiple of 32" in lib.nq_last_error()
    with pytest.raises(ValueError, match="multiple of 32"):
        _native.check(status)
    status = lib.nq_w4a4_gemv(*([None] * 11), 9, 2048, 2048, 0, 1, 0, None, 0, None, 0, None)
    assert status == _native.NQ_ERR_SHAPE and b"outside [1, 8]" in lib.nq_last_error()
    status = lib.nq_dequantize_rows(None, None, None, None, 1, 64, 14, 1, -5, 0, None, 0, None)
    assert status == _native.NQ_ERR_ARGUMENT
    assert lib.nq_w4a4_gemv_workspace_bytes(1, 8192, 2048, 8, 1) == 8 * 2048 * 4
    # the attention's partial results: chunks of 4 pages while the launch stays within 32 (row, chunk) pairs,
    # 8 pages up to 100 pairs, 16 beyond
    assert lib.nq_nqkv_attention_parts(8, 23) == 4 and lib.nq_nqkv_attention_parts(1, 64) == 17
    assert lib.nq_nqkv_attention_parts(8, 256) == 17 and lib.nq_nqkv_attention_parts(8, 400) == 26
    assert lib.nq_nqkv_attention_parts(1, 256) == 33 and lib.nq_nqkv_attention_parts(4, 21) == 7
    assert lib.nq_nqkv_attention_parts(9, 21) == 4 and lib.nq_nqkv_attention_parts(16, 64) == 5
    assert lib.nq_nqkv_attention_parts(12, 64) == 5 and lib.nq_nqkv_attention_parts(0, 5) == 0
    assert lib.nq_nqkv_attention_workspace_bytes(8, 32, 64, 23) == 8 * 32 * 4 * 66 * 4
    status = lib.nq_attention_output_stage(None, 8, 32, 128, 7, None, 14, None, 4, 1, None, None, None, None, None)
    assert status == _native.NQ_ERR_SHAPE and b"head_dim 128 is not 64" in lib.nq_last_error()
    status = lib.nq_attention_output_stage(None, 8, 32, 64, 600, None, 14, None, 4, 1, None, None, None, None, None)
    assert status == _native.NQ_ERR_SHAPE and b"at most 512" in lib.nq_last_error()
    status = lib.nq_attention_output_stage(None, 8, 32, 64, 7, None, 14, None, 4, 1, None, None, None, None, None)
    assert status == _native.NQ_ERR_ARGUMENT and b"workspace" in lib.nq_last_error()
    # the sampler: shapes first, then pointers, then its workspace
    assert lib.nq_greedy_sample_workspace_bytes(8) == 32 + 8 * 32 * 12 and lib.nq_greedy_sample_workspace_bytes(0) == 0
    status = lib.nq_greedy_sample(None, 1, 8, 100, 50, None, None, None, None, 0, None, None, 0, None)
    assert status == _native.NQ_ERR_SHAPE and b"row_stride" in lib.nq_last_error()
    status = lib.nq_greedy_sample(None, 1, 8, 100, 100, None, None, None, None, 0, None, None, 0, None)
    assert status == _native.NQ_ERR_ARGUMENT and b"null pointer" in lib.nq_last_error()
    # the LM-head stream: row count, K, then pointers
    status = lib.nq_bf16_rows_linear(None, None, 17, 2048, 128256, None, None)
    assert status == _native.NQ_ERR_SHAPE and b"outside [1, 16]" in lib.nq_last_error()
    status = lib.nq_bf16_rows_linear(None, None, 8, 1024, 128256, None, None)
    assert status == _native.NQ_ERR_SHAPE and b"not 2048, 4096 or 8192" in lib.nq_last_error()
    status = lib.nq_bf16_rows_linear(None, None, 8, 2048, 128256, None, None)
    assert status == _native.NQ_ERR_ARGUMENT and b"null pointer" in lib.nq_last_error()
    status = lib.nq_bf16_rows_linear_grouped(None, None, 8, 8192, 4, None, None, None)
    assert status == _native.NQ_ERR_ARGUMENT and b"between one and three outputs" in lib.nq_last_error()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from nestquant_aiinfra_amd import _native
    monkeypatch.setattr(_native, "_LIB", None)
    monkeypatch.setattr(_native, "LIBRARY_PATH", tmp_path / "libnqhip.so")
    with pytest.raises(_native.NativeLibraryMissing, match="no fallback"):
        _native.library()
