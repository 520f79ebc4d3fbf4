"""CPU oracle for the packed W4A4KV4 path -- TEST INFRASTRUCTURE ONLY.

A numpy-facing loader for ``libnq_oracle.so`` (built from ``nq_oracle.c`` by the
Makefile beside it).  The C file restates the reference's torch-CPU algorithm;
this module only marshals arrays.  It must never be imported by the shipped
package: only the tests, the smoke check and the benchmark's CPU-baseline leg
use it, and only as the checker.

Function -> reference (paths relative to the reference checkout):
  nearest_e8            nestquant/core/lattice.py:37-81
  encode_nested         nestquant/core/codec.py:53-102
  decode_nested         nestquant/core/codec.py:105-142
  dither_stateless      nestquant/core/codec.py:176-224
  quantize_rows         nestquant/core/quantizer.py:214-301
  dequantize_rows       nestquant/core/quantizer.py:39-51
  pack_unsigned/unpack  nestquant/core/packing.py:191-225
  hadamard              nestquant/core/rotation.py:12-27
  nqkv_page_payload     nestquant/core/kv_format.py:71-131
  attention_dense       nestquant/runtime/nqkv_attention.py:14-86
"""

from __future__ import annotations

import ctypes
import math
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libnq_oracle.so"
_LIB = None

_f32p = ctypes.POINTER(ctypes.c_float)
_u8p = ctypes.POINTER(ctypes.c_uint8)
_i32p = ctypes.POINTER(ctypes.c_int32)
_u32p = ctypes.POINTER(ctypes.c_uint32)
_u64p = ctypes.POINTER(ctypes.c_uint64)


def build() -> Path:
    """Compile the oracle with gcc (idempotent)."""
    subprocess.run(["make", "-C", str(_HERE), "--no-print-directory"], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        if not _LIB_PATH.exists():
            build()
        _LIB = ctypes.CDLL(str(_LIB_PATH))
    return _LIB


def _p(array: np.ndarray, kind):
    return array.ctypes.data_as(kind)


def _f32(array) -> np.ndarray:
    return np.ascontiguousarray(array, dtype=np.float32)


def beta_table(betas) -> np.ndarray:
    """Python-double betas cast to float32, as every reference call site does."""
    return np.asarray([float(b) for b in betas], dtype=np.float32)


def nearest_e8(x) -> tuple[np.ndarray, np.ndarray]:
    x = _f32(x)
    out = np.empty_like(x)
    n = x.size // 8
    dist = np.empty(x.shape[:-1], dtype=np.float32)
    lib().nqo_nearest_e8(_p(x, _f32p), _p(out, _f32p), _p(dist, _f32p), ctypes.c_size_t(n))
    return out, dist


def encode_nested(x, q: int, dither=None) -> np.ndarray:
    x = _f32(x)
    d = None if dither is None else _f32(dither)
    code = np.empty(x.shape, dtype=np.int32)
    lib().nqo_encode_nested(_p(x, _f32p), None if d is None else _p(d, _f32p),
                            ctypes.c_int(q), _p(code, _i32p), ctypes.c_size_t(x.size // 8))
    return code


def decode_nested(code, q: int, dither=None) -> np.ndarray:
    code = np.ascontiguousarray(code, dtype=np.int32)
    d = None if dither is None else _f32(dither)
    out = np.empty(code.shape, dtype=np.float32)
    lib().nqo_decode_nested(_p(code, _i32p), None if d is None else _p(d, _f32p),
                            ctypes.c_int(q), _p(out, _f32p), ctypes.c_size_t(code.size // 8))
    return out


def hash_lcg31(counters, seed: int) -> np.ndarray:
    counters = np.ascontiguousarray(counters, dtype=np.uint64)
    out = np.empty(counters.shape, dtype=np.uint32)
    lib().nqo_hash_lcg31(_p(counters, _u64p), ctypes.c_uint64(seed), _p(out, _u32p),
                         ctypes.c_size_t(counters.size))
    return out


def dither_stateless(count: int, seed: int, block_offset: int = 0) -> np.ndarray:
    if not 0 <= seed < (1 << 31):
        raise ValueError("seed must be an integer in [0, 2**31)")
    if block_offset + count > (1 << 31) // 8:
        raise ValueError("block range exceeds the stateless dither counter space")
    out = np.empty((count, 8), dtype=np.float32)
    lib().nqo_dither_stateless(ctypes.c_uint64(count), ctypes.c_uint64(seed),
                               ctypes.c_uint64(block_offset), _p(out, _f32p))
    return out


def row_norms(x) -> np.ndarray:
    x = _f32(x)
    rows, n = x.shape
    out = np.empty(rows, dtype=np.float32)
    lib().nqo_row_norms(_p(x, _f32p), ctypes.c_size_t(rows), ctypes.c_size_t(n), _p(out, _f32p))
    return out


def quantize_rows(x, q: int, betas, dither=None):
    """Returns (codes u8 [R, n/8, 8], beta_idx u8 [R, n/8], norms f32 [R])."""
    x = _f32(x)
    rows, n = x.shape
    if n % 8 or rows == 0:
        raise ValueError("matrix must have nonempty rows and a feature count divisible by 8")
    table = beta_table(betas)
    d = None if dither is None else _f32(dither)
    codes = np.empty((rows, n // 8, 8), dtype=np.uint8)
    beta_idx = np.empty((rows, n // 8), dtype=np.uint8)
    norms = np.empty(rows, dtype=np.float32)
    lib().nqo_quantize_rows(_p(x, _f32p), ctypes.c_size_t(rows), ctypes.c_size_t(n),
                            ctypes.c_int(q), _p(table, _f32p), ctypes.c_int(len(table)),
                            None if d is None else _p(d, _f32p),
                            _p(codes, _u8p), _p(beta_idx, _u8p), _p(norms, _f32p))
    return codes, beta_idx, norms


def dequantize_rows(codes, beta_idx, norms, betas, q: int, *, dither=None, seed=None) -> np.ndarray:
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    beta_idx = np.ascontiguousarray(beta_idx, dtype=np.uint8)
    norms = _f32(norms)
    rows = norms.shape[0]
    n = codes.size // rows
    table = beta_table(betas)
    d = None if dither is None else _f32(dither)
    out = np.empty((rows, n), dtype=np.float32)
    lib().nqo_dequantize_rows(_p(codes, _u8p), _p(beta_idx, _u8p), _p(norms, _f32p),
                              _p(table, _f32p), ctypes.c_int(q), ctypes.c_size_t(rows),
                              ctypes.c_size_t(n), None if d is None else _p(d, _f32p),
                              ctypes.c_int(0 if seed is None else 1),
                              ctypes.c_uint64(0 if seed is None else seed), _p(out, _f32p))
    return out


def pack_unsigned(values, width: int) -> np.ndarray:
    values = np.ascontiguousarray(values, dtype=np.uint8).reshape(-1)
    out = np.empty((values.size * width + 7) // 8, dtype=np.uint8)
    lib().nqo_pack_unsigned(_p(values, _u8p), ctypes.c_size_t(values.size), ctypes.c_int(width),
                            _p(out, _u8p))
    return out


def unpack_unsigned(payload, count: int, width: int) -> np.ndarray:
    payload = np.ascontiguousarray(payload, dtype=np.uint8).reshape(-1)
    if payload.size != (count * width + 7) // 8:
        raise ValueError("payload size does not match expected packed value count")
    out = np.empty(count, dtype=np.uint8)
    lib().nqo_unpack_unsigned(_p(payload, _u8p), ctypes.c_size_t(count), ctypes.c_int(width),
                              _p(out, _u8p))
    return out


def hadamard(x) -> np.ndarray:
    x = np.array(x, dtype=np.float32, order="C", copy=True)
    n = x.shape[-1]
    if n < 1 or n & (n - 1):
        raise ValueError("feature dimension must be a positive power of two")
    lib().nqo_hadamard_f32(_p(x, _f32p), ctypes.c_size_t(x.size // n), ctypes.c_size_t(n))
    return x


def matmul_nt(a, w) -> np.ndarray:
    """out[m, n] = sum_k a[m, k] * w[n, k], float32 operands, double accumulation."""
    a, w = _f32(a), _f32(w)
    m, k = a.shape
    n = w.shape[0]
    out = np.empty((m, n), dtype=np.float32)
    lib().nqo_matmul_nt(_p(a, _f32p), _p(w, _f32p), ctypes.c_size_t(m), ctypes.c_size_t(n),
                        ctypes.c_size_t(k), _p(out, _f32p))
    return out


def attention_dense(query, key, value, scale: float | None = None) -> np.ndarray:
    """query [Hq, D]; key/value [T, Hkv, D] float32 -> [Hq, D]."""
    query, key, value = _f32(query), _f32(key), _f32(value)
    q_heads, dim = query.shape
    tokens, kv_heads, _ = key.shape
    if scale is None:
        scale = 1.0 / math.sqrt(dim)
    out = np.empty((q_heads, dim), dtype=np.float32)
    lib().nqo_attention_dense(_p(query, _f32p), _p(key, _f32p), _p(value, _f32p),
                              ctypes.c_size_t(tokens), ctypes.c_int(q_heads),
                              ctypes.c_int(kv_heads), ctypes.c_int(dim),
                              ctypes.c_float(scale), _p(out, _f32p))
    return out


def nqkv_page_payload(key, value, *, page_size: int, q: int, key_betas, value_betas):
    """Six payload streams of one packed page (kv_format.py:71-131).

    key/value: float32 [valid_tokens, Hkv, D] (callers promote BF16 first).
    Returns dict with key_codes, key_betas, key_norms, value_codes, value_betas, value_norms.
    """
    key, value = _f32(key), _f32(value)
    valid, heads, dim = key.shape
    rows = page_size * heads
    result = {}
    for name, tensor, betas in (("key", key, key_betas), ("value", value, value_betas)):
        padded = np.zeros((rows, dim), dtype=np.float32)
        padded[: valid * heads] = tensor.reshape(valid * heads, dim)
        codes, beta_idx, norms = quantize_rows(padded, q, betas)
        result[f"{name}_codes"] = pack_unsigned(codes, 4)
        result[f"{name}_betas"] = pack_unsigned(beta_idx, 2)
        result[f"{name}_norms"] = norms
    return result


def count_div14_mismatches() -> int:
    """Exhaustive float32 check of the kernels' fused three-operation division by 14."""
    fn = lib().nqo_count_div14_mismatches
    fn.restype = ctypes.c_longlong
    return int(fn())


def count_reciprocal_division_mismatches(divisor: float) -> int:
    """Exhaustive float32 check (2^-61 <= |a| < 2^40) of the many-row encoder's division through the reciprocal."""
    fn = lib().nqo_count_reciprocal_division_mismatches
    fn.restype = ctypes.c_longlong
    fn.argtypes = [ctypes.c_float]
    return int(fn(ctypes.c_float(divisor)))


def num_threads() -> int:
    return int(lib().nqo_num_threads())


def set_num_threads(n: int) -> None:
    lib().nqo_set_num_threads(ctypes.c_int(n))


def bf16_round(x) -> np.ndarray:
    """float32 -> nearest-even bfloat16 -> float32 (for the BF16-operand product)."""
    bits = _f32(x).view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return rounded.astype(np.uint32).view(np.float32).reshape(np.shape(x))

