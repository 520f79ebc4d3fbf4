"""NQKV page container: the on-disk / on-wire form of one packed Key/Value page.

Byte-compatible with the reference's `PackedNQKVPage` (nestquant/core/kv_format.py:48-336):

    header   "<4sBBBBHHHHHHH[H]IIII"  magic "NQKV", version (1: one beta table, 2: separate key
             and value tables), layout (1 = NHD), norm dtype (1 = float32), output dtype id,
             codec id (1 = upstream E8), page_size, valid_tokens, kv heads, head_dim, q,
             key beta count, [value beta count, version 2 only], then the byte lengths of the
             key index container, key norms, value index container, value norms
    body     key betas (float32), [value betas], key indices (a PackedNestQuantIndices
             container of shape [page_size * heads, head_dim / 8, 8]), key norms (float32),
             value indices, value norms
    trailer  SHA-256 of everything before it

The page itself is always encoded and decoded on the GPU (`quantize_nqkv_page_cuda`,
`dequantize_nqkv_page`); this module only moves the six streams between device tensors and bytes.
"""

from __future__ import annotations

import hashlib
import math
import struct
from dataclasses import dataclass
from typing import Sequence

import numpy as np
import torch

from .codec import UPSTREAM_CODEC_SEMANTICS
from .packing import PackedNestQuantIndices, bits_for_cardinality

MAGIC = b"NQKV"
DIGEST_BYTES = 32
_FIXED = "<4sBBBBHHHHHH"                    # up to and including q
_LAYOUTS = {1: struct.Struct(_FIXED + "H" + "IIII"), 2: struct.Struct(_FIXED + "HH" + "IIII")}
_DTYPE_IDS = {torch.bfloat16: 1, torch.float16: 2, torch.float32: 3, torch.float64: 4}
_DTYPES = {number: dtype for dtype, number in _DTYPE_IDS.items()}


def _beta_tuple(betas: Sequence[float]) -> tuple[float, ...]:
    try:
        values = tuple(float(b) for b in betas)
    except (TypeError, ValueError) as error:
        raise TypeError("betas must be a nonempty sequence of numbers") from error
    if not values or any(not math.isfinite(b) or b <= 0 for b in values):
        raise ValueError("betas must contain positive finite values")
    return values


def _norm_vector(blob: bytes) -> torch.Tensor:
    return torch.from_numpy(np.frombuffer(blob, dtype="<f4").copy())


@dataclass(frozen=True)
class PackedNQKVPage:
    """One fixed-capacity packed K/V page in NHD layout, held as host bytes.  The index streams
    always cover the whole physical page (rows after `valid_tokens` are encoded zeros)."""

    page_size: int
    valid_tokens: int
    num_kv_heads: int
    head_dim: int
    q: int
    betas: tuple[float, ...]
    output_dtype: torch.dtype
    key_indices: PackedNestQuantIndices
    key_norms: torch.Tensor
    value_indices: PackedNestQuantIndices
    value_norms: torch.Tensor
    codec_semantics: str = UPSTREAM_CODEC_SEMANTICS
    value_betas: tuple[float, ...] | None = None

    # -- construction --------------------------------------------------------------------------
    @classmethod
    def from_tensors(cls, key: torch.Tensor, value: torch.Tensor, *, page_size: int, q: int,
                     betas: Sequence[float] | None = None, key_betas: Sequence[float] | None = None,
                     value_betas: Sequence[float] | None = None) -> "PackedNQKVPage":
        """Encode an NHD prefix [tokens, kv_heads, head_dim] (on the GPU) into a page.  `betas`
        gives the one-table form (version 1), `key_betas` + `value_betas` version 2."""
        from ..runtime.nqkv import quantize_nqkv_page_cuda
        if betas is not None and (key_betas is not None or value_betas is not None):
            raise ValueError("pass legacy betas or key_betas/value_betas, not both")
        if betas is None and (key_betas is None or value_betas is None):
            raise ValueError("v2 requires both key_betas and value_betas")
        if betas is not None:
            prepared = quantize_nqkv_page_cuda(key, value, page_size=page_size, q=q, betas=_beta_tuple(betas))
            return cls.from_prepared(prepared, betas=betas)
        prepared = quantize_nqkv_page_cuda(key, value, page_size=page_size, q=q, key_betas=_beta_tuple(key_betas),
                                           value_betas=_beta_tuple(value_betas))
        return cls.from_prepared(prepared, key_betas=key_betas, value_betas=value_betas)

    @classmethod
    def from_prepared(cls, page, *, betas: Sequence[float] | None = None, key_betas: Sequence[float] | None = None,
                      value_betas: Sequence[float] | None = None) -> "PackedNQKVPage":
        """Copy a device-resident PreparedNQKVPage to the host.  The beta tables are taken from the
        arguments (exact Python floats, as the reference stores them) or, when none is given, from
        the page's float32 tables (version 2)."""
        if betas is not None:
            key_table, value_table = _beta_tuple(betas), None
        elif key_betas is not None and value_betas is not None:
            key_table, value_table = _beta_tuple(key_betas), _beta_tuple(value_betas)
        else:
            key_table = tuple(float(b) for b in page.key_beta_table.cpu().tolist())
            value_table = tuple(float(b) for b in page.value_beta_table.cpu().tolist())
        shape = (page.page_size * page.num_kv_heads, page.head_dim // 8, 8)

        def indices(codes, ids, count):
            return PackedNestQuantIndices(shape, page.q, count, codes.cpu().numpy().tobytes(),
                                          ids.cpu().numpy().tobytes())
        return cls(page.page_size, page.valid_tokens, page.num_kv_heads, page.head_dim, page.q, key_table,
                   page.output_dtype, indices(page.key_code_payload, page.key_beta_payload, len(key_table)),
                   page.key_norms.detach().float().cpu().contiguous(),
                   indices(page.value_code_payload, page.value_beta_payload,
                           len(key_table if value_table is None else value_table)),
                   page.value_norms.detach().float().cpu().contiguous(), UPSTREAM_CODEC_SEMANTICS, value_table)

    def to_prepared(self, device: torch.device | str = "cuda"):
        """The page as device tensors, ready for `NQKVPagePool.store_prepared` or
        `dequantize_nqkv_page`."""
        from ..runtime.nqkv import PreparedNQKVPage
        self._validate()
        target = torch.device(device)

        def stream(blob):
            return torch.from_numpy(np.frombuffer(blob, dtype=np.uint8).copy()).to(target)
        return PreparedNQKVPage(
            stream(self.key_indices.code_payload), stream(self.key_indices.beta_payload), self.key_norms.to(target),
            stream(self.value_indices.code_payload), stream(self.value_indices.beta_payload),
            self.value_norms.to(target), torch.tensor(self.betas, dtype=torch.float32, device=target),
            torch.tensor(self.resolved_value_betas, dtype=torch.float32, device=target), self.page_size,
            self.valid_tokens, self.num_kv_heads, self.head_dim, self.q, bits_for_cardinality(self.q),
            bits_for_cardinality(len(self.betas)), self.output_dtype)

    # -- accounting ----------------------------------------------------------------------------
    @property
    def format_version(self) -> int:
        return 1 if self.value_betas is None else 2

    @property
    def resolved_value_betas(self) -> tuple[float, ...]:
        return self.betas if self.value_betas is None else self.value_betas

    @property
    def physical_rows(self) -> int:
        return self.page_size * self.num_kv_heads

    @property
    def payload_bytes(self) -> int:
        """Bytes of the six streams, without container metadata."""
        return sum(len(i.code_payload) + len(i.beta_payload) for i in (self.key_indices, self.value_indices)) + 4 * (
            self.key_norms.numel() + self.value_norms.numel())

    @property
    def serialized_bytes(self) -> int:
        return len(self.to_bytes())

    def storage_report(self) -> dict[str, int | float | str]:
        entries = 2 * self.physical_rows * self.head_dim
        pair = (self.key_indices, self.value_indices)
        return {
            "format": f"NQKV-v{self.format_version}", "layout": "NHD", "page_size": self.page_size,
            "valid_tokens": self.valid_tokens, "physical_entries": entries,
            "code_bytes": sum(len(i.code_payload) for i in pair), "beta_bytes": sum(len(i.beta_payload) for i in pair),
            "norm_bytes": 4 * (self.key_norms.numel() + self.value_norms.numel()),
            "payload_bytes": self.payload_bytes, "container_bytes": self.serialized_bytes,
            "payload_bits_per_entry": self.payload_bytes * 8 / entries,
        }

    # -- decode --------------------------------------------------------------------------------
    def dequantize(self, *, device: torch.device | str = "cuda",
                   output_dtype: torch.dtype | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        """The valid NHD prefix of keys and values, decoded on the GPU."""
        from ..runtime.nqkv import dequantize_nqkv_page
        dtype = self.output_dtype if output_dtype is None else output_dtype
        if dtype not in _DTYPE_IDS:
            raise TypeError("output_dtype must be bfloat16, float16, float32, or float64")
        kernel_dtype = torch.float32 if dtype == torch.float64 else dtype
        key, value = dequantize_nqkv_page(self.to_prepared(device), output_dtype=kernel_dtype)
        return key.to(dtype), value.to(dtype)

    # -- bytes ---------------------------------------------------------------------------------
    def to_bytes(self) -> bytes:
        self._validate()
        version = self.format_version
        tables = [self.betas] + ([self.resolved_value_betas] if version == 2 else [])
        parts = [struct.pack(f"<{len(t)}f", *t) for t in tables]
        streams = [self.key_indices.to_bytes(), self.key_norms.numpy().astype("<f4").tobytes(),
                   self.value_indices.to_bytes(), self.value_norms.numpy().astype("<f4").tobytes()]
        counts = [len(t) for t in tables]
        header = _LAYOUTS[version].pack(MAGIC, version, 1, 1, _DTYPE_IDS[self.output_dtype], 1, self.page_size,
                                        self.valid_tokens, self.num_kv_heads, self.head_dim, self.q, *counts,
                                        *(len(s) for s in streams))
        body = b"".join([header, *parts, *streams])
        return body + hashlib.sha256(body).digest()

    @classmethod
    def from_bytes(cls, data) -> "PackedNQKVPage":
        view = memoryview(data)
        if len(view) < _LAYOUTS[1].size + DIGEST_BYTES:
            raise ValueError("input is shorter than the NQKV header and checksum")
        magic, version = struct.unpack_from("<4sB", view)
        if magic != MAGIC:
            raise ValueError("invalid NQKV magic")
        if version not in _LAYOUTS:
            raise ValueError(f"unsupported NQKV version: {version}")
        layout = _LAYOUTS[version]
        if len(view) < layout.size + DIGEST_BYTES:
            raise ValueError("input is shorter than the NQKV header and checksum")
        fields = layout.unpack_from(view)
        (_, _, order, norm_id, dtype_id, codec_id, page_size, valid_tokens, heads, head_dim, q) = fields[:11]
        table_counts, lengths = fields[11:-4], fields[-4:]
        for found, wanted, what in ((order, 1, "layout"), (norm_id, 1, "norm dtype"), (codec_id, 1, "codec semantics")):
            if found != wanted:
                raise ValueError(f"unsupported NQKV {what}")
        if dtype_id not in _DTYPES:
            raise ValueError("unsupported NQKV output dtype")
        if len(view) != layout.size + 4 * sum(table_counts) + sum(lengths) + DIGEST_BYTES:
            raise ValueError("NQKV payload lengths do not match the container size")
        if hashlib.sha256(view[:-DIGEST_BYTES]).digest() != bytes(view[-DIGEST_BYTES:]):
            raise ValueError("NQKV checksum mismatch")
        cursor = layout.size
        tables = []
        for count in table_counts:
            tables.append(tuple(float(b) for b in struct.unpack_from(f"<{count}f", view, cursor)))
            cursor += 4 * count
        blobs = []
        for length in lengths:
            blobs.append(bytes(view[cursor:cursor + length]))
            cursor += length
        page = cls(page_size, valid_tokens, heads, head_dim, q, tables[0], _DTYPES[dtype_id],
                   PackedNestQuantIndices.from_bytes(blobs[0]), _norm_vector(blobs[1]),
                   PackedNestQuantIndices.from_bytes(blobs[2]), _norm_vector(blobs[3]), UPSTREAM_CODEC_SEMANTICS,
                   tables[1] if version == 2 else None)
        page._validate()
        return page

    # -- validation ----------------------------------------------------------------------------
    def _validate(self) -> None:
        if self.codec_semantics != UPSTREAM_CODEC_SEMANTICS:
            raise ValueError("NQKV requires upstream E8 codec semantics")
        if self.output_dtype not in _DTYPE_IDS:
            raise TypeError("unsupported NQKV output dtype")
        if not 1 <= self.valid_tokens <= self.page_size <= 65535:
            raise ValueError("valid_tokens must be in [1, page_size]")
        if not 1 <= self.num_kv_heads <= 65535:
            raise ValueError("num_kv_heads must be in [1, 65535]")
        if not 1 <= self.head_dim <= 65535 or self.head_dim % 8:
            raise ValueError("head_dim must be positive and divisible by 8")
        key_table, value_table = _beta_tuple(self.betas), _beta_tuple(self.resolved_value_betas)
        if max(len(key_table), len(value_table)) > 65535:
            raise ValueError("NQKV supports at most 65535 beta values per table")
        shape = (self.physical_rows, self.head_dim // 8, 8)
        for name, indices, norms, table in (("key", self.key_indices, self.key_norms, key_table),
                                            ("value", self.value_indices, self.value_norms, value_table)):
            if tuple(indices.shape) != shape:
                raise ValueError(f"{name} packed shape disagrees with page metadata")
            if indices.q != self.q or indices.beta_count != len(table):
                raise ValueError(f"{name} packing parameters disagree with page metadata")
            if (tuple(norms.shape) != (self.physical_rows,) or norms.dtype != torch.float32
                    or norms.device.type != "cpu"):
                raise ValueError(f"{name} norms must be a contiguous CPU float32 vector")
            if not norms.is_contiguous() or not bool(torch.isfinite(norms).all()):
                raise ValueError(f"{name} norms must be contiguous and finite")
