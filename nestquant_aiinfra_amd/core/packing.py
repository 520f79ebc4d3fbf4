"""NQPK v1: fixed-width, LSB-first byte streams of E8 residue codes and beta ids.

Container layout and error behaviour follow nestquant/core/packing.py:18-225:
header ``<4sBBHHQQ`` = magic "NQPK", version 1, ndim, q, beta_count, code bytes, beta
bytes; then ndim little-endian u64 dims; then the two payloads.  Value ``i`` of a flat
stream occupies bits ``[(i % per_byte) * width, +width)`` of byte ``i // per_byte``.
"""

from __future__ import annotations

import math
import struct
from dataclasses import dataclass

import numpy as np
import torch

_HEADER = struct.Struct("<4sBBHHQQ")
_MAGIC = b"NQPK"
_VERSION = 1


class ByteReader:
    """Front-to-back reader over a bytes-like container: every read names what it wants and fails
    with that name when the container is too short; `finish` fails when bytes are left over."""

    def __init__(self, data, *, what: str) -> None:
        self._view, self._at, self._what = memoryview(data).cast("B"), 0, what

    def take(self, count: int, name: str) -> bytes:
        if count < 0 or self._at + count > len(self._view):
            raise ValueError(f"{self._what} is shorter than its {name} ({count} bytes at offset {self._at}, "
                             f"{len(self._view)} in all)")
        piece = bytes(self._view[self._at:self._at + count])
        self._at += count
        return piece

    def unpack(self, layout: struct.Struct, name: str) -> tuple:
        return layout.unpack(self.take(layout.size, name))

    def remaining(self) -> int:
        return len(self._view) - self._at

    def finish(self) -> None:
        if self._at != len(self._view):
            raise ValueError(f"{self._what} has {len(self._view) - self._at} bytes after its last payload: "
                             "stated lengths do not add up to the container size")


def bits_for_cardinality(cardinality: int) -> int:
    if cardinality < 1:
        raise ValueError("cardinality must be positive")
    return max(1, math.ceil(math.log2(cardinality)))


def _ceil_bytes(count: int, width: int) -> int:
    return (count * width + 7) // 8


def _check_cardinalities(q: int, beta_count: int) -> None:
    if q < 2 or q > 256 or beta_count < 1 or beta_count > 256:
        raise ValueError("q must be in [2, 256] and beta_count in [1, 256]")
    if bits_for_cardinality(q) not in (1, 2, 4, 8) or bits_for_cardinality(beta_count) not in (1, 2, 4, 8):
        raise ValueError("packing format supports only 1, 2, 4, or 8 bits per value")


def pack_unsigned(values: np.ndarray, width: int) -> bytes:
    flat = np.ascontiguousarray(values, dtype=np.uint8).reshape(-1)
    per_byte = 8 // width
    padded = np.zeros(_ceil_bytes(flat.size, width) * per_byte, dtype=np.uint8)
    padded[: flat.size] = flat
    lanes = padded.reshape(-1, per_byte).astype(np.uint16)
    shifts = (np.arange(per_byte, dtype=np.uint16) * width)[None, :]
    return np.bitwise_or.reduce(lanes << shifts, axis=1).astype(np.uint8).tobytes()


def unpack_unsigned(payload: bytes, count: int, width: int) -> np.ndarray:
    if len(payload) != _ceil_bytes(count, width):
        raise ValueError("payload size does not match expected packed value count")
    packed = np.frombuffer(payload, dtype=np.uint8)
    per_byte = 8 // width
    remainder = count % per_byte
    if remainder and int(packed[-1]) >> (remainder * width):
        raise ValueError("nonzero padding bits in packed payload")
    shifts = (np.arange(per_byte, dtype=np.uint8) * width)[None, :]
    values = (packed[:, None] >> shifts) & ((1 << width) - 1)
    return values.reshape(-1)[:count].copy()


@dataclass(frozen=True)
class PackedNestQuantIndices:
    """Packed residue and beta-index streams of one quantized tensor."""

    shape: tuple[int, ...]
    q: int
    beta_count: int
    code_payload: bytes
    beta_payload: bytes

    @property
    def code_bit_width(self) -> int:
        return bits_for_cardinality(self.q)

    @property
    def beta_index_bit_width(self) -> int:
        return bits_for_cardinality(self.beta_count)

    @property
    def header_bytes(self) -> int:
        return _HEADER.size + 8 * len(self.shape)

    @property
    def serialized_bytes(self) -> int:
        return self.header_bytes + len(self.code_payload) + len(self.beta_payload)

    def to_bytes(self) -> bytes:
        if len(self.shape) < 2 or len(self.shape) > 255 or any(d < 1 for d in self.shape) or self.shape[-1] != 8:
            raise ValueError("shape must contain 2 to 255 positive dimensions and end in 8")
        _check_cardinalities(self.q, self.beta_count)
        if (len(self.code_payload) != _ceil_bytes(math.prod(self.shape), self.code_bit_width)
                or len(self.beta_payload) != _ceil_bytes(math.prod(self.shape[:-1]), self.beta_index_bit_width)):
            raise ValueError("payload lengths do not match tensor shape and bit widths")
        header = _HEADER.pack(_MAGIC, _VERSION, len(self.shape), self.q, self.beta_count,
                              len(self.code_payload), len(self.beta_payload))
        return header + struct.pack(f"<{len(self.shape)}Q", *self.shape) + self.code_payload + self.beta_payload

    @classmethod
    def from_bytes(cls, data) -> "PackedNestQuantIndices":
        """Parse a container.  The header fixes every size that follows it, so the container is
        taken apart by a reader that refuses to run past the end, and the sizes the header states
        are then compared with the ones the shape implies."""
        reader = ByteReader(data, what="NestQuant packing container")
        magic, version, ndim, q, beta_count, code_bytes, beta_bytes = reader.unpack(_HEADER, "header")
        if magic != _MAGIC:
            raise ValueError(f"invalid NestQuant packing magic {bytes(magic)!r}")
        if version != _VERSION:
            raise ValueError(f"unsupported NestQuant packing version: {version}")
        if ndim < 2:
            raise ValueError("a packed tensor has at least a row axis and the axis of eight block coordinates")
        _check_cardinalities(q, beta_count)
        shape = reader.unpack(struct.Struct(f"<{ndim}Q"), "shape")
        if min(shape) < 1 or shape[-1] != 8:
            raise ValueError(f"shape {tuple(shape)} must be positive and end in the E8 dimension 8")
        stated = {"residue": code_bytes, "beta-index": beta_bytes}
        implied = {"residue": _ceil_bytes(math.prod(shape), bits_for_cardinality(q)),
                   "beta-index": _ceil_bytes(math.prod(shape[:-1]), bits_for_cardinality(beta_count))}
        for stream in stated:
            if stated[stream] != implied[stream]:
                raise ValueError(f"{stream} payload of {stated[stream]} bytes, but shape {tuple(shape)} implies "
                                 f"{implied[stream]}")
        codes, betas = reader.take(code_bytes, "residue payload"), reader.take(beta_bytes, "beta-index payload")
        reader.finish()
        return cls(tuple(shape), q, beta_count, codes, betas)

    def unpack(self, *, device: torch.device | str = "cpu") -> tuple[torch.Tensor, torch.Tensor]:
        """Host-side inspection helper: int64 codes ``shape`` and beta ids ``shape[:-1]``."""
        codes = unpack_unsigned(self.code_payload, math.prod(self.shape), self.code_bit_width)
        betas = unpack_unsigned(self.beta_payload, math.prod(self.shape[:-1]), self.beta_index_bit_width)
        if codes.size and int(codes.max()) >= self.q:
            raise ValueError("decoded residue is outside [0, q)")
        if betas.size and int(betas.max()) >= self.beta_count:
            raise ValueError("decoded beta index is outside [0, beta_count)")
        return (torch.from_numpy(codes.astype(np.int64)).reshape(self.shape).to(device),
                torch.from_numpy(betas.astype(np.int64)).reshape(self.shape[:-1]).to(device))


    def unpack_rows(self, start: int, end: int, *, device: torch.device | str = "cpu"
                    ) -> tuple[torch.Tensor, torch.Tensor]:
        """Rows [start, end) of the leading dimension (nestquant/core/packing.py:108-135): only the
        bytes of those rows are read, also when a row's beta ids begin inside a byte."""
        if any(isinstance(v, bool) or not isinstance(v, int) for v in (start, end)):
            raise TypeError("row bounds must be integers")
        if start < 0 or end < start or end > self.shape[0]:
            raise ValueError("row range is outside packed tensor bounds")
        per_row_codes, per_row_betas = math.prod(self.shape[1:]), math.prod(self.shape[1:-1])
        codes = _unpack_window(self.code_payload, start * per_row_codes, end * per_row_codes, self.code_bit_width)
        betas = _unpack_window(self.beta_payload, start * per_row_betas, end * per_row_betas,
                               self.beta_index_bit_width)
        if codes.size and int(codes.max()) >= self.q:
            raise ValueError("decoded residue is outside [0, q)")
        if betas.size and int(betas.max()) >= self.beta_count:
            raise ValueError("decoded beta index is outside [0, beta_count)")
        rows = end - start
        return (torch.from_numpy(codes.astype(np.int64)).reshape((rows, *self.shape[1:])).to(device),
                torch.from_numpy(betas.astype(np.int64)).reshape((rows, *self.shape[1:-1])).to(device))


def _unpack_window(payload: bytes, first: int, last: int, width: int) -> np.ndarray:
    """Values [first, last) of a fixed-width stream, touching only the bytes that hold them."""
    if first == last:
        return np.empty(0, dtype=np.uint8)
    per_byte = 8 // width
    byte0, byte1 = first // per_byte, -(-last // per_byte)
    window = np.frombuffer(payload, dtype=np.uint8, count=byte1 - byte0, offset=byte0)
    shifts = (np.arange(per_byte, dtype=np.uint8) * width)[None, :]
    values = ((window[:, None] >> shifts) & ((1 << width) - 1)).reshape(-1)
    skip = first - byte0 * per_byte
    return values[skip:skip + (last - first)].copy()


def pack_nestquant_indices(codes: torch.Tensor, beta_indices: torch.Tensor, *, q: int,
                           beta_count: int) -> PackedNestQuantIndices:
    """Pack integer code / beta-id tensors (nestquant/core/packing.py:137-171)."""
    integer = (torch.int8, torch.uint8, torch.int16, torch.int32, torch.int64)
    if not isinstance(codes, torch.Tensor) or codes.dtype not in integer:
        raise TypeError("codes must be an integer torch.Tensor")
    if not isinstance(beta_indices, torch.Tensor) or beta_indices.dtype not in integer:
        raise TypeError("beta_indices must be an integer torch.Tensor")
    if codes.ndim < 2 or codes.shape[-1] != 8:
        raise ValueError("codes must end in E8 dimension 8")
    if tuple(beta_indices.shape) != tuple(codes.shape[:-1]):
        raise ValueError("beta_indices shape must equal codes.shape[:-1]")
    if q < 2 or q > 256:
        raise ValueError("q must be in [2, 256]")
    if beta_count < 1 or beta_count > 256:
        raise ValueError("beta_count must be in [1, 256]")
    code_width, beta_width = bits_for_cardinality(q), bits_for_cardinality(beta_count)
    if code_width not in (1, 2, 4, 8) or beta_width not in (1, 2, 4, 8):
        raise ValueError("this format version supports only bit widths 1, 2, 4, or 8")
    for tensor, cardinality in ((codes, q), (beta_indices, beta_count)):
        if tensor.numel() and (int(tensor.min()) < 0 or int(tensor.max()) >= cardinality):
            raise ValueError(f"all values must be in [0, {cardinality})")
    return PackedNestQuantIndices(
        tuple(codes.shape), q, beta_count,
        pack_unsigned(codes.detach().to(torch.uint8).cpu().numpy(), code_width),
        pack_unsigned(beta_indices.detach().to(torch.uint8).cpu().numpy(), beta_width),
    )
