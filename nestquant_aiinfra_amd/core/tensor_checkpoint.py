"""NQRT v4: one packed NestQuant weight tensor with stateless-dither metadata.

Byte layout follows nestquant/core/tensor_checkpoint.py:28-31, 124-256: header
``<4sBBIQQQ`` = "NQRT", version, dither mode, len(metadata), len(indices), len(norms),
len(dither); compact JSON metadata (fixed key order, ``separators=(",", ":")``); an NQPK
blob of shape ``(rows, features / 8, 8)``; row norms in ``output_dtype``.

Only what the packed execution path consumes is implemented: dither mode 3 (seed +
``lcg31_mix_v1``) and mode 0 (no dither), versions 2-4.  Records carrying a stored dither
tensor or a generator state (modes 1, 2) or version 1 are rejected: the packed kernels
cannot run them either (nestquant/runtime/triton_fused_linear.py:146-165).
"""

from __future__ import annotations

import json
import struct
from dataclasses import dataclass

import torch

from .codec import (CURRENT_CODEC_SEMANTICS, LEGACY_CODEC_SEMANTICS, STATELESS_DITHER_ALGORITHM,
                    STATELESS_MODULUS, UPSTREAM_CODEC_SEMANTICS)
from .packing import ByteReader, PackedNestQuantIndices

_HEADER = struct.Struct("<4sBBIQQQ")
_MAGIC = b"NQRT"
_VERSION = 4
_DTYPE_TO_NAME = {torch.float16: "float16", torch.bfloat16: "bfloat16",
                  torch.float32: "float32", torch.float64: "float64"}
_NAME_TO_DTYPE = {name: dtype for dtype, name in _DTYPE_TO_NAME.items()}


def _tensor_to_bytes(tensor: torch.Tensor) -> bytes:
    """Raw little-endian bytes of a tensor of any dtype."""
    flat = tensor.detach().cpu().contiguous().reshape(-1)
    if flat.numel() == 0:
        return b""
    return flat.view(torch.uint8).numpy().tobytes()


def _tensor_from_bytes(blob: bytes, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
    if not blob:
        return torch.empty(shape, dtype=dtype)
    return torch.frombuffer(bytearray(blob), dtype=dtype).reshape(shape)


def _validate_stateless(seed, algorithm) -> None:
    if isinstance(seed, bool) or not isinstance(seed, int) or not 0 <= seed < STATELESS_MODULUS:
        raise ValueError("dither_seed must be an integer in [0, 2**31)")
    if algorithm != STATELESS_DITHER_ALGORITHM:
        raise ValueError(f"unsupported stateless dither algorithm: {algorithm}")


def _metadata_fields(blob: bytes) -> dict:
    """The JSON metadata of a record as typed values; anything missing or of the wrong kind is one error."""
    try:
        raw = json.loads(blob.decode("utf-8"))
    except (UnicodeDecodeError, json.JSONDecodeError) as error:
        raise ValueError("invalid tensor checkpoint metadata") from error
    try:
        fields = {"tensor_name": raw["tensor_name"], "rows": int(raw["rows"]), "feature_count": int(raw["feature_count"]),
                  "betas": tuple(float(value) for value in raw["betas"]), "output_dtype": _NAME_TO_DTYPE[raw["output_dtype"]]}
    except (KeyError, TypeError, ValueError, AttributeError) as error:
        raise ValueError("missing or invalid tensor checkpoint metadata fields") from error
    if not isinstance(fields["tensor_name"], str):
        raise ValueError("invalid tensor name")
    for optional in ("q", "beta_count", "dither_seed", "dither_algorithm", "codec_semantics"):
        fields[optional] = raw.get(optional)
    return fields


@dataclass(frozen=True)
class PackedNestQuantTensor:
    """Self-contained serialized data of one quantized matrix tensor."""

    tensor_name: str
    indices: PackedNestQuantIndices
    row_norms: torch.Tensor
    betas: tuple[float, ...]
    feature_count: int
    output_dtype: torch.dtype
    dither: torch.Tensor | None = None
    dither_generator_state: bytes | None = None
    dither_generator_device: str | None = None
    dither_torch_version: str | None = None
    dither_seed: int | None = None
    dither_algorithm: str | None = None
    codec_semantics: str = CURRENT_CODEC_SEMANTICS

    def _validate(self) -> None:
        if not self.tensor_name or not isinstance(self.tensor_name, str):
            raise ValueError("tensor_name must be a nonempty string")
        if self.dither is not None or self.dither_generator_state is not None:
            raise ValueError("only seed-based (stateless) dither is supported by the packed path")
        if self.output_dtype not in _DTYPE_TO_NAME:
            raise ValueError("unsupported row-norm dtype")
        rows = self.indices.shape[0]
        if self.indices.shape != (rows, self.feature_count // 8, 8) or self.feature_count <= 0 or self.feature_count % 8:
            raise ValueError("metadata feature shape disagrees with packed indices")
        if tuple(self.row_norms.shape) != (rows,) or self.row_norms.dtype != self.output_dtype:
            raise ValueError("row norms must be one value per row in output_dtype")
        if len(self.betas) != self.indices.beta_count:
            raise ValueError("beta table length disagrees with packed beta_count")
        if self.codec_semantics not in {UPSTREAM_CODEC_SEMANTICS, LEGACY_CODEC_SEMANTICS}:
            raise ValueError("unsupported tensor checkpoint codec semantics")
        if self.dither_seed is not None:
            _validate_stateless(self.dither_seed, self.dither_algorithm)

    @property
    def serialized_bytes(self) -> int:
        return len(self.to_bytes())

    def to_bytes(self) -> bytes:
        self._validate()
        dither_mode = 3 if self.dither_seed is not None else 0
        metadata = json.dumps({
            "tensor_name": self.tensor_name,
            "q": self.indices.q,
            "beta_count": self.indices.beta_count,
            "betas": list(self.betas),
            "rows": self.indices.shape[0],
            "feature_count": self.feature_count,
            "output_dtype": _DTYPE_TO_NAME[self.output_dtype],
            "dither_generator_device": None,
            "dither_torch_version": None,
            "dither_seed": self.dither_seed,
            "dither_algorithm": self.dither_algorithm,
            "codec_semantics": self.codec_semantics,
        }, ensure_ascii=False, separators=(",", ":")).encode("utf-8")
        indices_blob = self.indices.to_bytes()
        norms_blob = _tensor_to_bytes(self.row_norms)
        header = _HEADER.pack(_MAGIC, _VERSION, dither_mode, len(metadata), len(indices_blob),
                              len(norms_blob), 0)
        return header + metadata + indices_blob + norms_blob

    @classmethod
    def from_bytes(cls, data) -> "PackedNestQuantTensor":
        """Parse an NQRT record (versions 2 to 4).  Only the payload-free dither modes reach the
        packed path: none (0) and the stateless counter hash (3)."""
        # magic and version sit in the first five bytes of every version: they are judged before the rest
        prefix = bytes(memoryview(data).cast("B")[:5])
        if len(prefix) < 5:
            raise ValueError("input is shorter than the tensor checkpoint header")
        magic, version = struct.unpack("<4sB", prefix)
        if magic != _MAGIC:
            raise ValueError("invalid tensor checkpoint magic")
        if version not in (2, 3, 4):
            raise ValueError(f"unsupported tensor checkpoint version: {version}")
        reader = ByteReader(data, what="tensor checkpoint")
        _, _, dither_mode, *lengths = reader.unpack(_HEADER, "header")
        if dither_mode in (1, 2):
            raise ValueError("stored-dither and generator-state records are not supported by the packed path")
        if dither_mode not in (0, 3):
            raise ValueError(f"invalid dither storage mode {dither_mode}")
        metadata_bytes, indices_bytes, norms_bytes, dither_bytes = lengths
        if metadata_bytes + indices_bytes + norms_bytes + dither_bytes != reader.remaining():
            raise ValueError("tensor checkpoint payload lengths do not match file size")
        if dither_bytes:
            raise ValueError("a record whose dither is regenerated carries no dither payload")
        fields = _metadata_fields(reader.take(metadata_bytes, "metadata"))
        indices = PackedNestQuantIndices.from_bytes(reader.take(indices_bytes, "index container"))
        norms_blob = reader.take(norms_bytes, "row norms")
        reader.finish()

        rows, features, dtype = fields["rows"], fields["feature_count"], fields["output_dtype"]
        if (fields["q"], fields["beta_count"]) != (indices.q, indices.beta_count):
            raise ValueError("metadata disagrees with packed index parameters")
        if features <= 0 or features % 8 or indices.shape != (rows, features // 8, 8):
            raise ValueError(f"metadata says {rows} rows of {features} features, the index container holds "
                             f"shape {indices.shape}")
        if len(norms_blob) != rows * torch.empty((), dtype=dtype).element_size():
            raise ValueError("row norm payload size disagrees with metadata")
        seed = algorithm = None
        if dither_mode == 3:
            if version < 4:
                raise ValueError("stateless dither requires NQRT v4")
            seed, algorithm = fields["dither_seed"], fields["dither_algorithm"]
            _validate_stateless(seed, algorithm)
        record = cls(tensor_name=fields["tensor_name"], indices=indices,
                     row_norms=_tensor_from_bytes(norms_blob, (rows,), dtype), betas=fields["betas"],
                     feature_count=features, output_dtype=dtype, dither_seed=seed, dither_algorithm=algorithm,
                     codec_semantics=fields["codec_semantics"] if version >= 3 else LEGACY_CODEC_SEMANTICS)
        record._validate()
        return record

    def dequantize(self, *, device: torch.device | str = "cuda") -> torch.Tensor:
        """Float32 reconstruction on the GPU (QuantizedRows.dequantize semantics)."""
        from ..runtime.w4a4_linear import dequantize_record
        return dequantize_record(self, device=device)
