"""NQMC v1: model-level container of dense tensors and packed NQRT records, with a
seek-based reader.  Byte layout follows nestquant/core/model_checkpoint.py:26-28, 109-147
and nestquant/core/model_checkpoint_file.py:33-205: header ``<4sBQQ`` = "NQMC", 1,
len(manifest), len(payload); compact JSON manifest {format, version, entries[{name, kind,
offset, length, shape, dtype}], aliases, model_metadata, payload_sha256}; dense entries
sorted by name first, then nestquant entries sorted by name.
"""

from __future__ import annotations

import hashlib
import json
import os
import struct
import tempfile
from dataclasses import dataclass
from pathlib import Path
from typing import Mapping

import torch

from .tensor_checkpoint import PackedNestQuantTensor, _tensor_from_bytes, _tensor_to_bytes

_HEADER = struct.Struct("<4sBQQ")
_MAGIC = b"NQMC"
_VERSION = 1
_DTYPE_TO_NAME = {
    torch.bool: "bool", torch.uint8: "uint8", torch.int8: "int8", torch.int16: "int16",
    torch.int32: "int32", torch.int64: "int64", torch.float16: "float16",
    torch.bfloat16: "bfloat16", torch.float32: "float32", torch.float64: "float64",
}
_NAME_TO_DTYPE = {name: dtype for dtype, name in _DTYPE_TO_NAME.items()}
PAPER_HADAMARD_FORMAT = "local_hadamard_linear_v1"


@dataclass(frozen=True)
class NQMCEntry:
    name: str
    kind: str
    offset: int
    length: int
    shape: tuple[int, ...]
    dtype: torch.dtype


def write_nqmc(path: str | Path, *, dense_tensors: Mapping[str, torch.Tensor],
               quantized_tensors: Mapping[str, PackedNestQuantTensor],
               aliases: Mapping[str, str] | None = None,
               model_metadata: Mapping[str, object] | None = None) -> None:
    """Stream an NQMC file to disk (payload first, then header + manifest, atomically)."""
    destination = Path(path)
    destination.parent.mkdir(parents=True, exist_ok=True)
    aliases = dict(aliases or {})
    if (set(dense_tensors) | set(quantized_tensors)) & set(aliases):
        raise ValueError("alias names cannot also be stored tensor names")
    entries, offset, digest = [], 0, hashlib.sha256()
    with tempfile.NamedTemporaryFile(mode="wb", dir=destination.parent, delete=False) as payload:
        payload_path = Path(payload.name)
        for name in sorted(dense_tensors):
            tensor = dense_tensors[name]
            if tensor.dtype not in _DTYPE_TO_NAME:
                raise ValueError(f"unsupported dense tensor dtype: {name}")
            blob = _tensor_to_bytes(tensor)
            entries.append({"name": name, "kind": "dense", "offset": offset, "length": len(blob),
                            "shape": list(tensor.shape), "dtype": _DTYPE_TO_NAME[tensor.dtype]})
            payload.write(blob); digest.update(blob); offset += len(blob)
        for name in sorted(quantized_tensors):
            record = quantized_tensors[name]
            if record.tensor_name != name:
                raise ValueError(f"quantized record name mismatch: {name}")
            blob = record.to_bytes()
            entries.append({"name": name, "kind": "nestquant", "offset": offset, "length": len(blob),
                            "shape": [record.indices.shape[0], record.feature_count],
                            "dtype": _DTYPE_TO_NAME[record.output_dtype]})
            payload.write(blob); digest.update(blob); offset += len(blob)
    manifest = json.dumps({
        "format": "NQMC", "version": _VERSION, "entries": entries, "aliases": aliases,
        "model_metadata": dict(model_metadata or {}), "payload_sha256": digest.hexdigest(),
    }, ensure_ascii=False, separators=(",", ":")).encode("utf-8")
    try:
        with tempfile.NamedTemporaryFile(mode="wb", dir=destination.parent, delete=False) as out:
            out_path = Path(out.name)
            out.write(_HEADER.pack(_MAGIC, _VERSION, len(manifest), offset))
            out.write(manifest)
            with payload_path.open("rb") as source:
                while block := source.read(8 << 20):
                    out.write(block)
        os.replace(out_path, destination)
    finally:
        payload_path.unlink(missing_ok=True)


class NQMCFileReader:
    """Validated, seek-based reader for an NQMC v1 file."""

    def __init__(self, path: str | Path, *, verify_checksum: bool = True, chunk_bytes: int = 8 << 20):
        self.path = Path(path)
        if chunk_bytes <= 0:
            raise ValueError("chunk_bytes must be positive")
        self.file_bytes = self.path.stat().st_size
        with self.path.open("rb") as stream:
            header = stream.read(_HEADER.size)
            if len(header) != _HEADER.size:
                raise ValueError("input is shorter than the model checkpoint header")
            magic, version, manifest_len, payload_len = _HEADER.unpack(header)
            if magic != _MAGIC:
                raise ValueError("invalid model checkpoint magic")
            if version != _VERSION:
                raise ValueError(f"unsupported model checkpoint version: {version}")
            self.payload_start = _HEADER.size + manifest_len
            self.payload_bytes = payload_len
            if self.payload_start + payload_len != self.file_bytes:
                raise ValueError("model checkpoint lengths do not match file size")
            blob = stream.read(manifest_len)
        try:
            manifest = json.loads(blob.decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as error:
            raise ValueError("invalid model checkpoint manifest") from error
        if manifest.get("format") != "NQMC" or manifest.get("version") != _VERSION:
            raise ValueError("manifest format or version disagrees with the header")
        entries = []
        for item in manifest.get("entries", []):
            if item.get("kind") not in ("dense", "nestquant") or item.get("dtype") not in _NAME_TO_DTYPE:
                raise ValueError("invalid NQMC entry")
            if item["offset"] < 0 or item["offset"] + item["length"] > payload_len:
                raise ValueError("NQMC entry lies outside the payload")
            entries.append(NQMCEntry(item["name"], item["kind"], int(item["offset"]), int(item["length"]),
                                     tuple(int(d) for d in item["shape"]), _NAME_TO_DTYPE[item["dtype"]]))
        self.entries = tuple(entries)
        self.aliases = dict(manifest.get("aliases", {}))
        self.model_metadata = dict(manifest.get("model_metadata", {}))
        self._entries_by_name = {entry.name: entry for entry in self.entries}
        if verify_checksum:
            digest = hashlib.sha256()
            with self.path.open("rb") as stream:
                stream.seek(self.payload_start)
                remaining = payload_len
                while remaining:
                    block = stream.read(min(chunk_bytes, remaining))
                    if not block:
                        raise ValueError("truncated model checkpoint payload")
                    digest.update(block)
                    remaining -= len(block)
            if digest.hexdigest() != manifest.get("payload_sha256"):
                raise ValueError("model checkpoint payload checksum mismatch")

    @property
    def tensor_count(self) -> int:
        return len(self.entries) + len(self.aliases)

    def canonical_name(self, name: str) -> str:
        if name in self._entries_by_name:
            return name
        try:
            return self.aliases[name]
        except KeyError as error:
            raise KeyError(f"tensor is not present in NQMC: {name}") from error

    def get_entry(self, name: str) -> NQMCEntry:
        return self._entries_by_name[self.canonical_name(name)]

    def read_entry_blob(self, entry: NQMCEntry) -> bytes:
        with self.path.open("rb") as stream:
            stream.seek(self.payload_start + entry.offset)
            blob = stream.read(entry.length)
        if len(blob) != entry.length:
            raise ValueError("truncated NQMC record")
        return blob

    def read_entry(self, entry: NQMCEntry):
        blob = self.read_entry_blob(entry)
        if entry.kind == "nestquant":
            return PackedNestQuantTensor.from_bytes(blob)
        return _tensor_from_bytes(blob, entry.shape, entry.dtype)

    def read_named_record(self, name: str):
        entry = self.get_entry(name)
        return entry, self.read_entry(entry)
