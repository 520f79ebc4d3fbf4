"""Containers and constants of the packed formats (nestquant/core/__init__.py for this path)."""

from __future__ import annotations

import importlib

_EXPORTS = {
    "bits_for_cardinality": "packing",
    "pack_unsigned": "packing",
    "unpack_unsigned": "packing",
    "PackedNestQuantIndices": "packing",
    "pack_nestquant_indices": "packing",
    "PackedNestQuantTensor": "tensor_checkpoint",
    "PackedNQKVPage": "kv_format",
    "NQMCEntry": "model_checkpoint",
    "write_nqmc": "model_checkpoint",
    "NQMCFileReader": "model_checkpoint",
    "hadamard": "rotation",
    "signed_hadamard": "rotation",
    "UPSTREAM_CODEC_SEMANTICS": "codec",
    "LEGACY_CODEC_SEMANTICS": "codec",
    "CURRENT_CODEC_SEMANTICS": "codec",
    "STATELESS_DITHER_ALGORITHM": "codec",
    "STATELESS_MODULUS": "codec",
    "E8_DIMENSION": "codec",
}

__all__ = sorted(_EXPORTS)


def __getattr__(name: str):
    # resolved on first use: importing the package does not import torch, transformers or the library
    module = _EXPORTS.get(name)
    if module is None:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
    value = getattr(importlib.import_module(f"{__name__}.{module}"), name)
    globals()[name] = value
    return value


def __dir__():
    return sorted(set(globals()) | set(_EXPORTS))
