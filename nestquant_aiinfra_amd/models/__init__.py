"""The fused Linear module, model conversion and the 1B runner assembly."""

from __future__ import annotations

import importlib

_EXPORTS = {
    "SharedHadamardCache": "fused_linear",
    "SharedPackedActivationCache": "fused_linear",
    "FusedNQRTLinear": "fused_linear",
    "FusedNQRTConversionReport": "fused_linear",
    "convert_linears_to_fused_nqrt_": "fused_linear",
    "projection_names": "llama_w4a4kv4",
    "write_w4_checkpoint": "llama_w4a4kv4",
    "build_w4a4kv4_runner": "llama_w4a4kv4",
    "attach_w4a4kv4_cache": "llama_w4a4kv4",
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
