"""Normalized Sylvester-Hadamard transform along the last axis, with the reference's rounding
(nestquant/core/rotation.py:12-36): log2(n) stages of sums and differences at distances
1, 2, 4, ..., each rounded to the input dtype, then one division by sqrt(n).

Tensors on the GPU go through the library's kernel (nq_hadamard, one launch, bit-equal to the
staged form); tensors on the host take the staged form below.  Used for weight preparation and
tests: the decode path rotates inside the encoder, writer and attention kernels."""

from __future__ import annotations

import math

import torch

_KERNEL_DTYPES = (torch.float32, torch.bfloat16, torch.float16)
_KERNEL_MAX_FEATURES = 32768


def _feature_count(x: torch.Tensor) -> int:
    if not isinstance(x, torch.Tensor) or x.ndim == 0 or not x.is_floating_point():
        raise ValueError("expected a floating-point tensor with a feature axis")
    n = x.shape[-1]
    if n < 1 or n & (n - 1):
        raise ValueError("feature dimension must be a positive power of two")
    return n


def _staged(rows: torch.Tensor, n: int) -> torch.Tensor:
    """The butterfly network on [count, n]: stage of distance d pairs element i with i + d inside
    blocks of 2 d, sums to the lower half of the block and differences to the upper half."""
    distance = 1
    while distance < n:
        blocks = rows.view(rows.shape[0], n // (2 * distance), 2 * distance)
        lower, upper = blocks[..., :distance], blocks[..., distance:]
        rows = torch.cat((lower + upper, lower - upper), dim=-1).view(rows.shape[0], n)
        distance *= 2
    return rows / math.sqrt(n)


def hadamard(x: torch.Tensor) -> torch.Tensor:
    n = _feature_count(x)
    if x.is_cuda and x.dtype in _KERNEL_DTYPES and 2 <= n <= _KERNEL_MAX_FEATURES and x.numel():
        from ..runtime.w4a4_linear import hadamard_cuda
        return hadamard_cuda(x.contiguous())
    return _staged(x.reshape(-1, n).contiguous(), n).reshape(x.shape)


def signed_hadamard(x: torch.Tensor, signs: torch.Tensor, *, inverse: bool = False) -> torch.Tensor:
    """x D H for a diagonal D of signs, or its inverse y H D."""
    n = _feature_count(x)
    if not isinstance(signs, torch.Tensor) or tuple(signs.shape) != (n,):
        raise ValueError("signs must be a vector matching the feature dimension")
    if signs.device != x.device or not bool((signs.abs() == 1).all()):
        raise ValueError("signs must contain +/-1 on the input device")
    return hadamard(x) * signs if inverse else hadamard(x * signs)
