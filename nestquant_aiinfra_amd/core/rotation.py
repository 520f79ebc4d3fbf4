"""Normalized Sylvester-Hadamard transform along the last axis
(nestquant/core/rotation.py:12-36): butterflies of growing width in the input dtype, then
one division by sqrt(n).  Plain tensor ops: used for weight preparation and tests; the
decode path rotates inside the HIP kernels."""

import math

import torch


def hadamard(x: torch.Tensor) -> torch.Tensor:
    if x.ndim == 0 or not x.is_floating_point():
        raise ValueError("expected a floating-point tensor with a feature axis")
    n = x.shape[-1]
    if n < 1 or n & (n - 1):
        raise ValueError("feature dimension must be a positive power of two")
    y = x.reshape(-1, n)
    width = 1
    while width < n:
        pairs = y.reshape(-1, n // (2 * width), 2, width)
        left, right = pairs[:, :, 0], pairs[:, :, 1]
        y = torch.stack((left + right, left - right), dim=2).reshape(-1, n)
        width *= 2
    return (y / math.sqrt(n)).reshape(x.shape)


def signed_hadamard(x: torch.Tensor, signs: torch.Tensor, *, inverse: bool = False) -> torch.Tensor:
    if x.ndim == 0 or signs.ndim != 1 or signs.shape[0] != x.shape[-1]:
        raise ValueError("signs must be a vector matching the feature dimension")
    return hadamard(x) * signs if inverse else hadamard(x * signs)
