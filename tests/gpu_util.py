"""Helpers for the GPU parity tests: seeded inputs and oracle-side references."""

from __future__ import annotations

import numpy as np
import torch

from conftest import ACTIVATION_BETAS, Q, WEIGHT_BETAS


def bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().numpy()


def student_t_rows(rows: int, n: int, seed: int) -> torch.Tensor:
    """Heavy-tailed activations, Student-t with 4 degrees of freedom per entry."""
    rng = np.random.default_rng(seed)
    return torch.from_numpy(rng.standard_t(4, size=(rows, n)).astype(np.float32))


def outlier_rows(rows: int, n: int, seed: int) -> torch.Tensor:
    """N(0, 1) with 1 % of the channels scaled to 20 sigma."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, n)).astype(np.float32)
    channels = rng.choice(n, size=max(1, n // 100), replace=False)
    x[:, channels] *= 20.0
    return torch.from_numpy(x)


def oracle_weight(oracle, n_out: int, k: int, seed: int, dither_seed: int):
    """Hadamard-rotated N(0, 0.02) weight quantized by the oracle -> packed streams."""
    rng = np.random.default_rng(seed)
    w = oracle.hadamard((0.02 * rng.standard_normal((n_out, k))).astype(np.float32))
    dither = oracle.dither_stateless(n_out * k // 8, dither_seed).reshape(n_out, k // 8, 8)
    codes, beta, norms = oracle.quantize_rows(w, Q, WEIGHT_BETAS, dither=dither)
    return w, codes, beta, norms


def relative_error(actual: np.ndarray, expected: np.ndarray) -> float:
    """max |actual - expected| / max |expected| (the tolerance the parity bar is stated in)."""
    scale = float(np.abs(expected).max())
    return float(np.abs(actual.astype(np.float64) - expected.astype(np.float64)).max() / max(scale, 1e-30))
