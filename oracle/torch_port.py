"""Test infrastructure, not product code: the reference's CPU codec path restated with whole-tensor
torch operations on the CPU, the way the reference itself evaluates it (one encode + decode pass
over the full tensor per beta, then an argmin over the passes).  It exists for two things only:
the `cpu_baseline` leg of bench.py times it beside the C restatement, and the CPU tests check it
element for element against the C restatement (which the reference's golden vectors pin), so both
CPU baselines compute the same codes.  Nothing in the product path may import this module.

Reference, function by function:
  nearest_e8        nestquant/core/lattice.py:18-81   (round, parity repair, two cosets, ties to the half coset)
  encode / decode   nestquant/core/codec.py:53-142    (coordinates mod q; coset point, reduce by q * nearest)
  dither_stateless  nestquant/core/codec.py:176-224   (lcg31_mix_v1 on counters, fold into the Voronoi cell)
  quantize_rows     nestquant/core/quantizer.py:214-301
  dequantize_rows   nestquant/core/quantizer.py:39-51
"""

from __future__ import annotations

import math

import torch

_MASK31 = (1 << 31) - 1


def _nearest_d8(points: torch.Tensor) -> torch.Tensor:
    nearest = points.round()
    residual = points - nearest
    odd = nearest.sum(dim=-1, keepdim=True).remainder(2) != 0
    worst = residual.abs().argmax(dim=-1, keepdim=True)                 # first index on ties
    toward = torch.where(residual.gather(-1, worst) >= 0, 1.0, -1.0).to(points.dtype)
    return nearest.scatter_add(-1, worst, toward * odd.to(points.dtype))


def nearest_e8(x: torch.Tensor) -> torch.Tensor:
    whole = _nearest_d8(x)
    halves = _nearest_d8(x - 0.5) + 0.5
    whole_error = (x - whole).square().sum(dim=-1)
    halves_error = (x - halves).square().sum(dim=-1)
    return torch.where((whole_error < halves_error).unsqueeze(-1), whole, halves)


def _coordinates(point: torch.Tensor) -> torch.Tensor:
    """Integer generator coordinates of lattice points (the triangular solve, exact in float32)."""
    last = point[..., 7]
    c = [None] * 8
    c[7] = 2.0 * last
    c[6] = point[..., 6] - last
    for j in range(5, 0, -1):
        c[j] = point[..., j] + c[j + 1] - last
    c[0] = 0.5 * (point[..., 0] + c[1] - last)
    return torch.stack(c, dim=-1).round().to(torch.int64)


def _coset_point(code: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    f = code.to(dtype)
    half = 0.5 * f[..., 7:8]
    head = 2.0 * f[..., 0:1] - f[..., 1:2] + half
    middle = f[..., 1:6] - f[..., 2:7] + half
    return torch.cat((head, middle, f[..., 6:7] + half, half), dim=-1)


def encode_nested(x: torch.Tensor, q: int, dither: torch.Tensor | None = None) -> torch.Tensor:
    shifted = x if dither is None else x + dither
    return _coordinates(nearest_e8(shifted)).remainder(q)


def decode_nested(code: torch.Tensor, q: int, dither: torch.Tensor | None = None,
                  dtype: torch.dtype = torch.float32) -> torch.Tensor:
    point = _coset_point(code, dtype)
    if dither is not None:
        point = point - dither
    return point - q * nearest_e8(point / q)


def dither_stateless(count: int, seed: int, block_offset: int = 0) -> torch.Tensor:
    counters = torch.arange(block_offset * 8, (block_offset + count) * 8, dtype=torch.int64)
    v = (counters + seed) & _MASK31
    v = v ^ (v >> 16)
    v = (v * 1103515245 + 12345) & _MASK31
    v = v ^ (v >> 13)
    v = (v * 134775813 + 1) & _MASK31
    v = v ^ (v >> 16)
    uniform = (v.to(torch.float32) * (2.0 / 2 ** 31)).reshape(count, 8)
    return uniform - nearest_e8(uniform)


def quantize_rows(x: torch.Tensor, q: int, betas, dither: torch.Tensor | None = None):
    """[rows, n] float32 -> (codes int64 [rows, n/8, 8], beta ids int64 [rows, n/8], norms [rows])."""
    rows, n = x.shape
    norms = torch.linalg.vector_norm(x, ord=2, dim=-1)
    live = norms > 0
    scale = math.sqrt(n) / torch.where(live, norms, torch.ones_like(norms))
    blocks = torch.where(live.unsqueeze(-1), x * scale.unsqueeze(-1), torch.zeros_like(x)).reshape(rows, n // 8, 8)
    passes, errors = [], []
    for beta in betas:                                   # one full-tensor encode + decode per beta
        code = encode_nested(blocks / beta, q, dither)
        passes.append(code)
        errors.append((decode_nested(code, q, dither, x.dtype) * beta - blocks).square().sum(dim=-1))
    best = torch.stack(errors).argmin(dim=0)             # first minimum wins
    picked = torch.stack(passes).gather(0, best[None, :, :, None].expand(1, rows, n // 8, 8))[0]
    return picked, best, norms


def dequantize_rows(codes: torch.Tensor, beta_ids: torch.Tensor, norms: torch.Tensor, betas, q: int,
                    dither: torch.Tensor | None = None) -> torch.Tensor:
    rows, blocks, _ = codes.shape
    table = torch.tensor(tuple(betas), dtype=torch.float32)
    decoded = decode_nested(codes, q, dither) * table[beta_ids].unsqueeze(-1)
    return decoded.reshape(rows, blocks * 8) * (norms / math.sqrt(blocks * 8)).unsqueeze(-1)
