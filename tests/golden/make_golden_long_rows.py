"""Writes reference_long_rows.npz: the reference's CPU `quantize_rows` on rows of 8192 and
4096 features (the down_proj activation width), so that the row-norm and scaling arithmetic
of the oracle is pinned beyond the 2048-feature rows of reference_vectors.npz.

Run once, in the build container only (the reference checkout is not available anywhere else):

    python tests/golden/make_golden_long_rows.py [/path/to/reference]

Outputs are data only: seeded inputs (stored as BF16 bit patterns, the activation dtype) and the
reference's codes, beta indices and row norms for them.
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
REFERENCE = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
sys.path.insert(0, str(REFERENCE))

from nestquant.core.quantizer import quantize_rows  # noqa: E402
from nestquant.core.rotation import signed_hadamard  # noqa: E402

Q = 14
ACTIVATION_BETAS = tuple(value / 14 for value in (3.47, 4.74, 6.90, 18.11))


def main() -> None:
    out = {}
    for name, rows, n, seed in (("qr8192", 3, 8192, 301), ("qr4096", 2, 4096, 302)):
        g = torch.Generator().manual_seed(seed)
        x0 = torch.randn(rows, n, generator=g)
        x0[:, torch.randperm(n, generator=g)[: n // 100]] *= 20.0        # outlier channels, as in activations
        signs = (2 * torch.randint(0, 2, (n,), generator=g) - 1).float()
        xr = signed_hadamard(x0, signs).to(torch.bfloat16)
        result = quantize_rows(xr.float(), Q, ACTIVATION_BETAS)
        out[f"{name}_x_bf16"] = xr.view(torch.int16).numpy()
        out[f"{name}_codes"] = result.codes.numpy().astype(np.uint8)
        out[f"{name}_beta"] = result.beta_indices.numpy().astype(np.uint8)
        out[f"{name}_norms"] = result.row_norms.numpy()
    np.savez_compressed(HERE / "reference_long_rows.npz", **out)
    print({k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
