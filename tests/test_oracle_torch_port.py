"""The torch-vectorised CPU restatement (oracle/torch_port.py, timed by bench.py's cpu_baseline
beside the C restatement) computes what the C restatement computes, element for element; the C
restatement in turn is pinned by the reference's golden vectors (test_oracle_golden.py)."""

import numpy as np
import torch

from conftest import ACTIVATION_BETAS, Q, WEIGHT_BETAS


def test_torch_port_equals_the_c_restatement(oracle, golden):
    from oracle import torch_port

    x = torch.from_numpy(golden["e8_x"].astype(np.float32))
    assert np.array_equal(torch_port.nearest_e8(x).numpy(), golden["e8_point"])

    g = torch.Generator().manual_seed(77)
    rows, n = 24, 512
    matrix = torch.randn(rows, n, generator=g) * torch.logspace(-3, 2, rows).unsqueeze(-1)
    matrix[5] = 0.0                                               # a zero row stays zero
    seed = 20261025
    dither = torch_port.dither_stateless(rows * n // 8, seed)
    assert np.array_equal(dither.numpy(), oracle.dither_stateless(rows * n // 8, seed))
    for betas, d in ((ACTIVATION_BETAS, None), (WEIGHT_BETAS, dither.reshape(rows, n // 8, 8))):
        codes, ids, norms = torch_port.quantize_rows(matrix, Q, betas, d)
        want_codes, want_ids, want_norms = oracle.quantize_rows(matrix.numpy(), Q, betas,
                                                                None if d is None else d.numpy())
        assert np.array_equal(codes.numpy(), want_codes) and np.array_equal(ids.numpy(), want_ids)
        assert np.array_equal(norms.numpy(), want_norms)
        back = torch_port.dequantize_rows(codes, ids, norms, betas, Q, d)
        want_back = oracle.dequantize_rows(want_codes, want_ids, want_norms, betas, Q,
                                           dither=None if d is None else d.numpy())
        assert np.array_equal(back.numpy(), want_back)
        assert not back[5].any()
