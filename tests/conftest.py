"""Shared fixtures.  `gpu` marks tests that need a real MI355X."""

from __future__ import annotations

import json
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN_DIR = Path(__file__).resolve().parent / "golden"

Q = 14
ACTIVATION_BETAS = tuple(v / 14 for v in (3.47, 4.74, 6.90, 18.11))
WEIGHT_BETAS = tuple(v / 14 for v in (4.0, 5.5, 7.0, 18.0))
KEY_BETAS = tuple(v / 14 for v in (3.50, 4.58, 6.47, 17.06))
VALUE_BETAS = tuple(v / 14 for v in (3.53, 5.59, 9.62, 29.03))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    """Vectors written by tests/golden/make_golden.py from the reference's CPU core."""
    with np.load(GOLDEN_DIR / "reference_vectors.npz") as data:
        return {name: data[name] for name in data.files}


@pytest.fixture(scope="session")
def golden_long_rows():
    """Rows of 8192 and 4096 features through the reference's quantize_rows
    (tests/golden/make_golden_long_rows.py); inputs are BF16 bit patterns."""
    with np.load(GOLDEN_DIR / "reference_long_rows.npz") as data:
        return {name: data[name] for name in data.files}


@pytest.fixture(scope="session")
def golden_meta():
    return json.loads((GOLDEN_DIR / "reference_vectors.json").read_text())


@pytest.fixture(scope="session")
def oracle():
    import oracle as module
    module.build()
    return module
