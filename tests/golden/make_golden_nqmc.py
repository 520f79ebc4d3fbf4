"""Writes reference_nqmc.bin: a small NQMC v1 model container produced by the reference's
own writer, so that the container reader / writer of this package is pinned to its bytes.

Run once, in the build container only (the reference checkout is not available anywhere else):

    python tests/golden/make_golden_nqmc.py [/path/to/reference]

Content (all seeded or taken from reference_vectors.npz): a BF16 dense tensor, an int64 dense
tensor, the 32 x 128 NQRT4 record of reference_vectors.npz, one alias of the dense tensor and a
metadata block.  Output is data only.
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
REFERENCE = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
sys.path.insert(0, str(REFERENCE))

from nestquant.core.model_checkpoint import PackedNestQuantModel  # noqa: E402
from nestquant.core.tensor_checkpoint import PackedNestQuantTensor  # noqa: E402


def main() -> None:
    vectors = np.load(HERE / "reference_vectors.npz")
    record = PackedNestQuantTensor.from_bytes(vectors["nqrt_bytes"].tobytes())
    g = torch.Generator().manual_seed(20261201)
    embed = torch.randn(6, 16, generator=g).to(torch.bfloat16)
    state = {
        "model.embed_tokens.weight": embed,
        "lm_head.weight": embed,                                        # tied: becomes an alias
        "model.layers.0.position_ids": torch.arange(5, dtype=torch.int64),
        record.tensor_name: torch.zeros(record.indices.shape[0], record.feature_count),
    }
    model = PackedNestQuantModel.from_state_dict(
        state, {record.tensor_name: record},
        model_metadata={"hadamard_rotation": {"format": "local_hadamard_linear_v1",
                                              "converted_linear_names": [record.tensor_name.rsplit(".", 1)[0]]},
                        "note": "golden"})
    blob = model.to_bytes()
    assert PackedNestQuantModel.from_bytes(blob).aliases == {"lm_head.weight": "model.embed_tokens.weight"}
    (HERE / "reference_nqmc.bin").write_bytes(blob)
    print(f"reference_nqmc.bin: {len(blob)} bytes, record name {record.tensor_name!r}")


if __name__ == "__main__":
    main()
