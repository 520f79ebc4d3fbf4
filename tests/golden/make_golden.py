"""Writes the golden fixtures in this directory by running the reference's CPU core.

Run once, in the build container only (the reference checkout is not available
anywhere else):

    python tests/golden/make_golden.py [/path/to/reference]

It covers only what no closed form, known answer or invariant pins: decisions of
the E8 nearest-point routine on exact Voronoi ties under torch's CPU float order
(hence undithered decodes and the per-block beta choice), the bits of
``torch.linalg.vector_norm``, and the byte layout of the NQRT / NQKV containers.
Outputs are data only: seeded inputs and the reference's outputs for them.
"""

from __future__ import annotations

import hashlib
import json
import sys
import time
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
REFERENCE = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
sys.path.insert(0, str(REFERENCE))

from nestquant.core.codec import decode_nested, encode_nested, generate_e8_dither_stateless  # noqa: E402
from nestquant.core.kv_format import PackedNQKVPage  # noqa: E402
from nestquant.core.lattice import nearest_e8  # noqa: E402
from nestquant.core.quantizer import quantize_rows  # noqa: E402
from nestquant.core.rotation import hadamard, signed_hadamard  # noqa: E402
from nestquant.core.tensor_checkpoint import PackedNestQuantTensor  # noqa: E402

Q = 14
ACTIVATION_BETAS = tuple(v / 14 for v in (3.47, 4.74, 6.90, 18.11))
WEIGHT_BETAS = tuple(v / 14 for v in (4.0, 5.5, 7.0, 18.0))
KEY_BETAS = tuple(v / 14 for v in (3.50, 4.58, 6.47, 17.06))
VALUE_BETAS = tuple(v / 14 for v in (3.53, 5.59, 9.62, 29.03))


def sha(array_or_bytes) -> str:
    data = array_or_bytes if isinstance(array_or_bytes, (bytes, bytearray)) else np.ascontiguousarray(array_or_bytes).tobytes()
    return hashlib.sha256(data).hexdigest()


def main() -> None:
    torch.manual_seed(0)
    out: dict[str, np.ndarray] = {}
    meta: dict[str, object] = {"torch": torch.__version__, "threads": torch.get_num_threads(), "q": Q}

    # --- E8 nearest point on random points and on exact ties ------------------
    g = torch.Generator().manual_seed(101)
    pts = torch.randn(4096, 8, generator=g) * 2.5
    ties = torch.randint(-8, 9, (2048, 8), generator=g).float() * 0.25   # quarter-integers: many exact ties
    x = torch.cat([pts, ties])
    point, dist = nearest_e8(x)
    out["e8_x"], out["e8_point"], out["e8_dist"] = x.numpy(), point.numpy(), dist.numpy()

    # --- undithered decode of every-residue samples + the three boundary blocks ---
    codes = torch.randint(0, Q, (8192, 8), generator=g)
    boundary = torch.tensor([[5, 12, 3, 0, 7, 3, 9, 2], [5, 5, 2, 7, 2, 4, 10, 2], [3, 0, 2, 12, 4, 9, 7, 2]])
    codes = torch.cat([boundary, codes])
    out["decode_codes"] = codes.numpy().astype(np.uint8)
    out["decode_out"] = decode_nested(codes, Q).numpy()

    # --- stateless dither ----------------------------------------------------------
    for seed in (0, 20261025, 2**31 - 1):
        out[f"dither_{seed}"] = generate_e8_dither_stateless(64, seed).numpy()
    out["dither_offset_1000_seed_20261025"] = generate_e8_dither_stateless(16, 20261025, block_offset=1000).numpy()

    # --- quantize_rows, undithered (activation / KV flavour) -----------------------
    for name, rows, n, seed in (("qr64", 64, 64, 201), ("qr2048", 16, 2048, 202)):
        gg = torch.Generator().manual_seed(seed)
        x0 = torch.randn(rows, n, generator=gg)
        signs = (2 * torch.randint(0, 2, (n,), generator=gg) - 1).float()
        xr = signed_hadamard(x0, signs)
        if name == "qr64":
            xr[5] = 0.0                       # zero row stays zero
        result = quantize_rows(xr, Q, ACTIVATION_BETAS)
        out[f"{name}_x"] = xr.numpy()
        out[f"{name}_codes"] = result.codes.numpy().astype(np.uint8)
        out[f"{name}_beta"] = result.beta_indices.numpy().astype(np.uint8)
        out[f"{name}_norms"] = result.row_norms.numpy()
        out[f"{name}_deq"] = result.dequantize().numpy()

    # --- NQRT4 record: dithered weight 32 x 128 ---------------------------------------
    gg = torch.Generator().manual_seed(203)
    w = hadamard(0.02 * torch.randn(32, 128, generator=gg))
    seed = 20261029
    dither = generate_e8_dither_stateless(32 * 16, seed).reshape(32, 16, 8)
    rows = quantize_rows(w, Q, WEIGHT_BETAS, dither=dither)
    record = PackedNestQuantTensor.from_quantized_rows("model.layers.0.self_attn.q_proj.weight", rows, dither_seed=seed)
    blob = record.to_bytes()
    out["nqrt_w"] = w.numpy()
    out["nqrt_bytes"] = np.frombuffer(blob, dtype=np.uint8).copy()
    out["nqrt_code_payload"] = np.frombuffer(record.indices.code_payload, dtype=np.uint8).copy()
    out["nqrt_beta_payload"] = np.frombuffer(record.indices.beta_payload, dtype=np.uint8).copy()
    out["nqrt_norms"] = record.row_norms.numpy()
    out["nqrt_deq"] = PackedNestQuantTensor.from_bytes(blob).dequantize().numpy()
    meta["nqrt_seed"] = seed

    # --- NQKV page [16, 8, 64], BF16 inputs, dual beta tables (v2) and legacy (v1) -------
    gg = torch.Generator().manual_seed(204)
    key = hadamard(torch.randn(16, 8, 64, generator=gg)).to(torch.bfloat16)
    value = torch.randn(16, 8, 64, generator=gg).to(torch.bfloat16)
    page = PackedNQKVPage.from_tensors(key, value, page_size=16, q=Q, key_betas=KEY_BETAS, value_betas=VALUE_BETAS)
    out["kv_key_bf16_bits"] = key.view(torch.int16).numpy()
    out["kv_value_bf16_bits"] = value.view(torch.int16).numpy()
    out["kv_key_codes"] = np.frombuffer(page.key_indices.code_payload, dtype=np.uint8).copy()
    out["kv_key_betas"] = np.frombuffer(page.key_indices.beta_payload, dtype=np.uint8).copy()
    out["kv_key_norms"] = page.key_norms.numpy()
    out["kv_value_codes"] = np.frombuffer(page.value_indices.code_payload, dtype=np.uint8).copy()
    out["kv_value_betas"] = np.frombuffer(page.value_indices.beta_payload, dtype=np.uint8).copy()
    out["kv_value_norms"] = page.value_norms.numpy()
    dk, dv = page.dequantize(output_dtype=torch.float32)
    out["kv_key_deq"], out["kv_value_deq"] = dk.numpy(), dv.numpy()
    meta["kv_payload_bytes"] = page.payload_bytes
    meta["kv_container_v2_bytes"] = page.serialized_bytes
    meta["kv_container_v2_sha256"] = sha(page.to_bytes())
    partial = PackedNQKVPage.from_tensors(key[:5], value[:5], page_size=16, q=Q, betas=KEY_BETAS)
    meta["kv_container_v1_bytes"] = partial.serialized_bytes
    out["kv_partial_key_codes"] = np.frombuffer(partial.key_indices.code_payload, dtype=np.uint8).copy()
    out["kv_partial_key_norms"] = partial.key_norms.numpy()

    # --- config 1: 2048 x 2048, hashes only (plus wall time of the reference itself) -------
    g = torch.Generator().manual_seed(58)
    x0 = torch.randn(2048, 2048, generator=g)
    signs = (2 * torch.randint(0, 2, (2048,), generator=g) - 1).float()
    xr = signed_hadamard(x0, signs)
    act = signed_hadamard(torch.randn(1, 2048, generator=g), signs)
    t0 = time.perf_counter()
    a = quantize_rows(xr, Q, ACTIVATION_BETAS)
    t1 = time.perf_counter()
    from nestquant.core.packing import pack_nestquant_indices
    pa = pack_nestquant_indices(a.codes, a.beta_indices, q=Q, beta_count=4)
    dseed = 20261025
    dither = generate_e8_dither_stateless(2048 * 256, dseed).reshape(2048, 256, 8)
    t2 = time.perf_counter()
    b = quantize_rows(xr, Q, WEIGHT_BETAS, dither=dither)
    t3 = time.perf_counter()
    pb = pack_nestquant_indices(b.codes, b.beta_indices, q=Q, beta_count=4)
    qa = quantize_rows(act, Q, ACTIVATION_BETAS)
    t4 = time.perf_counter()
    y = b.dequantize() @ qa.dequantize().T
    t5 = time.perf_counter()
    meta["config1"] = {
        "input_sha256": sha(xr.numpy()),
        "A_code_sha256": sha(pa.code_payload), "A_beta_sha256": sha(pa.beta_payload),
        "A_norm_sha256": sha(a.row_norms.numpy()),
        "B_code_sha256": sha(pb.code_payload), "B_beta_sha256": sha(pb.beta_payload),
        "act_code_sha256": sha(pack_nestquant_indices(qa.codes, qa.beta_indices, q=Q, beta_count=4).code_payload),
        "reference_quantize_rows_undithered_s": t1 - t0,
        "reference_quantize_rows_dithered_s": t3 - t2,
        "reference_dequantize_matvec_s": t5 - t4,
        "dither_seed": dseed,
    }
    out["config1_y"] = y.numpy().reshape(-1)
    out["config1_act"] = act.numpy()

    np.savez_compressed(HERE / "reference_vectors.npz", **out)
    (HERE / "reference_vectors.json").write_text(json.dumps(meta, indent=1, sort_keys=True) + "\n")
    print(json.dumps(meta, indent=1, sort_keys=True))


if __name__ == "__main__":
    main()
