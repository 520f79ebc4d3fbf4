"""The NQMC v1 model container against a file written by the reference's own writer
(tests/golden/make_golden_nqmc.py -> reference_nqmc.bin): the reader parses it, the records
come back byte for byte, and the writer of this package reproduces the file exactly.
Mirrors tests/unit/core/test_model_checkpoint.py of the reference (round trip, aliases,
checksum and truncation errors)."""

from pathlib import Path

import numpy as np
import pytest
import torch

from nestquant_aiinfra_amd.core.model_checkpoint import NQMCFileReader, write_nqmc

GOLDEN = Path(__file__).parent / "golden" / "reference_nqmc.bin"
RECORD = "model.layers.0.self_attn.q_proj.weight"


@pytest.fixture()
def reader(tmp_path):
    path = tmp_path / "reference.nqmc"
    path.write_bytes(GOLDEN.read_bytes())
    return NQMCFileReader(path)


def test_reader_parses_the_reference_container(reader, golden):
    assert reader.tensor_count == 4
    assert reader.aliases == {"lm_head.weight": "model.embed_tokens.weight"}
    assert reader.canonical_name("lm_head.weight") == "model.embed_tokens.weight"
    assert reader.model_metadata["hadamard_rotation"]["format"] == "local_hadamard_linear_v1"
    assert [entry.name for entry in reader.entries] == [
        "model.embed_tokens.weight", "model.layers.0.position_ids", RECORD]       # dense sorted, then packed
    entry, embed = reader.read_named_record("lm_head.weight")
    assert entry.kind == "dense" and entry.dtype == torch.bfloat16 and tuple(embed.shape) == (6, 16)
    g = torch.Generator().manual_seed(20261201)
    assert torch.equal(embed, torch.randn(6, 16, generator=g).to(torch.bfloat16))
    _, positions = reader.read_named_record("model.layers.0.position_ids")
    assert positions.dtype == torch.int64 and positions.tolist() == [0, 1, 2, 3, 4]
    entry, record = reader.read_named_record(RECORD)
    assert entry.kind == "nestquant" and entry.shape == (32, 128)
    assert reader.read_entry_blob(entry) == golden["nqrt_bytes"].tobytes()
    assert np.array_equal(np.frombuffer(record.indices.code_payload, dtype=np.uint8), golden["nqrt_code_payload"])
    assert np.array_equal(record.row_norms.numpy(), golden["nqrt_norms"])
    with pytest.raises(KeyError):
        reader.get_entry("missing.weight")


def test_writer_reproduces_the_reference_bytes(reader, tmp_path):
    dense = {entry.name: reader.read_entry(entry) for entry in reader.entries if entry.kind == "dense"}
    packed = {entry.name: reader.read_entry(entry) for entry in reader.entries if entry.kind == "nestquant"}
    path = tmp_path / "ours.nqmc"
    write_nqmc(path, dense_tensors=dense, quantized_tensors=packed, aliases=reader.aliases,
               model_metadata=reader.model_metadata)
    assert path.read_bytes() == GOLDEN.read_bytes()


def test_corruption_is_detected(tmp_path):
    blob = bytearray(GOLDEN.read_bytes())
    path = tmp_path / "bad.nqmc"
    path.write_bytes(bytes(blob[:-1]))
    with pytest.raises(ValueError, match="lengths"):
        NQMCFileReader(path)
    flipped = bytearray(blob)
    flipped[-1] ^= 1
    path.write_bytes(bytes(flipped))
    with pytest.raises(ValueError, match="checksum"):
        NQMCFileReader(path)
    NQMCFileReader(path, verify_checksum=False)                 # explicit opt-out still parses
    wrong_magic = bytearray(blob)
    wrong_magic[0:4] = b"NQMX"
    path.write_bytes(bytes(wrong_magic))
    with pytest.raises(ValueError, match="magic"):
        NQMCFileReader(path)
