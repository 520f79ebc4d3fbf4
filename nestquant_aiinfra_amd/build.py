"""Builds libnqhip.so (the gfx950 kernels behind the C ABI in include/nqhip.h) in-tree.

    python -m nestquant_aiinfra_amd.build [-v] [--define NAME ...] [--output PATH]

`--define NQ_PHASE_STAMPS --output PATH` makes a measuring build beside the product library: the
row encoder then stamps the wall clock at its phase boundaries (read with nq_debug_phase_stamps;
`bench.py --only encode_phases --library PATH` prints the table).  Two more names serve timing
comparisons on one GPU: `NQ_ATTN_FORCE_PAGES=4|8|16` fixes the decode attention's pages per chunk,
`NQ_MFMA_FROM_ROWS=N` the row count from which the decode linears run on the matrix cores.

hipcc cross-compiles for gfx950 without a GPU.  Flags that are part of the contract:
  -ffp-contract=off   the codec's float32 operation order is specified; fused
                      multiply-adds appear only where the source spells fmaf;
  -fhip-fp32-correctly-rounded-divide-sqrt   IEEE division and sqrt on the device;
  -packed-fp32-ops off   no packed-FP32 VALU instructions.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE = Path(__file__).resolve().parent
CSRC = PACKAGE / "csrc"
LIBRARY = PACKAGE / "libnqhip.so"
ARCH = "gfx950"

FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-pragmas",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build(verbose: bool = False, defines: tuple[str, ...] = (), output: Path = LIBRARY) -> Path:
    """Compile every csrc/*.hip for gfx950 and link the library (libnqhip.so unless `output`
    names another file).  Always recompiles."""
    hipcc = os.environ.get("HIPCC", "hipcc")
    objects = []
    suffix = ".o" if output == LIBRARY else f".{Path(output).stem}.o"

    def compile_one(source: Path) -> Path:
        obj = source.with_suffix(suffix)
        command = [hipcc, *FLAGS, *(f"-D{name}" for name in defines), "-c", str(source), "-o", str(obj)]
        if verbose:
            print(" ".join(command), flush=True)
        result = subprocess.run(command, capture_output=True, text=True)
        # the host pass warns that it does not know the packed-fp32 feature: harmless
        noise = "is not a recognized feature for this target"
        stderr = "\n".join(line for line in result.stderr.splitlines() if noise not in line)
        if result.returncode != 0:
            raise RuntimeError(f"hipcc failed on {source.name}:\n{stderr}")
        if verbose and stderr.strip():
            print(stderr, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(sources()) or 1)) as pool:
        objects = list(pool.map(compile_one, sources()))
    link = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(output), *map(str, objects)]
    result = subprocess.run(link, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"link failed:\n{result.stderr}")
    for obj in objects:
        obj.unlink(missing_ok=True)
    return Path(output)


if __name__ == "__main__":
    import argparse
    parser = argparse.ArgumentParser()
    parser.add_argument("-v", action="store_true")
    parser.add_argument("--define", action="append", default=[])
    parser.add_argument("--output", type=Path, default=LIBRARY)
    options = parser.parse_args()
    print(build(verbose=options.v, defines=tuple(options.define), output=options.output.resolve()))
