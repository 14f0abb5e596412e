"""Build recipe for the gfx950 kernel library (libhyclora.so, next to this file).

    python hyc-lora-release_amd/build.py            # compile every .hip under csrc/

hipcc cross-compiles for gfx950 without a GPU present.  The flags matter:
  -ffp-contract=off            the integer-code arithmetic relies on explicit fmaf only;
  -packed-fp32-ops disabled    packed FP32 VALU forms are kept out of the generated code.
"""
from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB = HERE / "libhyclora.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(str(p) for p in CSRC.glob("*.hip"))


def build(verbose: bool = True) -> Path:
    """Compile csrc/*.hip into libhyclora.so (always recompiles)."""
    cmd = [HIPCC, *FLAGS, "-o", str(LIB), *sources()]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err:
        print(err, file=sys.stderr)
    return LIB


if __name__ == "__main__":
    build()
