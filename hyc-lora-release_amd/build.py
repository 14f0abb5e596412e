"""Build recipe for the gfx950 kernel library (libhyclora.so, next to this file).

    python hyc-lora-release_amd/build.py            # compile every .hip under csrc/

hipcc cross-compiles for gfx950 without a GPU present.  Each source is compiled to an object of
its own (in parallel, objects under csrc/_obj/) and the objects are linked into the library.
The flags matter:
  -ffp-contract=off            the integer-code arithmetic relies on explicit fmaf only;
  -packed-fp32-ops disabled    packed FP32 VALU forms are kept out of the generated code.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
OBJ = CSRC / "_obj"
LIB = HERE / "libhyclora.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def sources():
    return sorted(str(p) for p in CSRC.glob("*.hip"))


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}): {' '.join(cmd)}\n{err}")
    if verbose and err:
        print(err, file=sys.stderr)


def build(verbose: bool = True, only=None) -> Path:
    """Compile csrc/*.hip into libhyclora.so.  Always recompiles every source, unless `only`
    names the sources (file names) to recompile and the other objects are already there."""
    OBJ.mkdir(exist_ok=True)
    todo = []
    objects = []
    for src in sources():
        obj = OBJ / (Path(src).stem + ".o")
        objects.append(str(obj))
        if only is None or Path(src).name in only or not obj.exists():
            todo.append([HIPCC, *FLAGS, "-c", "-o", str(obj), src])
    jobs = max(1, min(len(todo), int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)), 16))
    with ThreadPoolExecutor(jobs) as pool:
        list(pool.map(lambda c: _run(c, verbose), todo))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *objects], verbose)
    return LIB


if __name__ == "__main__":
    build(only=set(sys.argv[1:]) or None)
