"""Builds the scalar C restatement used to pin the torch oracle (test infrastructure).

    python oracle/build.py   ->  oracle/_build/libscalar_ref.so

The reference is pure Python (Triton kernels); there is nothing of its own that could
be compiled into oracle/_ref/, so that directory is never produced.
"""
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT = HERE / "_build" / "libscalar_ref.so"


def build(verbose: bool = True) -> Path:
    OUT.parent.mkdir(exist_ok=True)
    cmd = ["gcc", "-O2", "-fPIC", "-shared", "-ffp-contract=off", "-o", str(OUT), str(HERE / "scalar_ref.c"), "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    build()
