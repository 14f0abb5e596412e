"""Runs the exhaustive host-side proof that the quantiser's reciprocal-based code rule gives
the same integer codes as IEEE division + roundf for every bf16 input and every accepted bf16 step
(tests/native/check_fastdiv.c; about 10^9 pairs, ~15 s on 8 cores)."""
import subprocess
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def test_fast_quotient_matches_ieee_exhaustively(tmp_path):
    exe = tmp_path / "check_fastdiv"
    subprocess.run(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", f"-I{ROOT / 'hyc-lora-release_amd' / 'csrc'}",
                    str(ROOT / "tests" / "native" / "check_fastdiv.c"), "-lm", "-o", str(exe)], check=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, res.stdout
    assert "mismatches=0" in res.stdout
    pairs = int(res.stdout.split("pairs=")[1].split()[0])
    assert pairs > 900_000_000
