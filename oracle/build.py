"""Compile oracle/masked_ref.c with gcc into oracle/_build/libmasked_ref.so (test infrastructure)."""
from __future__ import annotations

import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT_DIR = HERE / "_build"
LIB = OUT_DIR / "libmasked_ref.so"


def build_oracle(verbose: bool = True) -> Path:
    OUT_DIR.mkdir(exist_ok=True)
    cmd = ["gcc", "-O2", "-fPIC", "-shared", "-fopenmp", "-ffp-contract=off", "-o", str(LIB),
           str(HERE / "masked_ref.c"), "-lm"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"gcc failed on oracle/masked_ref.c:\n{proc.stderr}")
    if verbose:
        print(f"[oracle.build] wrote {LIB}", flush=True)
    return LIB


if __name__ == "__main__":
    build_oracle()
