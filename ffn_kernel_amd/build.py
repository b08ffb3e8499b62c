"""Build libffnk.so (the HIP kernels + C ABI) for gfx950 with hipcc.

    python -m ffn_kernel_amd.build            # compile every csrc/*.hip and link

hipcc cross-compiles without a GPU.  The library is written next to this file so that it
travels with the source tree; nothing is installed outside the tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
OBJ_DIR = CSRC / "build"
LIB_PATH = PKG_DIR / "libffnk.so"

ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    "-Wno-unused-function",
    # scalar fp32 code only: keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; libffnk.so cannot be built")
    return exe


def _compile(src: Path) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_library(jobs: int | None = None, verbose: bool = True) -> Path:
    """Compile csrc/*.hip and link libffnk.so.  Always recompiles."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    if not sources:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    jobs = jobs or min(len(sources), os.cpu_count() or 4, 16)
    if verbose:
        print(f"[ffn_kernel_amd.build] hipcc {ARCH}: {len(sources)} files, {jobs} jobs", flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, sources))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[ffn_kernel_amd.build] wrote {LIB_PATH} ({LIB_PATH.stat().st_size >> 10} KiB)", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
