"""Builds libadamas_hip.so (hand-written HIP kernels + the C ABI) for gfx950 with hipcc.

The library is built in-tree (adamas_amd/lib/) so that it travels with the source tree; nothing is
installed into site-packages and nothing is compiled at import time.
"""
from __future__ import annotations

import os
import shutil
import subprocess
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libadamas_hip.so"

SOURCES = ["hadamard.hip", "estimate.hip", "topk.hip", "attention.hip", "fused_step.hip",
           "decoder_ops.hip"]

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    # packed fp32 instructions are switched off for all device code of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: set HIPCC or put /opt/rocm/bin on PATH")


def _run(cmd, verbose):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or proc.returncode != 0:
        print(" ".join(cmd))
        print(proc.stdout)
        print(proc.stderr)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed with exit code {proc.returncode}")


def build_library(verbose: bool = False, jobs: int = 0) -> Path:
    """Compile every HIP source (one hipcc process each, side by side) and link them into
    adamas_amd/lib/libadamas_hip.so; returns its path.  Every call recompiles everything."""
    from concurrent.futures import ThreadPoolExecutor

    LIB_DIR.mkdir(parents=True, exist_ok=True)
    obj_dir = LIB_DIR / "obj"
    obj_dir.mkdir(exist_ok=True)
    hipcc = find_hipcc()
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 1, 8)
    objects = [obj_dir / (Path(src).stem + ".o") for src in SOURCES]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda so: _run([hipcc, *HIPCC_FLAGS, "-c", str(CSRC_DIR / so[0]), "-o",
                                       str(so[1])], verbose), zip(SOURCES, objects)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *[str(o) for o in objects], "-o",
          str(LIB_PATH)], verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
