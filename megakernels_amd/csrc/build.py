"""Builds libmk_llama.so (the HIP megakernel and its C ABI) for gfx950.

    python megakernels_amd/csrc/build.py

The library is built in-tree next to its sources.  Flags that matter:
``-ffp-contract=off`` (only the explicit fmaf() calls fuse, so results are
reproducible), and packed-fp32 code generation turned off.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
SOURCE = HERE / "mk_llama.hip"
LIBRARY = HERE / "libmk_llama.so"

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def find_hipcc() -> str:
    candidates = [os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"]
    for cand in candidates:
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (set HIPCC)")


def build(verbose: bool = False) -> Path:
    cmd = [find_hipcc(), *HIPCC_FLAGS, str(SOURCE), "-o", str(LIBRARY)]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    noise = "packed-fp32-ops"
    for line in (proc.stdout + proc.stderr).splitlines():
        if noise not in line and verbose:
            print(line)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed")
    return LIBRARY


if __name__ == "__main__":
    print(build(verbose=True))
