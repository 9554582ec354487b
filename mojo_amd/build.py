"""Compile the HIP sources under ``mojo_amd/csrc`` into ``mojo_amd/libqmm.so``.

One explicit ``hipcc`` line for gfx950; nothing is built at import time.
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libqmm.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-shared",
    # quantisers are specified as separate IEEE operations; hot loops call fmaf explicitly
    "-ffp-contract=off",
    # no compiler-generated packed fp32 arithmetic
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose: bool = False) -> str:
    cmd = [HIPCC, *FLAGS, "-o", LIB, *sources()]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed building libqmm.so")
    if verbose and proc.stderr.strip():
        sys.stderr.write(proc.stderr)
    return LIB


if __name__ == "__main__":
    build(verbose=True)
