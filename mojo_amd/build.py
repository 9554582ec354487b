"""Compile the HIP sources under ``mojo_amd/csrc`` into ``mojo_amd/libqmm.so``.

Explicit ``hipcc`` lines for gfx950: one object per source file (compiled side by side), then one
link.  Nothing is built at import time.
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libqmm.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    # quantisers are specified as separate IEEE operations; hot loops call fmaf explicitly
    "-ffp-contract=off",
    # no compiler-generated packed fp32 arithmetic
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


# Per-file additions.  Kernel-argument preloading (the first dwords of the argument block arrive in scalar registers
# with the wavefront instead of through a scalar load) for the decode kernels whose first microsecond decides a launch.
PER_FILE_FLAGS = {
    "gemv_q4k_lanes.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=12"],
    "gemv_q4k_mm.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=12"],
    "gemm_q4_0.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=12"],
    "gemv_q4_0.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=14"],
}


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _headers_mtime() -> float:
    hdrs = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(HERE, "..", "include", "*.h"))
    return max(os.path.getmtime(h) for h in hdrs)


def _compile(src: str, obj: str, verbose: bool) -> None:
    cmd = [HIPCC, *FLAGS, *PER_FILE_FLAGS.get(os.path.basename(src), []), "-c", "-o", obj, src]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError(f"hipcc failed on {os.path.basename(src)}")
    noise = "not a recognized feature for this target"  # the host pass does not know the gfx950 feature flag
    rest = [ln for ln in proc.stderr.splitlines() if ln.strip() and noise not in ln]
    if verbose and rest:
        sys.stderr.write("\n".join(rest) + "\n")


def build(verbose: bool = False, force: bool = True, jobs: int | None = None) -> str:
    """Compile every source (``force=False``: only those newer than their object) and link the library."""
    os.makedirs(OBJ, exist_ok=True)
    hdr_time = _headers_mtime()
    todo, objs = [], []
    for src in sources():
        obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        if force or not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(src), hdr_time):
            todo.append((src, obj))
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        for fut in [pool.submit(_compile, s, o, verbose) for s, o in todo]:
            fut.result()
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed linking libqmm.so")
    return LIB


if __name__ == "__main__":
    build(verbose=True, force="--incremental" not in sys.argv)
