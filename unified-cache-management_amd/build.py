"""Builds libucm_hip.so (gfx950) in place with hipcc.

    python unified-cache-management_amd/build.py

-ffp-contract=off: the kernels spell every fused multiply-add as
__builtin_fmaf so that their fp32 results equal the reference's CPU arithmetic
bit for bit; the compiler must not fuse or split anything else.
Packed fp32 instructions are switched off for all device code.
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libucm_hip.so")

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-command-line-argument",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"),
    "-I" + CSRC,
]
OBJ_DIR = os.path.join(HERE, "build")


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature and says so: harmless
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)


def build(verbose: bool = False, incremental: bool = False) -> str:
    """Compiles every source file to an object (in parallel) and links the library.  With ``incremental`` a file
    whose object is newer than it and than every header is not compiled again."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    headers = glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(ROOT, "include", "*.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    jobs, objects = [], []
    for src in sources():
        obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
        objects.append(obj)
        fresh = os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header)
        if not (incremental and fresh):
            jobs.append([hipcc] + FLAGS + ["-c", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=min(8, max(len(jobs), 1))) as pool:
        list(pool.map(lambda c: _run(c, verbose), jobs))
    _run([hipcc, "--offload-arch=gfx950", "-fPIC", "-shared", "-fno-gpu-rdc", "-o", LIB] + objects, verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, incremental="--incremental" in sys.argv))
