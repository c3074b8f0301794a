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
    "-shared",
    "-ffp-contract=off",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-command-line-argument",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"),
    "-I" + CSRC,
]


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + ["-o", LIB] + sources()
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
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
