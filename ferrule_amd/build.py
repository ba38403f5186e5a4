"""Builds the provider's shared library in-tree with hipcc for gfx950.

    python -m ferrule_amd.build          # compile every csrc/*.hip -> libferrule_hip.so

The library has a plain C ABI (include/ferrule_hip_provider.h) and links only
against the HIP runtime; no torch headers are involved.
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libferrule_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Wall",
    "-Wno-unused-function",
    # hipcc -O3 may otherwise fuse scalar fp32 code into packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def build(verbose: bool = True) -> str:
    cmd = ["hipcc", *HIPCC_FLAGS, "-o", LIB, *sources()]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


def is_built() -> bool:
    if not os.path.exists(LIB):
        return False
    newest = max(os.path.getmtime(p) for p in sources() + glob.glob(os.path.join(CSRC, "*.cuh")))
    return os.path.getmtime(LIB) >= newest


if __name__ == "__main__":
    build()
    sys.exit(0)
