"""Builds the provider's shared library in-tree with hipcc for gfx950.

    python -m ferrule_amd.build          # compile every csrc/*.hip -> libferrule_hip.so

The library has a plain C ABI (include/ferrule_hip_provider.h) and links only
against the HIP runtime; no torch headers are involved.

Every translation unit is compiled on its own (in parallel) into ``build/`` and
the objects are linked into ``libferrule_hip.so``.  A digest of every source and
header the library is made from is compiled into it
(``ferrule_hip_source_digest``); ``abi.load()`` compares it with the digest of the
files on disk, so a library left over from older sources or older ABI structs is
refused instead of being called with blocks it would misread.
"""
from __future__ import annotations

import glob
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libferrule_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # the direct-to-LDS loads set M0 in inline assembly and say so in their clobber lists; the
    # compiler warns about every reserved register named there
    "-Wno-inline-asm",
    # hipcc -O3 may otherwise fuse scalar fp32 code into packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def headers() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.cuh")) + glob.glob(os.path.join(CSRC, "*.h")) +
                  glob.glob(os.path.join(INCLUDE, "*.h")))


def source_digest() -> str:
    """sha256 over the names and contents of every file the library is compiled from."""
    h = hashlib.sha256()
    for path in sources() + headers():
        h.update(os.path.basename(path).encode())
        h.update(b"\0")
        with open(path, "rb") as f:
            h.update(f.read())
        h.update(b"\0")
    return h.hexdigest()


def _compile(args: tuple[str, str, str, bool]) -> str:
    src, obj, digest, verbose = args
    cmd = ["hipcc", *HIPCC_FLAGS, "-c", src, "-o", obj]
    if os.path.basename(src) == "manifest.hip":  # the one unit that exports the digest
        cmd.insert(1, f'-DFERRULE_HIP_SOURCE_DIGEST="{digest}"')
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return obj


def build(verbose: bool = True, jobs: int | None = None, changed_only: bool = False) -> str:
    """Compile every source and link the library.  ``changed_only`` (a development
    shortcut, ``--changed`` on the command line) keeps an object that is newer than its
    source and every header."""
    os.makedirs(OBJ, exist_ok=True)
    digest = source_digest()
    work = [(src, os.path.join(OBJ, os.path.basename(src)[:-4] + ".o"), digest, verbose) for src in sources()]
    objects_all = [w[1] for w in work]
    if changed_only:
        newest_header = max(os.path.getmtime(p) for p in headers())
        work = [w for w in work if os.path.basename(w[0]) == "manifest.hip" or not os.path.exists(w[1]) or
                os.path.getmtime(w[1]) < max(os.path.getmtime(w[0]), newest_header)]
    if jobs is None:
        jobs = max(1, min(len(work), os.cpu_count() or 1, 16))
    if not work:
        jobs = 1
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_compile, work))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objects_all]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


def is_built() -> bool:
    """True when the library exists; whether it matches the sources is checked at load
    time through the digest it carries."""
    return os.path.exists(LIB)


if __name__ == "__main__":
    build(changed_only="--changed" in sys.argv[1:])
    sys.exit(0)
