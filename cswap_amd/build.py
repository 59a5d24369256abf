"""Builds ``cswap_amd/libcswap_hip.so`` for gfx950 with hipcc.

    python -m cswap_amd.build            # compile (cross-compiles without a GPU)

The library is built in-tree so that it is the file the tests, the smoke test
and the benchmark load.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libcswap_hip.so")

SOURCES = ["common.cpp", "zfp_kernels.hip", "zvc_kernels.hip", "select.cpp", "planner.cpp", "swap_engine.cpp",
           "compat.cpp"]

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    "-ffp-contract=off",          # the codec has no a*b+c, keep it that way
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc() -> str:
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if c and os.path.exists(c):
            return c
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False) -> str:
    objs = []
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    for s in srcs:
        o = os.path.join(objdir, s + ".o")
        cmd = [hipcc(), *HIPCC_FLAGS, "-x", "hip", "-c", os.path.join(CSRC, s), "-o", o]
        if verbose:
            print(" ".join(cmd))
        r = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {s}:\n{err}")
        if err.strip() and verbose:
            print(err)
        objs.append(o)
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
