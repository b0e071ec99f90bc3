"""Builds libmoonep_hip.so (the HIP kernels + C ABI) in-tree for gfx950.

    python -m moonep_amd.build

hipcc cross-compiles without a GPU.  The library sits next to the package so
that it travels with the source tree; nothing is installed.
"""

from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmoonep_hip.so")
SOURCES = ["capi.hip", "planner.hip", "dispatch.hip", "combine.hip", "prefetch.hip",
           "grouped_gemm.hip"]
FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared",
    "-Wall", "-Wno-unused-function",
    # packed-fp32 VALU forms are kept off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build(verbose: bool = True) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *FLAGS, *[os.path.join(CSRC, s) for s in SOURCES], "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
