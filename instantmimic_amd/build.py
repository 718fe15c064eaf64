"""Builds ``libimhip.so`` in-tree with hipcc for gfx950 (cross-compiles without a GPU)."""

from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libimhip.so")

SOURCES = ["tree_plan.cpp", "tree_kernels.hip"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # every fused multiply-add is spelled in the source: results must not depend
    # on what the compiler decides to contract
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build_library(verbose: bool = True) -> str:
    cmd = ["hipcc", *FLAGS, "-x", "hip", *[os.path.join(CSRC, s) for s in SOURCES], "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build_library()
    sys.exit(0)
