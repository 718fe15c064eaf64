"""Builds ``libimhip.so`` in-tree with hipcc for gfx950 (cross-compiles without a GPU).

Besides the hand-written sources, one kernel per known dof tree is generated
(``codegen/tree_row16.py``) and compiled in: the five benchmark trees' best plans.
Other trees run on the generic table-driven kernel.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
GEN = os.path.join(CSRC, "gen")
OBJ = os.path.join(HERE, "_obj")
LIB = os.path.join(HERE, "libimhip.so")

SOURCES = ["tree_plan.cpp", "tree_kernels.hip", "muscle_kernels.hip", "muscle_geometry.hip", "sparse_kernels.hip", "blocked_kernels.hip", "tree_reduce_kernels.hip", "newton_kernels.hip"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # every fused multiply-add is spelled in the source: results must not depend
    # on what the compiler decides to contract
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unused-variable",
    "-Wno-unused-command-line-argument",
]  # fmt: skip


def _python_planner(parents):
    """The reference planner's result for a tree, through the library's host planner
    when it is already built, else through a local restatement (bootstrap)."""
    from .codegen import plan_bootstrap

    return plan_bootstrap.best_plan(parents)


def generate_sources() -> list[str]:
    from . import synth
    from .codegen import tree_row16

    os.makedirs(GEN, exist_ok=True)
    out = []
    only = os.environ.get("IMHIP_GEN_ONLY")  # development aid: comma-separated shape names
    for name, shape in synth.SHAPES.items():
        if only and name not in only.split(","):
            continue
        st, groups, trunk, eligible = _python_planner(list(shape.parents))
        if not eligible or len(st[0]) > 64:
            continue
        src = tree_row16.generate(name, *st, groups, trunk)
        path = os.path.join(GEN, f"tree_row16_{name}.hip")
        if not os.path.exists(path) or open(path).read() != src:
            with open(path, "w") as f:
                f.write(src)
        out.append(path)
    return out


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    deps = [src] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    deps.append(os.path.join(HERE, "..", "include", "imhip.h"))
    if os.path.exists(obj) and not os.environ.get("IMHIP_REBUILD"):
        if os.path.getmtime(obj) > max(os.path.getmtime(d) for d in deps):
            return obj
    cmd = ["hipcc", *FLAGS, "-c", "-x", "hip", src, "-o", obj]
    subprocess.run(cmd, check=True)
    return obj


def build_library(verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    sources = [os.path.join(CSRC, s) for s in SOURCES] + generate_sources()
    if verbose:
        print("hipcc", " ".join(FLAGS), "\n  " + "\n  ".join(sources), flush=True)
    with ThreadPoolExecutor(max_workers=8) as pool:
        objs = list(pool.map(_compile, sources))
    subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB], check=True)
    return LIB


if __name__ == "__main__":
    build_library()
    sys.exit(0)
