"""Builds ``libimhip.so`` in-tree with hipcc for gfx950 (cross-compiles without a GPU).

Besides the hand-written sources, one kernel per known dof tree is generated
(``codegen/tree_row16.py``) and compiled in: the five benchmark trees' best plans.
Kernels for any other tree are generated when its plan is created (``codegen/jit.py``); the
table-driven kernel serves plans the generator declines.
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

SOURCES = ["tree_plan.cpp", "sparse_plan.cpp", "tree_kernels.hip", "muscle_kernels.hip", "muscle_geometry.hip", "sparse_kernels.hip", "blocked_kernels.hip", "tile_kernels.hip", "dense_column_kernels.hip", "tree_reduce_kernels.hip", "newton_kernels.hip", "newton_search_kernels.hip", "newton_init_kernels.hip", "implicit_kernels.hip"]

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


PLANNER_LIB = os.path.join(OBJ, "libimplan_host.so")


def _host_planner():
    """The library's own host planner (csrc/tree_plan.cpp), built alone ahead of everything
    else: the kernel generator needs each known tree's plan before ``libimhip.so`` exists."""
    import ctypes as C

    src = os.path.join(CSRC, "tree_plan.cpp")
    os.makedirs(OBJ, exist_ok=True)
    stale = not os.path.exists(PLANNER_LIB) or os.path.getmtime(PLANNER_LIB) < max(
        os.path.getmtime(p) for p in (src, os.path.join(CSRC, "common.h"), os.path.join(HERE, "..", "include", "imhip.h"))
    )
    if stale or os.environ.get("IMHIP_REBUILD"):
        cmd = ["hipcc", "--offload-arch=gfx950", "-O1", "-std=c++17", "-fPIC", "-shared", "-DIM_PLANNER_ONLY",
               "-Wno-unused-command-line-argument", "-x", "hip", src, "-o", PLANNER_LIB]  # fmt: skip
        subprocess.run(cmd, check=True)
    return C.CDLL(PLANNER_LIB)


def _plan_of_tree(parents, groups: int = 0):
    """((rowadr, rownnz, colind), groups, trunk, eligible) of a dof tree from the host planner."""
    import ctypes as C

    from . import _lib, synth

    rowadr, rownnz, colind = synth.csr_from_parents(parents)
    lib = _host_planner()
    handle = C.c_void_p()
    vp = lambda a: C.c_void_p(a.ctypes.data)  # noqa: E731
    status = lib.im_tree_plan_create(len(parents), vp(rowadr), vp(rownnz), vp(colind), int(colind.size), int(groups), 1, C.byref(handle))
    if status != 0:
        raise RuntimeError(f"host planner refused the tree (status {status})")
    info = _lib.TreePlanInfo()
    lib.im_tree_plan_get_info(handle, C.byref(info))
    import numpy as np

    gptr, gdofs, trunk = np.zeros(info.ngroups + 1, np.int32), np.zeros(max(info.nv - info.ntrunk, 1), np.int32), np.zeros(max(info.ntrunk, 1), np.int32)
    lib.im_tree_plan_get_arrays(handle, vp(gptr), vp(gdofs), vp(trunk), None)
    lib.im_tree_plan_destroy.argtypes = [C.c_void_p]
    lib.im_tree_plan_destroy(handle)
    groups = tuple(tuple(int(d) for d in gdofs[gptr[j] : gptr[j + 1]]) for j in range(info.ngroups))
    st = tuple(tuple(int(v) for v in a) for a in (rowadr, rownnz, colind))
    return st, groups, tuple(int(d) for d in trunk[: info.ntrunk]), bool(info.beats_dense)


def generate_sources() -> list[str]:
    from . import synth
    from .codegen import tree_row16

    os.makedirs(GEN, exist_ok=True)
    out = []
    only = os.environ.get("IMHIP_GEN_ONLY")  # development aid: comma-separated shape names
    for name, shape in synth.SHAPES.items():
        if only and name not in only.split(","):
            continue
        st, groups, trunk, eligible = _plan_of_tree(list(shape.parents))
        if not eligible or len(st[0]) > 64:
            continue
        src = tree_row16.generate(name, *st, groups, trunk)
        path = os.path.join(GEN, f"tree_row16_{name}.hip")
        if not os.path.exists(path) or open(path).read() != src:
            with open(path, "w") as f:
                f.write(src)
        out.append(path)
    return out


def prebuild_kernels(trees, group_counts=(0,)) -> list[str]:
    """Code objects of the generated kernels for the given dof trees (parent lists) and group
    counts (0 = the best plan), into the kernel cache beside the library: what plan creation would
    otherwise compile on first use."""
    from .codegen import jit, tree_row16

    # code objects of other generator versions or settings are never loaded again: out with them
    tag = jit._source_tag()
    for name in os.listdir(jit.cache_dir()):
        if name.startswith("tree_row16_") and name.endswith(".co") and not name.endswith(f"_{tag}.co"):
            os.remove(os.path.join(jit.cache_dir(), name))
    keys = set()
    for parents in trees:
        for count in group_counts:
            st, groups, trunk, _ = _plan_of_tree(list(parents), count)
            if len(st[0]) > 96:
                continue
            if jit.code_object(st, groups, trunk) is not None:
                keys.add(f"{tree_row16.structure_key(*st, groups, trunk):016x}")
    return sorted(keys)


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    deps = [src] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    deps.append(os.path.join(HERE, "..", "include", "imhip.h"))
    if os.path.exists(obj) and not os.environ.get("IMHIP_REBUILD"):
        if os.path.getmtime(obj) > max(os.path.getmtime(d) for d in deps):
            return obj
    cmd = ["hipcc", *FLAGS, *os.environ.get("IMHIP_EXTRA_FLAGS", "").split(), "-c", "-x", "hip", src, "-o", obj]  # extra flags: development aid
    if os.path.dirname(src) != GEN:
        subprocess.run(cmd, check=True)
        return obj
    # a generated kernel: the compiler's resource remarks say whether it keeps to registers.  The
    # resident Newton kernels get fewer workgroups per CU, one at a time, while they spill.
    from .codegen import tree_row16

    import hashlib

    text = open(src).read()
    name, occ = tree_row16.occupancy_of(text)
    # the occupancy that an earlier build of the same source and headers settled on is tried first
    stamp = hashlib.sha256(text.encode())
    for d in sorted(deps[1:]):
        stamp.update(open(d, "rb").read())
    note = obj + ".nocc"
    first = occ
    if os.path.exists(note):
        saved = open(note).read().split()
        if len(saved) == 2 and saved[0] == stamp.hexdigest() and saved[1].isdigit():
            first = max(1, min(occ, int(saved[1])))
    for newton_occ in range(first, 0, -1):
        extra = [] if newton_occ == occ else [f"-DIM_NOCC_{name}={newton_occ}"]
        done = subprocess.run([*cmd, *extra, "-Rpass-analysis=kernel-resource-usage"], capture_output=True, text=True)
        if done.returncode != 0:
            sys.stderr.write(done.stderr)
            raise subprocess.CalledProcessError(done.returncode, cmd)
        spilling = _spilling_kernels(done.stderr, fused=True)
        if spilling:
            os.remove(obj)
            raise RuntimeError(f"{os.path.basename(src)}: fused kernels spill registers to memory: {spilling}")
        if not _spilling_kernels(done.stderr, fused=False):
            break
    with open(note, "w") as f:
        f.write(f"{stamp.hexdigest()} {newton_occ}\n")
    return obj


def _spilling_kernels(remarks: str, *, fused: bool) -> list[str]:
    """Kernels with a private segment, from the text of ``-Rpass-analysis=kernel-resource-usage``:
    the fused kernels (first template argument true), or the kernels built for the Newton
    occupancy (the resident Newton kernels and the solve-only kernel)."""
    import re

    out, name = [], None
    for line in remarks.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
        if not (m and name and int(m.group(1)) > 0):
            continue
        if ("tree_row16_" in name and "ILb1E" in name) if fused else ("newton_row16_" in name or ("tree_row16_" in name and "ILb0E" in name)):
            out.append(f"{name}: {m.group(1)} B/lane")
    return out


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
