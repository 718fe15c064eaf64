"""Generated tree kernels for models the library was not built with: source from
:mod:`tree_row16` (module form), compiled to a gfx950 code object with ``hipcc --genco`` and
handed to ``im_tree_plan_attach_kernels``.  The reference does the same when it creates a model's
scratch (src/instantmimic/utils/mjw_kernels/tree_ldl.py:393-416: straight-line code for the
model, compiled by Warp at first use).  Code objects are kept on disk under their 64-bit
structure key, so a model is compiled once (a few seconds).

``IMHIP_TREE_JIT=0`` turns this off (plans then run the table-driven kernel);
``IMHIP_KERNEL_CACHE`` names the directory (default: ``_obj/kernels`` beside the library, else
``~/.cache/instantmimic_amd``, else the temporary directory)."""

from __future__ import annotations

import ctypes as C
import hashlib
import os
import shutil
import subprocess
import tempfile

from .. import _lib
from . import tree_row16

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_HERE, "..", "csrc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-fno-fast-math", "-Xclang", "-target-feature",
         "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", "--genco"]  # fmt: skip


def enabled() -> bool:
    # IMHIP_TREE_KERNEL=generic asks for the table-driven kernel: nothing to generate then
    return os.environ.get("IMHIP_TREE_JIT", "1") != "0" and os.environ.get("IMHIP_TREE_KERNEL") != "generic"


def cache_dir() -> str:
    named = os.environ.get("IMHIP_KERNEL_CACHE")
    choices = [named] if named else [
        os.path.join(_HERE, "..", "_obj", "kernels"),
        os.path.join(os.path.expanduser("~"), ".cache", "instantmimic_amd"),
        os.path.join(tempfile.gettempdir(), "instantmimic_amd_kernels"),
    ]
    for path in choices:
        try:
            os.makedirs(path, exist_ok=True)
            if os.access(path, os.W_OK):
                return path
        except OSError:
            continue
    raise OSError("no writable directory for generated kernels")


def _source_tag() -> str:
    """Changes whenever the generator or the header the kernels include changes."""
    h = hashlib.sha256()
    for path in (os.path.join(_HERE, "tree_row16.py"), os.path.join(_CSRC, "tree_row16.h")):
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:12]


def code_object(structure, groups, trunk) -> bytes | None:
    """The code object of a (structure, plan), from the cache or freshly compiled; ``None`` when no
    compiler is at hand."""
    key = tree_row16.structure_key(*structure, groups, trunk)
    path = os.path.join(cache_dir(), f"tree_row16_{key:016x}_{_source_tag()}.co")
    if os.path.exists(path):
        with open(path, "rb") as f:
            return f.read()
    hipcc = shutil.which("hipcc") or ("/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else None)
    if hipcc is None:
        return None
    if any(len(g) == 0 for g in groups):
        return None  # a plan with an empty group: the table-driven kernel serves it
    src = tree_row16.generate(f"k{key:016x}", *structure, groups, trunk, module=True)
    with tempfile.TemporaryDirectory(prefix="imhip_jit_") as tmp:
        hip, out = os.path.join(tmp, "kernel.hip"), os.path.join(tmp, "kernel.co")
        with open(hip, "w") as f:
            f.write(src)
        subprocess.run([hipcc, *FLAGS, "-I", _CSRC, "-x", "hip", hip, "-o", out], check=True, capture_output=True)
        with open(out, "rb") as f:
            blob = f.read()
    tmp_path = f"{path}.{os.getpid()}.tmp"
    with open(tmp_path, "wb") as f:
        f.write(blob)
    os.replace(tmp_path, path)  # whole files only, also with several processes at once
    return blob


def attach(plan_ptr, structure, groups, trunk) -> bool:
    """Gives a device-ready plan generated kernels unless it has them already; False when it keeps
    the table-driven kernel (generation off, no compiler, or a shape the generator does not take)."""
    key, has = C.c_ulonglong(0), C.c_int(0)
    _lib.check(_lib.lib().im_tree_plan_kernel_key(plan_ptr, C.byref(key), C.byref(has)), "im_tree_plan_kernel_key")
    if has.value:
        return True
    if not enabled() or len(structure[0]) > 96:
        return False
    if key.value != tree_row16.structure_key(*structure, groups, trunk):
        raise RuntimeError("the generator's structure key differs from the library's")
    blob = code_object(structure, groups, trunk)
    if blob is None:
        return False
    buf = C.create_string_buffer(blob, len(blob))
    status = _lib.lib().im_tree_plan_attach_kernels(plan_ptr, buf)
    if status == _lib.IM_ERR_UNSUPPORTED:
        return False
    _lib.check(status, "im_tree_plan_attach_kernels")
    return True
