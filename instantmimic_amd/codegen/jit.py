"""Generated tree kernels for models the library was not built with: source from
:mod:`tree_row16` (module form), compiled to a gfx950 code object with ``hipcc --genco`` and
handed to ``im_tree_plan_attach_kernels``.  The reference does the same when it creates a model's
scratch (src/instantmimic/utils/mjw_kernels/tree_ldl.py:393-416: straight-line code for the
model, compiled by Warp at first use).  Code objects are kept on disk under their 64-bit
structure key, so a model is compiled once (a few seconds).

``IMHIP_TREE_JIT=0`` turns this off (plans then run the table-driven kernel);
``IMHIP_KERNEL_CACHE`` names the directory (default: ``_obj/kernels`` beside the library, else
``~/.cache/instantmimic_amd``; a directory owned by another user is never used)."""

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
    ]
    for path in choices:
        try:
            os.makedirs(path, mode=0o700, exist_ok=True)
            # code objects are loaded into the GPU as they are: only a directory of this user's own
            if os.access(path, os.W_OK) and os.stat(path).st_uid == os.getuid():
                return path
        except OSError:
            continue
    raise OSError("no writable directory of this user's own for generated kernels (set IMHIP_KERNEL_CACHE)")


def _source_tag() -> str:
    """Changes whenever the generator, the header the kernels include, the compiler flags or one
    of the environment knobs that alter the generated source changes: a code object built under
    one setting is never loaded under another."""
    h = hashlib.sha256()
    for path in (os.path.join(_HERE, "tree_row16.py"), os.path.join(_CSRC, "tree_row16.h")):
        with open(path, "rb") as f:
            h.update(f.read())
    h.update("\0".join(FLAGS).encode())
    for knob in tree_row16.SOURCE_KNOBS:
        h.update(f"\0{knob}={os.environ.get(knob, '')}".encode())
    return h.hexdigest()[:12]


def kernel_resources(blob: bytes) -> dict[str, tuple[int, int]]:
    """{kernel name: (LDS bytes, private-segment bytes per lane)} of a gfx9 code object, read from
    the kernel descriptors (the 64-byte ``<name>.kd`` objects: group segment size at byte 0,
    private segment size at byte 4).  Takes the ELF itself or clang's offload bundle around it."""
    import struct

    start = blob.find(b"\x7fELF")
    if start < 0:
        raise ValueError("no ELF image in the code object")
    elf = memoryview(blob)[start:]
    if elf[4] != 2 or elf[5] != 1:
        raise ValueError("not a little-endian ELF64 image")
    shoff, = struct.unpack_from("<Q", elf, 0x28)
    shentsize, shnum, _ = struct.unpack_from("<HHH", elf, 0x3A)
    sections = [struct.unpack_from("<IIQQQQIIQQ", elf, shoff + i * shentsize) for i in range(shnum)]
    out = {}
    for _, kind, _, _, offset, size, link, _, _, entsize in sections:
        if kind not in (2, 11) or entsize == 0:  # SHT_SYMTAB, SHT_DYNSYM
            continue
        strtab = sections[link]
        for k in range(size // entsize):
            name_off, _, _, shndx, value, _ = struct.unpack_from("<IBBHQQ", elf, offset + k * entsize)
            end = bytes(elf[strtab[4] + name_off : strtab[4] + name_off + 256]).split(b"\0", 1)[0]
            if not end.endswith(b".kd") or shndx == 0 or shndx >= shnum:
                continue
            home = sections[shndx]
            at = home[4] + (value - home[3])
            lds, private = struct.unpack_from("<II", elf, at)
            out[end[:-3].decode()] = (int(lds), int(private))
    return out


def spilling_kernels(blob: bytes) -> list[str]:
    """The fused kernels of a code object that use a private segment (register spills to memory)."""
    return sorted(name for name, (_, private) in kernel_resources(blob).items() if private and name in ("im_row16_fused", "im_row16_fused_long"))


def code_object(structure, groups, trunk) -> bytes | None:
    """The code object of a (structure, plan), from the cache or freshly compiled; ``None`` when no
    compiler is at hand, when the generator declines the plan, when the compiler fails on the
    generated source, or when a fused kernel came out with register spills to memory (no such
    kernel is handed to the library; the plan then keeps the table-driven kernel)."""
    key = tree_row16.structure_key(*structure, groups, trunk)
    path = os.path.join(cache_dir(), f"tree_row16_{key:016x}_{_source_tag()}.co")
    if os.path.exists(path):
        with open(path, "rb") as f:
            blob = f.read()
        return None if not blob or spilling_kernels(blob) else blob
    hipcc = shutil.which("hipcc") or ("/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else None)
    if hipcc is None:
        return None
    try:
        src = tree_row16.generate(f"k{key:016x}", *structure, groups, trunk, module=True)
    except tree_row16.Declined:
        return None
    with tempfile.TemporaryDirectory(prefix="imhip_jit_") as tmp:
        hip, out = os.path.join(tmp, "kernel.hip"), os.path.join(tmp, "kernel.co")
        with open(hip, "w") as f:
            f.write(src)
        done = subprocess.run([hipcc, *FLAGS, "-I", _CSRC, "-x", "hip", hip, "-o", out], capture_output=True)
        if done.returncode != 0 or not os.path.exists(out):
            import warnings

            warnings.warn(f"hipcc failed on the generated tree kernel {key:016x}: {done.stderr.decode(errors='replace')[-400:]}")
            return None
        with open(out, "rb") as f:
            blob = f.read()
    tmp_path = f"{path}.{os.getpid()}.tmp"
    with open(tmp_path, "wb") as f:
        f.write(blob)
    os.replace(tmp_path, path)  # whole files only, also with several processes at once
    return None if spilling_kernels(blob) else blob


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
