"""Generated tree kernels for models the library was not built with: source from
:mod:`tree_row16` (module form), compiled to a gfx950 code object inside this process through
``libhiprtc`` (or, where that library is missing or fails, by a ``hipcc --genco`` subprocess) and
handed to ``im_tree_plan_attach_kernels``.  The reference does the same when it creates a model's
scratch (src/instantmimic/utils/mjw_kernels/tree_ldl.py:393-416: straight-line code for the
model, compiled by Warp at first use).  Code objects are kept on disk under their 64-bit
structure key, so a model is compiled once (a few seconds).

``IMHIP_TREE_JIT=0`` turns this off (plans then run the table-driven kernel);
``IMHIP_JIT_COMPILER=hiprtc`` or ``hipcc`` allows only that one of the two compilers;
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
COMMON_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-fno-fast-math", "-Xclang",
                "-target-feature", "-Xclang", "-packed-fp32-ops"]  # fmt: skip
FLAGS = COMMON_FLAGS + ["-Wno-unused-command-line-argument", "--genco"]  # the subprocess's


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
    """Changes whenever the generator, a header the kernels may include, the compiler flags or one
    of the environment knobs that alter the generated source changes: a code object built under
    one setting is never loaded under another."""
    h = hashlib.sha256()
    headers = sorted(os.path.join(_CSRC, name) for name in os.listdir(_CSRC) if name.endswith(".h"))
    for path in (os.path.join(_HERE, "tree_row16.py"), *headers):
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


def _rocm_root() -> str:
    return os.environ.get("ROCM_PATH") or "/opt/rocm"


_HIPRTC = None


def _hiprtc():
    """libhiprtc, loaded once; ``None`` where there is none."""
    global _HIPRTC
    if _HIPRTC is None:
        _HIPRTC = False
        for name in ("libhiprtc.so", os.path.join(_rocm_root(), "lib", "libhiprtc.so")):
            try:
                lib = C.CDLL(name)
            except OSError:
                continue
            lib.hiprtcCreateProgram.argtypes = [C.POINTER(C.c_void_p), C.c_char_p, C.c_char_p, C.c_int, C.c_void_p, C.c_void_p]
            lib.hiprtcCompileProgram.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_char_p)]
            lib.hiprtcGetProgramLogSize.argtypes = lib.hiprtcGetCodeSize.argtypes = [C.c_void_p, C.POINTER(C.c_size_t)]
            lib.hiprtcGetProgramLog.argtypes = lib.hiprtcGetCode.argtypes = [C.c_void_p, C.c_char_p]
            lib.hiprtcDestroyProgram.argtypes = [C.POINTER(C.c_void_p)]
            _HIPRTC = lib
            break
    return _HIPRTC or None


def compile_hiprtc(src: str, label: str, defines: tuple[str, ...] = ()) -> bytes | None:
    """The code object of ``src`` from the run-time compiler inside this process; ``None`` (with a
    warning that carries the compiler's log) when the library is missing or the compile fails."""
    import warnings

    rtc = _hiprtc()
    if rtc is None:
        return None
    prog = C.c_void_p()
    if rtc.hiprtcCreateProgram(C.byref(prog), src.encode(), f"tree_row16_{label}.hip".encode(), 0, None, None) != 0:
        return None
    try:
        # the generated source includes this package's headers, which include HIP's by name
        options = [o.encode() for o in COMMON_FLAGS + ["-I" + os.path.abspath(_CSRC), "-I" + os.path.join(_rocm_root(), "include"), *defines]]
        status = rtc.hiprtcCompileProgram(prog, len(options), (C.c_char_p * len(options))(*options))
        if status != 0:
            n = C.c_size_t(0)
            rtc.hiprtcGetProgramLogSize(prog, C.byref(n))
            log = C.create_string_buffer(n.value + 1)
            rtc.hiprtcGetProgramLog(prog, log)
            warnings.warn(f"hiprtc failed on the generated tree kernel {label}: {log.value.decode(errors='replace')[-400:]}")
            return None
        n = C.c_size_t(0)
        if rtc.hiprtcGetCodeSize(prog, C.byref(n)) != 0 or n.value == 0:
            return None
        code = C.create_string_buffer(n.value)
        if rtc.hiprtcGetCode(prog, code) != 0:
            return None
        return code.raw
    finally:
        rtc.hiprtcDestroyProgram(C.byref(prog))


def compile_hipcc(src: str, label: str, defines: tuple[str, ...] = ()) -> bytes | None:
    """The same from a ``hipcc --genco`` subprocess; ``None`` without a compiler or when it fails."""
    hipcc = shutil.which("hipcc") or next((p for p in (os.path.join(_rocm_root(), "bin", "hipcc"),) if os.path.exists(p)), None)
    if hipcc is None:
        return None
    with tempfile.TemporaryDirectory(prefix="imhip_jit_") as tmp:
        hip, out = os.path.join(tmp, "kernel.hip"), os.path.join(tmp, "kernel.co")
        with open(hip, "w") as f:
            f.write(src)
        done = subprocess.run([hipcc, *FLAGS, *defines, "-I", _CSRC, "-x", "hip", hip, "-o", out], capture_output=True)
        if done.returncode != 0 or not os.path.exists(out):
            import warnings

            warnings.warn(f"hipcc failed on the generated tree kernel {label}: {done.stderr.decode(errors='replace')[-400:]}")
            return None
        with open(out, "rb") as f:
            return f.read()


def compile_source(src: str, label: str) -> bytes | None:
    """In this process first, a compiler subprocess second; ``IMHIP_JIT_COMPILER`` names the only one to try."""
    only = os.environ.get("IMHIP_JIT_COMPILER", "")
    if only not in ("", "hiprtc", "hipcc"):
        raise ValueError("IMHIP_JIT_COMPILER is hiprtc or hipcc")

    def once(defines):
        blob = compile_hiprtc(src, label, defines) if only in ("", "hiprtc") else None
        if blob is None and only in ("", "hipcc"):
            blob = compile_hipcc(src, label, defines)
        return blob

    blob = once(())
    if blob is None:
        return None
    # The resident Newton kernels carry the loop's state on top of the stage's rows.  Where they
    # spill at the fused kernels' occupancy, one more compile gives them a workgroup per CU less;
    # if they still spill the library leaves them unused (the iterations are then stage launches).
    name, occ = tree_row16.occupancy_of(src)
    newton = ("im_row16_newton", "im_row16_newton_long", "im_row16_solve")  # the kernels built for IM_NOCC
    if occ > 1 and any(kernel_resources(blob).get(k, (0, 0))[1] for k in newton):
        again = once((f"-DIM_NOCC_{name}={occ - 1}",))
        if again is not None and sum(kernel_resources(again).get(k, (0, 0))[1] for k in newton) < sum(kernel_resources(blob).get(k, (0, 0))[1] for k in newton):
            blob = again
    return blob


def code_object(structure, groups, trunk) -> bytes | None:
    """The code object of a (structure, plan), from the cache or freshly compiled; ``None`` when
    neither compiler is at hand, when the generator declines the plan, when the compiler fails on the
    generated source, or when a fused kernel came out with register spills to memory (no such
    kernel is handed to the library; the plan then keeps the table-driven kernel)."""
    key = tree_row16.structure_key(*structure, groups, trunk)
    path = os.path.join(cache_dir(), f"tree_row16_{key:016x}_{_source_tag()}.co")
    if os.path.exists(path):
        with open(path, "rb") as f:
            blob = f.read()
        return None if not blob or spilling_kernels(blob) else blob
    try:
        src = tree_row16.generate(f"k{key:016x}", *structure, groups, trunk, module=True)
    except tree_row16.Declined:
        return None
    blob = compile_source(src, f"{key:016x}")
    if blob is None:
        return None
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
