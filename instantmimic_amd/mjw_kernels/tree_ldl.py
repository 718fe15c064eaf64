"""Tree-structured L'DL factor + solve of inertia-like matrices on MI355X.

Drop-in for the reference module ``instantmimic.utils.mjw_kernels.tree_ldl``
(src/instantmimic/utils/mjw_kernels/tree_ldl.py): same names, same arguments,
same eligibility decisions.  Planning is done by ``libimhip`` (host C++), the
numeric work by its HIP kernels; arrays are torch tensors on the GPU instead of
``wp.array``.  The extra entry :func:`assemble_tree_factor_solve` fuses the Newton
Hessian assembly ``H = M + J' diag(D active) J`` in front of the factorisation.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Any

import numpy as np

from .. import _lib

MAX_GROUPS = 4
MAX_SHARED_BYTES = 48 * 1024
MAX_SHORT_SPAN = 4096
MIN_DENSE_TO_SPAN_RATIO = 8.0
QUADRATIC = 1  # mjtConstraintState.mjCNSTRSTATE_QUADRATIC


@dataclass(frozen=True)
class TreeLdlPlan:
    """Same fields as the reference's ``TreeLdlPlan`` (tree_ldl.py:47-56)."""

    groups: tuple[tuple[int, ...], ...]
    trunk: tuple[int, ...]
    span: int
    dense_cost: int


class UnsupportedShape(RuntimeError):
    """The tree is valid but outside what the device kernels are built for."""


class _PlanHandle:
    """Owns one ``im_tree_plan``."""

    def __init__(self, structure, groups: int, host_only: bool):
        rowadr, rownnz, colind = (np.ascontiguousarray(a, dtype=np.int32) for a in structure)
        handle = C.c_void_p()
        status = _lib.lib().im_tree_plan_create(
            int(rowadr.size), rowadr.ctypes.data, rownnz.ctypes.data, colind.ctypes.data, int(colind.size),
            int(groups), 1 if host_only else 0, C.byref(handle),
        )  # fmt: skip
        _lib.check(status, "im_tree_plan_create")
        self.ptr = handle
        self.structure = tuple(tuple(int(v) for v in a) for a in (rowadr, rownnz, colind))

    def __del__(self):
        ptr, self.ptr = getattr(self, "ptr", None), None
        if ptr:
            try:
                _lib.lib().im_tree_plan_destroy(ptr)
            except Exception:
                pass

    def info(self) -> _lib.TreePlanInfo:
        info = _lib.TreePlanInfo()
        _lib.check(_lib.lib().im_tree_plan_get_info(self.ptr, C.byref(info)), "im_tree_plan_get_info")
        return info

    def arrays(self):
        info = self.info()
        gptr = np.zeros(info.ngroups + 1, np.int32)
        gdofs = np.zeros(max(info.nv - info.ntrunk, 1), np.int32)
        trunk = np.zeros(max(info.ntrunk, 1), np.int32)
        elim = np.zeros(info.nv, np.int32)
        _lib.check(
            _lib.lib().im_tree_plan_get_arrays(
                self.ptr, gptr.ctypes.data, gdofs.ctypes.data, trunk.ctypes.data, elim.ctypes.data
            ),
            "im_tree_plan_get_arrays",
        )
        return gptr, gdofs, trunk[: info.ntrunk], elim

    def plan(self) -> TreeLdlPlan:
        info = self.info()
        gptr, gdofs, trunk, _ = self.arrays()
        groups = tuple(tuple(int(v) for v in gdofs[gptr[j] : gptr[j + 1]]) for j in range(info.ngroups))
        return TreeLdlPlan(groups, tuple(int(v) for v in trunk), int(info.span), int(info.dense_cost))


@dataclass(frozen=True)
class TreeFactorSolveScratch:
    """Persistent, allocation-free state of one model's factor + solve."""

    kernel: Any  # the plan handle (the reference keeps a generated kernel here)
    groups: int
    cuda: bool
    plan: TreeLdlPlan


def _as_numpy(a) -> np.ndarray:
    if hasattr(a, "detach"):
        a = a.detach().cpu()
    if hasattr(a, "numpy"):
        a = a.numpy()
    return np.asarray(a)


def tree_ldl_structure(rowadr, rownnz, colind):
    """The CSR as tuples when it has the nested-ancestor form; else ``None``."""
    rowadr = np.ascontiguousarray(_as_numpy(rowadr), dtype=np.int64)
    rownnz = np.ascontiguousarray(_as_numpy(rownnz), dtype=np.int64)
    colind = np.ascontiguousarray(_as_numpy(colind), dtype=np.int64)
    nv = rowadr.size
    if nv == 0 or rownnz.size != nv:
        return None
    limit = np.iinfo(np.int32).max
    if max(rowadr.max(initial=0), rownnz.max(initial=0), colind.max(initial=0)) >= limit:
        return None
    r32, n32, c32 = (a.astype(np.int32) for a in (rowadr, rownnz, colind))
    status = _lib.lib().im_tree_structure_check(
        int(nv), r32.ctypes.data, n32.ctypes.data, c32.ctypes.data, int(c32.size)
    )
    if status == _lib.IM_ERR_STRUCTURE:
        return None
    _lib.check(status, "im_tree_structure_check")
    return tuple(int(v) for v in rowadr), tuple(int(v) for v in rownnz), tuple(int(v) for v in colind)


def plan_tree_ldl(rowadr, rownnz, colind, groups: int) -> TreeLdlPlan:
    """The plan with the shortest critical path for exactly ``groups`` groups."""
    return _PlanHandle((rowadr, rownnz, colind), groups, host_only=True).plan()


def best_tree_ldl_plan(rowadr, rownnz, colind) -> TreeLdlPlan:
    """The fastest plan whose trunk exchange fits 48 KB (fewest groups on ties)."""
    return _PlanHandle((rowadr, rownnz, colind), 0, host_only=True).plan()


def tree_ldl_beats_dense(plan: TreeLdlPlan) -> bool:
    return plan.span <= MAX_SHORT_SPAN or plan.dense_cost >= MIN_DENSE_TO_SPAN_RATIO * plan.span


def elimination_order(plan: TreeLdlPlan) -> tuple[int, ...]:
    """Dofs in elimination order: the groups in order, then the trunk descending."""
    return tuple(k for g in plan.groups for k in g) + tuple(reversed(plan.trunk))


def scratch_for_plan(structure, plan: TreeLdlPlan, device: Any) -> TreeFactorSolveScratch:
    import torch

    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError("the HIP tree L'DL runs on the GPU only (no CPU fallback)")
    with torch.cuda.device(dev):
        handle = _PlanHandle(structure, len(plan.groups), host_only=False)
    built = handle.plan()
    if built != plan:
        raise ValueError("plan does not belong to this structure")
    if not handle.info().device_ready:
        raise UnsupportedShape("shape outside the device kernels' limits (nv <= 96, nM <= 1024)")
    # straight-line kernels for this model, generated and compiled now unless the library has them
    from ..codegen import jit

    with torch.cuda.device(dev):
        attached = jit.attach(handle.ptr, handle.structure, plan.groups, plan.trunk)
    if not attached and handle.info().nv > 64:
        raise UnsupportedShape("more than 64 dofs run on generated kernels only, and none could be built")
    return TreeFactorSolveScratch(kernel=handle, groups=len(plan.groups), cuda=True, plan=plan)


def create_tree_factor_solve_scratch(m: Any, device: Any = None) -> TreeFactorSolveScratch | None:
    """The factor + solve for this model, or ``None`` when ineligible."""
    if getattr(m, "nv", 0) <= 0:
        return None
    arrays = [getattr(m, name, None) for name in ("M_rowadr", "M_rownnz", "M_colind")]
    if any(a is None for a in arrays):
        return None
    structure = tree_ldl_structure(*arrays)
    if structure is None:
        return None
    plan = best_tree_ldl_plan(*structure)
    if not tree_ldl_beats_dense(plan):
        return None
    if device is None:
        device = getattr(arrays[0], "device", None)
        if device is None or str(device) == "cpu":
            device = "cuda"
    try:
        return scratch_for_plan(structure, plan, device)
    except UnsupportedShape:
        return None


def _stream_ptr(tensor) -> int:
    import torch

    return int(torch.cuda.current_stream(tensor.device).cuda_stream)


def _check_rows(*tensors) -> None:
    # each world's row is indexed as a contiguous float run
    for t in tensors:
        if t.dim() != 2 or t.stride(1) != 1:
            raise ValueError("tree_factor_solve needs rows of contiguous floats")


def _check_against_plan(scratch, M, x, y, others=()) -> int:
    """Every array against the plan's sizes and against each other before a pointer leaves
    Python: the C ABI sees addresses and strides only.  Returns the world count."""
    info = scratch.kernel.info()
    nworld = int(M.shape[0])
    if M.shape[1] < info.nM or x.shape[1] < info.nv or y.shape[1] < info.nv:
        raise ValueError(f"rows shorter than the plan's sizes (nM {info.nM}, nv {info.nv})")
    for t in (x, y, *others):
        if t is not None and t.shape[0] != nworld:
            raise ValueError(f"{t.shape[0]} worlds where M has {nworld}")
    for t in (x, y, *others):
        if t is not None and t.device != M.device:
            raise ValueError("all arrays must live on one device")
    return nworld


def tree_factor_solve(scratch: TreeFactorSolveScratch, M, x, y) -> None:
    """x = M^-1 y for an M in the model's CSR layout (argument order of the
    reference: scratch, M, x, y)."""
    import torch

    _check_rows(M, x, y)
    for t in (M, x, y):
        if t.dtype != torch.float32 or not t.is_cuda:
            raise TypeError("tree_factor_solve needs float32 CUDA tensors")
    nworld = _check_against_plan(scratch, M, x, y)
    with torch.cuda.device(M.device):
        status = _lib.lib().im_tree_factor_solve(
            scratch.kernel.ptr, M.data_ptr(), M.stride(0), y.data_ptr(), y.stride(0), x.data_ptr(), x.stride(0),
            int(nworld), _stream_ptr(M),
        )  # fmt: skip
    _lib.check(status, "im_tree_factor_solve")


def assemble_tree_factor_solve(
    scratch: TreeFactorSolveScratch, M, J, D, state, nefc, grad, x, *, H_out=None, negate: bool = False,
    quad: int = QUADRATIC,
) -> None:  # fmt: skip
    """Fused Newton linear step on the tree pattern: ``H = M + J' diag(D [state ==
    quad]) J`` on M's CSR entries, L'DL, ``x = H^-1 grad`` (``-x`` with ``negate``).

    ``J`` (nworld, njmax, nv), ``D``/``state`` (nworld, njmax), ``nefc`` (nworld)
    int32 or ``None``; rows at or beyond ``nefc[w]`` are ignored.
    """
    import torch

    _check_rows(M, x, grad)
    if J.dim() != 3 or not J.is_contiguous() or not D.is_contiguous() or not state.is_contiguous():
        raise ValueError("J, D and state must be contiguous")
    if state.dtype != torch.int32 or (nefc is not None and nefc.dtype != torch.int32):
        raise TypeError("state and nefc must be int32")
    for t in (M, J, D, grad, x):
        if t.dtype != torch.float32 or not t.is_cuda:
            raise TypeError("assemble_tree_factor_solve needs float32 CUDA tensors")
    njmax, nv = int(J.shape[1]), int(J.shape[2])
    nworld = _check_against_plan(scratch, M, x, grad, (J, D, state, nefc, H_out))
    if nv != scratch.kernel.info().nv or njmax < 1:
        raise ValueError("J must be (nworld, njmax >= 1, nv) with the plan's nv")
    if tuple(D.shape) != (nworld, njmax) or tuple(state.shape) != (nworld, njmax) or (nefc is not None and nefc.numel() != nworld):
        raise ValueError("D and state must be (nworld, njmax), nefc (nworld,)")
    if H_out is not None and (not H_out.is_contiguous() or H_out.shape != (nworld, scratch.kernel.info().nM)):
        raise ValueError("H_out must be a contiguous (nworld, nM) tensor")
    with torch.cuda.device(M.device):
        status = _lib.lib().im_assemble_tree_ldl_solve(
            scratch.kernel.ptr, M.data_ptr(), M.stride(0), J.data_ptr(), int(njmax), D.data_ptr(), state.data_ptr(),
            nefc.data_ptr() if nefc is not None else None, int(quad), grad.data_ptr(), grad.stride(0), x.data_ptr(),
            x.stride(0), H_out.data_ptr() if H_out is not None else None, int(nworld),
            _lib.IM_FLAG_NEGATE if negate else 0, _stream_ptr(M),
        )  # fmt: skip
    _lib.check(status, "im_assemble_tree_ldl_solve")


def assemble_tree_factor_solve_iters(
    scratch: TreeFactorSolveScratch, M, J, D, states, nefc, grad, x, *, negate: bool = False, quad: int = QUADRATIC
) -> None:
    """``niter`` Newton linear steps that share ``M``, ``J`` and ``D``: ``states`` (niter, nworld,
    njmax) int32, ``x`` (niter, nworld, nv); ``grad`` is (nworld, nv) for one gradient or (niter,
    nworld, nv).  Same results as ``niter`` calls of :func:`assemble_tree_factor_solve``; one
    launch that reads ``M`` and ``J`` once where the library has a generated kernel for the tree."""
    import torch

    if states.dim() != 3 or x.dim() != 3 or states.shape[0] != x.shape[0]:
        raise ValueError("states must be (niter, nworld, njmax) and x (niter, nworld, nv)")
    niter = int(states.shape[0])
    grad0 = grad[0] if grad.dim() == 3 else grad
    if grad.dim() == 3 and grad.shape[0] != niter:
        raise ValueError("grad must be (nworld, nv) or (niter, nworld, nv)")
    _check_rows(M, x[0], grad0)
    if J.dim() != 3 or not J.is_contiguous() or not D.is_contiguous() or not states.is_contiguous():
        raise ValueError("J, D and states must be contiguous")
    if states.dtype != torch.int32 or (nefc is not None and nefc.dtype != torch.int32):
        raise TypeError("states and nefc must be int32")
    for t in (M, J, D, grad, x):
        if t.dtype != torch.float32 or not t.is_cuda:
            raise TypeError("assemble_tree_factor_solve_iters needs float32 CUDA tensors")
    njmax, nv = int(J.shape[1]), int(J.shape[2])
    nworld = _check_against_plan(scratch, M, x[0], grad0, (J, D, states[0], nefc))
    if nv != scratch.kernel.info().nv or njmax < 1:
        raise ValueError("J must be (nworld, njmax >= 1, nv) with the plan's nv")
    if tuple(D.shape) != (nworld, njmax) or tuple(states.shape[1:]) != (nworld, njmax) or (nefc is not None and nefc.numel() != nworld):
        raise ValueError("D must be (nworld, njmax), states (niter, nworld, njmax), nefc (nworld,)")
    if x.stride(2) != 1 or (grad.dim() == 3 and grad.stride(2) != 1):
        raise ValueError("rows of x and grad must be contiguous floats")
    with torch.cuda.device(M.device):
        status = _lib.lib().im_assemble_tree_ldl_solve_iters(
            scratch.kernel.ptr, M.data_ptr(), M.stride(0), J.data_ptr(), njmax, D.data_ptr(), states.data_ptr(),
            states.stride(0), nefc.data_ptr() if nefc is not None else None, int(quad), grad.data_ptr(),
            grad0.stride(0), grad.stride(0) if grad.dim() == 3 else 0, x.data_ptr(), x.stride(1), x.stride(0),
            int(nworld), niter, _lib.IM_FLAG_NEGATE if negate else 0, _stream_ptr(M),
        )  # fmt: skip
    _lib.check(status, "im_assemble_tree_ldl_solve_iters")


def pattern_violations(scratch: TreeFactorSolveScratch, J, D, state, nefc, violations, *, quad: int = QUADRATIC) -> None:
    """Adds to ``violations`` (nworld,) float32 the number of active constraint rows of every world
    whose dofs do not lie on one root-to-leaf chain: rows the fused tree solve cannot represent
    (their products outside M's pattern are dropped).  The counter accumulates, like the
    reference's ``violation_counter`` (sparse_hessian.py:786-796); zero it after a nonzero read."""
    import torch

    if J.dim() != 3 or not J.is_contiguous() or not D.is_contiguous() or not state.is_contiguous():
        raise ValueError("J, D and state must be contiguous")
    nworld, njmax, nv = (int(v) for v in J.shape)
    if nv != scratch.kernel.info().nv or tuple(D.shape) != (nworld, njmax) or tuple(state.shape) != (nworld, njmax):
        raise ValueError("J, D and state do not match the plan or each other")
    if violations.dtype != torch.float32 or violations.numel() != nworld or not violations.is_contiguous():
        raise TypeError("violations must be a contiguous float32 tensor with one element per world")
    if state.dtype != torch.int32 or (nefc is not None and (nefc.dtype != torch.int32 or nefc.numel() != nworld)):
        raise TypeError("state and nefc must be int32, nefc one element per world")
    with torch.cuda.device(J.device):
        status = _lib.lib().im_tree_pattern_violations(
            scratch.kernel.ptr, J.data_ptr(), njmax, D.data_ptr(), state.data_ptr(),
            nefc.data_ptr() if nefc is not None else None, int(quad), violations.data_ptr(), nworld, _stream_ptr(J),
        )  # fmt: skip
    _lib.check(status, "im_tree_pattern_violations")
