"""The per-iteration factor stage of the Newton loop on MI355X: incremental Hessian update
over the changed constraint rows, then refactor or solve-only.

Drop-in for ``factor_factory`` of the reference
(src/instantmimic/utils/mjw_kernels/newton_stages.py:614-742): with a sparse plan the
static-pattern L'DL stage (native modes of sparse_hessian.py:488-547), without one the
dense update and the augmented blocked Cholesky of ``augmented_factor_solve_factory``
(:473-611).  The reference inlines the stage into one resident kernel per world; here it is
one launch per iteration and the factor is carried in ``hfactor`` / ``U`` between launches.
"""

from __future__ import annotations

from typing import Any

from .. import _lib
from .sparse_hessian import QUADRATIC, SparseHessianPlan


def _check(tensors, nworld: int) -> None:
    for name, t in tensors.items():
        if t is None:
            continue
        if not t.is_cuda or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous CUDA tensor")
        if t.shape[0] != nworld:
            raise ValueError(f"{name} has {t.shape[0]} worlds, expected {nworld}")


def factor_factory(nv: int, pad: int, sparse_plan: SparseHessianPlan | None = None, *, tree_scratch: Any = None,
                   block: int = 32):
    """Launcher ``kernel(J, D, state, ids, changes, state_changes, done, grad, H, U, search,
    search_dot, decrement, dof_union)`` with the reference kernel's arrays: ids (nworld, njmax)
    changed rows, changes / state_changes (nworld,), grad and search (nworld, nv_pad) or
    (nworld, nv_pad, 1), H and U (nworld, nv_pad, nv_pad), dof_union (nworld, nv + 1).  With a
    sparse plan ``U`` is the hfactor buffer and ``H`` is not touched.

    ``tree_scratch`` (a scratch of ``tree_ldl.create_tree_factor_solve_scratch``; the reference
    has no such stage) selects the stage on the kinematic tree for models whose constraint rows
    stay on single root-to-leaf chains: the Hessian is assembled afresh on M's pattern and solved
    by the tree L'DL, nothing is carried from one iteration to the next, and ``H``, ``U``, ``ids``
    and ``dof_union`` are not touched.  Its launcher also takes ``M=`` (d.M), ``nefc=`` and
    ``skip=`` (ctx.search_unchanged, the bytes the gradient leaves: done or no state change);
    ``block`` is the lane count whose summation order the two dot products follow."""
    import torch

    if tree_scratch is not None:
        if sparse_plan is not None:
            raise ValueError("a sparse plan and a tree scratch: choose one factor stage")
        if not getattr(tree_scratch, "cuda", False) or tree_scratch.kernel.info().nv != nv:
            raise ValueError("the tree scratch belongs to another model or has no device state")

        def tree_kernel(J, D, state, ids, changes, state_changes, done, grad, H, U, search, search_dot, decrement,
                        dof_union, *, M, nefc=None, skip, quad: int = QUADRATIC) -> None:  # fmt: skip
            nworld, njmax, nvj = J.shape
            if nvj != nv:
                raise ValueError("J does not match the stage's nv")
            _check(dict(J=J, D=D, state=state, grad=grad, search=search, search_dot=search_dot, decrement=decrement,
                        M=M, skip=skip, nefc=nefc), nworld)  # fmt: skip
            if skip.dtype not in (torch.bool, torch.uint8):
                raise TypeError("skip must be a bool tensor")
            if M.dim() != 2 or M.shape[1] < tree_scratch.kernel.info().nM:
                raise ValueError("M must be (nworld, nM)")
            ldg, lds = grad[0].numel(), search[0].numel()
            with torch.cuda.device(J.device):
                status = _lib.lib().im_newton_tree_stage(
                    tree_scratch.kernel.ptr, skip.data_ptr(), M.data_ptr(), M.stride(0), J.data_ptr(), int(njmax),
                    D.data_ptr(), state.data_ptr(), None if nefc is None else nefc.data_ptr(), int(quad), grad.data_ptr(),
                    int(ldg), search.data_ptr(), int(lds), search_dot.data_ptr(), decrement.data_ptr(), int(block),
                    int(nworld), int(torch.cuda.current_stream(J.device).cuda_stream),
                )  # fmt: skip
            _lib.check(status, "im_newton_tree_stage")

        return tree_kernel

    if sparse_plan is not None:
        if sparse_plan.handle is None:
            raise RuntimeError("the plan has no device state (build it with device=...)")
        if sparse_plan.nv != nv or sparse_plan.nv_pad != pad:
            raise ValueError("the plan was built for another model size")

    def kernel(J, D, state, ids, changes, state_changes, done, grad, H, U, search, search_dot, decrement, dof_union,
               *, quad: int = QUADRATIC) -> None:  # fmt: skip
        nworld, njmax, nvj = J.shape
        if nvj != nv:
            raise ValueError("J does not match the stage's nv")
        _check(dict(J=J, D=D, state=state, ids=ids, changes=changes, state_changes=state_changes, done=done,
                    grad=grad, U=U, search=search, search_dot=search_dot, decrement=decrement,
                    dof_union=dof_union), nworld)  # fmt: skip
        if tuple(U.shape) != (nworld, pad, pad) or tuple(dof_union.shape) != (nworld, nv + 1):
            raise ValueError("U must be (nworld, nv_pad, nv_pad) and dof_union (nworld, nv + 1)")
        if ids.dtype != torch.int32 or dof_union.dtype != torch.int32 or changes.dtype != torch.int32:
            raise TypeError("ids, changes and dof_union must be int32")
        if done is not None and done.dtype not in (torch.bool, torch.uint8):
            raise TypeError("done must be a bool tensor")
        ldg, lds = grad[0].numel(), search[0].numel()
        stream = int(torch.cuda.current_stream(J.device).cuda_stream)
        done_ptr = None if done is None else done.data_ptr()
        L = _lib.lib()
        with torch.cuda.device(J.device):
            if sparse_plan is not None:
                if lds != nv:
                    raise ValueError("search must be (nworld, nv) on the sparse path")
                status = L.im_sparse_update_factor(
                    sparse_plan.ptr, done_ptr, state_changes.data_ptr(), changes.data_ptr(), ids.data_ptr(),
                    int(ids.shape[1]), J.data_ptr(), int(njmax), D.data_ptr(), state.data_ptr(), int(quad),
                    grad.data_ptr(), int(ldg), U.data_ptr(), dof_union.data_ptr(), search.data_ptr(),
                    search_dot.data_ptr(), decrement.data_ptr(), int(nworld), stream,
                )  # fmt: skip
                _lib.check(status, "im_sparse_update_factor")
            else:
                _check(dict(H=H), nworld)
                if tuple(H.shape) != (nworld, pad, pad):
                    raise ValueError("H must be (nworld, nv_pad, nv_pad)")
                status = L.im_dense_update_factor(
                    done_ptr, state_changes.data_ptr(), changes.data_ptr(), ids.data_ptr(), int(ids.shape[1]),
                    J.data_ptr(), int(njmax), D.data_ptr(), state.data_ptr(), int(quad), grad.data_ptr(), int(ldg),
                    H.data_ptr(), U.data_ptr(), int(nv), int(pad), dof_union.data_ptr(), search.data_ptr(), int(lds),
                    search_dot.data_ptr(), decrement.data_ptr(), int(nworld), stream,
                )  # fmt: skip
                _lib.check(status, "im_dense_update_factor")

    return kernel
