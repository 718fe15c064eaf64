"""The reference's fused Newton solve on MI355X: ``init_context``, ``run`` and the force recovery.

:func:`solve` is the constraint solve as the reference's step issues it
(src/instantmimic/utils/mjw_step_optimized.py:2588-2683): :func:`init_context`
(src/instantmimic/utils/mjw_kernels/newton_fusion.py:431-519, with ``_update_gradient_sparse``,
:480-519), :func:`run` (:330-409) and :func:`qfrc_constraint_from_grad` (:537-555).  Nothing in
it reads device memory back while the caller's stream is being captured, so a whole solve can be
one graph of the caller's.

:func:`run` takes one of two forms.  Where the context's scratch allows it, the iterations are one
resident kernel per solve with a wavefront per world, the reference's persistent block
(:57-298): ``im_newton_solve_tree`` (fused tree stage, plans with generated kernels) or
``im_newton_solve_sparse`` (static-pattern sparse stage).  Otherwise every iteration is eight
launches over all worlds (:func:`iteration`), each kernel returning for worlds that are done.

The stages are also callable by themselves.  :func:`mul_m` is the product ``M v`` (:171-176)
from the three tables of the upstream model (``m.M_mulm_rowadr``, ``m.M_mulm_col``,
``m.M_mulm_madr``, :378-380); :func:`mul_m_tables` builds them from the CSR for a model that does
not carry them (ancestors root first, the diagonal, then descendants ascending -- the upstream
order is not visible from the reference's tree).  :func:`gradient` is ``gradient_function``
(src/instantmimic/utils/mjw_kernels/newton_stages.py:745-798), :func:`jv` the ``J v`` step at the
head of the line search (:157-178), :func:`linesearch` its scalar search (:179-372),
:func:`advance` the step at its end (:373-381), :func:`eval_constraints` the constraints' new
forces and states (:385-444), :func:`changed_rows` the listing of the rows whose state changed
(:403-426), :func:`converged` the test that closes an iteration (newton_fusion.py:265-296),
:func:`init_empty_worlds` the kernel at the start of the solve (:412-428).  The per-row cost of
the line search and the constraint re-evaluation are upstream mujoco_warp functions that the
reference's tree does not hold; they are restated from MuJoCo's published primal line search.
"""

from __future__ import annotations

import os
from typing import Any

import numpy as np

from .. import _lib


# mujoco_warp's enums are not importable here; members are matched by name when the model
# carries enum objects and by MuJoCo's published integer values otherwise (mjtSolver: NEWTON = 2;
# mjtCone: PYRAMIDAL = 0; the DISCRETE integrator is an addition of the reference's mujoco_warp
# build and is matched by name only).
SOLVER_NEWTON = 2
CONE_PYRAMIDAL = 0


def _is_member(value, name: str, number) -> bool:
    label = getattr(value, "name", None)
    if label is not None:
        return str(label).upper() == name
    return number is not None and value is not None and int(value) == number


def _sparse_compact(ctx) -> bool:
    return bool(getattr(ctx, "sparse_compact", False)) if ctx is not None else False


def _option_gates(m) -> bool:
    """Newton solver with a positive iteration budget, pyramidal cone, not the DISCRETE
    integrator; a model without ``opt`` does not qualify."""
    opt = getattr(m, "opt", None)
    if opt is None:
        return False
    return (
        _is_member(getattr(opt, "solver", None), "NEWTON", SOLVER_NEWTON)
        and _is_member(getattr(opt, "cone", None), "PYRAMIDAL", CONE_PYRAMIDAL)
        and not _is_member(getattr(opt, "integrator", None), "DISCRETE", None)
        and int(getattr(opt, "iterations", 0)) > 0
    )


def eligible(m, ctx, *, compact: bool = False, device="cuda") -> bool:
    """Whether the fused Newton takes the model: ``eligible`` of the reference
    (src/instantmimic/utils/mjw_kernels/newton_fusion.py:307-322).  Fields the reference reads
    from the uploaded model are read from ``m`` and a missing one disqualifies.  Upstream's
    ``_use_incremental`` is taken as "Newton solver" (the gate the reference itself mirrors in
    src/instantmimic/utils/mjw_model.py:95-102) unless the model states ``use_incremental``;
    ``_sparse_compact`` is read from ``ctx.sparse_compact``.  ``device=None`` stands for
    planning on the host for a GPU run."""
    arr = getattr(m, "body_parentid", None)
    where = None if isinstance(arr, np.ndarray) else getattr(arr, "device", None)  # NumPy copies say nothing
    if where is not None:
        on_gpu = bool(getattr(where, "is_cuda", False) or getattr(where, "type", "") == "cuda")
    else:
        on_gpu = device is None or str(device).startswith("cuda")
    nv, nv_pad = int(m.nv), int(getattr(m, "nv_pad", 0))
    incremental = getattr(m, "use_incremental", None)
    if incremental is None:
        incremental = _is_member(getattr(getattr(m, "opt", None), "solver", None), "NEWTON", SOLVER_NEWTON)
    width = getattr(getattr(m, "block_dim", None), "linesearch_iterative", None)
    return bool(
        not compact
        and on_gpu
        and 0 < nv <= 79
        and nv_pad % 16 == 0
        and 0 < nv_pad <= 80
        and incremental
        and _option_gates(m)
        and getattr(m, "is_sparse", None) is False
        and not _sparse_compact(ctx)
        and width == 32
    )


def upstream_newton_structure(m, ctx, *, compact: bool = False) -> bool:
    """The gate of the upstream (non-fused) iteration with the sparse factor substituted
    (src/instantmimic/utils/mjw_kernels/sparse_hessian.py:738-746)."""
    hfactor = getattr(ctx, "hfactor", None) if ctx is not None else None
    return bool(
        _option_gates(m)
        and not compact
        and not _sparse_compact(ctx)
        and hfactor is not None
        and len(hfactor.shape) > 1
        and int(hfactor.shape[1]) == int(getattr(m, "nv_pad", -1))
    )


def newton_block_dim(m) -> int:
    """Physical Newton block width (newton_fusion.py:325-327)."""
    return 64 if int(m.nv_pad) >= 64 else int(m.block_dim.linesearch_iterative)


def mul_m_tables(rowadr, rownnz, colind):
    """(mulm_rowadr[nv + 1], mulm_col, mulm_madr) int32 for M's CSR (row = ancestors root
    first, diagonal last)."""
    rowadr, rownnz, colind = (np.asarray(a, np.int64) for a in (rowadr, rownnz, colind))
    nv = rowadr.size
    rows: list[list[tuple[int, int]]] = [[] for _ in range(nv)]
    for i in range(nv):
        for k in range(rowadr[i], rowadr[i] + rownnz[i]):
            rows[i].append((int(colind[k]), int(k)))
    for i in range(nv):  # descendants ascending: row i's off-diagonal entries mirrored
        for k in range(rowadr[i], rowadr[i] + rownnz[i] - 1):
            rows[int(colind[k])].append((i, int(k)))
    out_adr = np.zeros(nv + 1, np.int32)
    out_adr[1:] = np.cumsum([len(r) for r in rows])
    col = np.array([c for r in rows for c, _ in r], np.int32)
    madr = np.array([a for r in rows for _, a in r], np.int32)
    return out_adr, col, madr


def mul_m(M, vec, out, mulm_rowadr, mulm_col, mulm_madr, *, skip_world: Any = None) -> None:
    """``out[w] = M[w] vec[w]`` over the tables; worlds whose ``skip_world`` byte is set keep
    their row.  M (nworld, nM), vec and out (nworld, nv) float32 with contiguous rows; the
    tables int32 tensors on the same GPU."""
    import torch

    for t in (M, vec, out):
        if t.dtype != torch.float32 or not t.is_cuda:
            raise TypeError("mul_m needs float32 CUDA tensors")
        if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
            raise ValueError("mul_m needs rows of contiguous floats")
    for t in (mulm_rowadr, mulm_col, mulm_madr):
        if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
            raise TypeError("the row tables must be contiguous int32 CUDA tensors")
    nworld, nv = vec.shape
    if out.shape != vec.shape or M.shape[0] != nworld or mulm_rowadr.numel() != nv + 1 or mulm_madr.numel() != mulm_col.numel():
        raise ValueError("shapes of M, vec, out and the row table disagree")
    if skip_world is not None:
        if skip_world.dtype not in (torch.bool, torch.uint8) or skip_world.numel() != nworld or not skip_world.is_contiguous():
            raise TypeError("skip_world must be a contiguous bool or uint8 tensor with one element per world")
    with torch.cuda.device(M.device):
        status = _lib.lib().im_mul_m_sparse(
            M.data_ptr(), M.stride(0), int(M.shape[1]), mulm_rowadr.data_ptr(), mulm_col.data_ptr(),
            mulm_madr.data_ptr(), int(mulm_col.numel()), vec.data_ptr(), vec.stride(0), None if skip_world is None else skip_world.data_ptr(),
            out.data_ptr(), out.stride(0), int(nv), int(nworld), int(torch.cuda.current_stream(M.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_mul_m_sparse")


def gradient(nefc, efc_J, efc_force, qfrc_smooth, efc_Ma, state_changed_count, alpha, done, qfrc_constraint, grad,
             grad_dot, newton_decrement, grad_scale, search_unchanged, *, block: int = 64) -> None:  # fmt: skip
    """``qfrc_constraint = J' efc_force``, ``grad = efc_Ma - qfrc_smooth - qfrc_constraint`` and
    ``grad . grad`` for the worlds whose states changed; the rescaling of ``grad_dot``,
    ``newton_decrement`` and ``grad_scale`` for the others; ``search_unchanged`` for all (argument
    names of the reference's gradient_function).  ``efc_J`` (nworld, njmax, nv) contiguous float32;
    ``nefc`` int32 or None; ``done`` and ``search_unchanged`` bool or uint8; ``block`` = the lane
    count whose summation order ``grad_dot`` follows (32 or 64).  ``state_changed_count=None``
    counts every world as changed: the first gradient of a solve."""
    import torch

    if efc_J.dim() != 3 or not efc_J.is_contiguous() or efc_J.dtype != torch.float32 or not efc_J.is_cuda:
        raise TypeError("efc_J must be a contiguous float32 CUDA tensor (nworld, njmax, nv)")
    nworld, njmax, nv = efc_J.shape
    rows = (efc_force, qfrc_smooth, efc_Ma, qfrc_constraint, grad)
    for t, width in zip(rows, (njmax, nv, nv, nv, nv)):
        if t.dtype != torch.float32 or not t.is_cuda or t.dim() != 2 or t.shape != (nworld, width) or (width > 1 and t.stride(1) != 1):
            raise TypeError("force, smooth, Ma, constraint and grad must be float32 CUDA tensors with contiguous rows")
    for t in (alpha, grad_dot, newton_decrement, grad_scale):
        if t.dtype != torch.float32 or not t.is_cuda or t.numel() != nworld or not t.is_contiguous():
            raise TypeError("the per-world scalars must be contiguous float32 CUDA tensors")
    if state_changed_count is not None and (
        state_changed_count.dtype != torch.int32 or not state_changed_count.is_contiguous() or state_changed_count.numel() != nworld
    ):
        raise TypeError("state_changed_count must be a contiguous int32 tensor with one element per world")
    if nefc is not None and (nefc.dtype != torch.int32 or not nefc.is_contiguous() or nefc.numel() != nworld):
        raise TypeError("nefc must be a contiguous int32 tensor with one element per world")
    for t in (done, search_unchanged):
        if t is not None and (t.dtype not in (torch.bool, torch.uint8) or not t.is_contiguous() or t.numel() != nworld):
            raise TypeError("done and search_unchanged must be contiguous bool or uint8 tensors with one element per world")
    if search_unchanged is None:
        raise TypeError("search_unchanged is an output and cannot be None")
    with torch.cuda.device(efc_J.device):
        status = _lib.lib().im_newton_gradient(
            None if nefc is None else nefc.data_ptr(), efc_J.data_ptr(), int(njmax), efc_force.data_ptr(),
            efc_force.stride(0), qfrc_smooth.data_ptr(), qfrc_smooth.stride(0), efc_Ma.data_ptr(), efc_Ma.stride(0),
            None if state_changed_count is None else state_changed_count.data_ptr(), alpha.data_ptr(),
            None if done is None else done.data_ptr(),
            qfrc_constraint.data_ptr(), qfrc_constraint.stride(0), grad.data_ptr(), grad.stride(0), grad_dot.data_ptr(),
            newton_decrement.data_ptr(), grad_scale.data_ptr(), search_unchanged.data_ptr(), int(nv), int(block),
            int(nworld), int(torch.cuda.current_stream(efc_J.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_newton_gradient")


def jv(efc_J, search, jv_out, *, nefc=None, skip_world: Any = None) -> None:
    """``jv_out[w, r] = J[w, r, :] . search[w]`` for the rows below ``nefc[w]``, with the
    reference's summation rule (one chain up to 50 dofs, 20-dof partial sums beyond).  Worlds
    whose ``skip_world`` byte is set (done, or search direction unchanged) keep their row."""
    import torch

    if efc_J.dim() != 3 or not efc_J.is_contiguous() or efc_J.dtype != torch.float32 or not efc_J.is_cuda:
        raise TypeError("efc_J must be a contiguous float32 CUDA tensor (nworld, njmax, nv)")
    nworld, njmax, nv = efc_J.shape
    for t, width in ((search, nv), (jv_out, njmax)):
        if t.dtype != torch.float32 or not t.is_cuda or t.dim() != 2 or t.shape != (nworld, width) or (width > 1 and t.stride(1) != 1):
            raise TypeError("search (nworld, nv) and jv_out (nworld, njmax) must be float32 CUDA tensors with contiguous rows")
    if nefc is not None and (nefc.dtype != torch.int32 or not nefc.is_contiguous() or nefc.numel() != nworld):
        raise TypeError("nefc must be a contiguous int32 tensor with one element per world")
    if skip_world is not None and (
        skip_world.dtype not in (torch.bool, torch.uint8) or not skip_world.is_contiguous() or skip_world.numel() != nworld
    ):
        raise TypeError("skip_world must be a contiguous bool or uint8 tensor with one element per world")
    with torch.cuda.device(efc_J.device):
        status = _lib.lib().im_newton_jv(
            efc_J.data_ptr(), int(njmax), None if nefc is None else nefc.data_ptr(), search.data_ptr(), search.stride(0),
            None if skip_world is None else skip_world.data_ptr(), jv_out.data_ptr(), jv_out.stride(0), int(nv), int(nworld),
            int(torch.cuda.current_stream(efc_J.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_newton_jv")


def _per_world(t, nworld, dtypes, name):
    if t.dtype not in dtypes or not t.is_cuda or not t.is_contiguous() or t.numel() != nworld:
        raise TypeError(f"{name} must be a contiguous CUDA tensor with one element per world")


def _rows(t, nworld, width, dtype, name):
    if t.dtype != dtype or not t.is_cuda or t.dim() != 2 or t.shape != (nworld, width) or (width > 1 and t.stride(1) != 1):
        raise TypeError(f"{name} must be a ({nworld}, {width}) CUDA tensor with contiguous rows")


def advance(alpha, search, mv, jv_in, qacc, efc_Ma, Jaref, *, nefc=None, done=None) -> None:
    """In place: ``qacc += alpha search``, ``efc_Ma += alpha mv``, ``Jaref += alpha jv`` (rows
    below ``nefc``) for the worlds that are not done."""
    import torch

    nworld, nv = search.shape
    njmax = jv_in.shape[1]
    _per_world(alpha, nworld, (torch.float32,), "alpha")
    for t, width, name in ((search, nv, "search"), (mv, nv, "mv"), (qacc, nv, "qacc"), (efc_Ma, nv, "efc_Ma"),
                           (jv_in, njmax, "jv"), (Jaref, njmax, "Jaref")):  # fmt: skip
        _rows(t, nworld, width, torch.float32, name)
    if nefc is not None:
        _per_world(nefc, nworld, (torch.int32,), "nefc")
    if done is not None:
        _per_world(done, nworld, (torch.bool, torch.uint8), "done")
    with torch.cuda.device(search.device):
        status = _lib.lib().im_newton_advance(
            alpha.data_ptr(), search.data_ptr(), search.stride(0), mv.data_ptr(), mv.stride(0), jv_in.data_ptr(),
            jv_in.stride(0), None if nefc is None else nefc.data_ptr(), None if done is None else done.data_ptr(),
            qacc.data_ptr(), qacc.stride(0), efc_Ma.data_ptr(), efc_Ma.stride(0), Jaref.data_ptr(), Jaref.stride(0),
            int(nv), int(njmax), int(nworld), int(torch.cuda.current_stream(search.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_newton_advance")


def changed_rows(old_state, new_state, quad_changed_ids, quad_changed_count, state_changed_count, *, nefc=None,
                 done=None, quad: int = 1) -> None:  # fmt: skip
    """Rows whose being quadratic flipped, ascending, into ``quad_changed_ids`` with their count,
    and the count of rows whose state changed at all."""
    import torch

    nworld, njmax = old_state.shape
    for t, name in ((old_state, "old_state"), (new_state, "new_state")):
        if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous() or t.shape != (nworld, njmax):
            raise TypeError(f"{name} must be a contiguous int32 CUDA tensor (nworld, njmax)")
    if quad_changed_ids.dtype != torch.int32 or not quad_changed_ids.is_contiguous() or quad_changed_ids.dim() != 2 or quad_changed_ids.shape[0] != nworld:
        raise TypeError("quad_changed_ids must be a contiguous int32 CUDA tensor (nworld, width)")
    _per_world(quad_changed_count, nworld, (torch.int32,), "quad_changed_count")
    _per_world(state_changed_count, nworld, (torch.int32,), "state_changed_count")
    if nefc is not None:
        _per_world(nefc, nworld, (torch.int32,), "nefc")
    if done is not None:
        _per_world(done, nworld, (torch.bool, torch.uint8), "done")
    with torch.cuda.device(old_state.device):
        status = _lib.lib().im_newton_changed_rows(
            old_state.data_ptr(), new_state.data_ptr(), int(njmax), None if nefc is None else nefc.data_ptr(), int(quad),
            None if done is None else done.data_ptr(), quad_changed_ids.data_ptr(), int(quad_changed_ids.shape[1]),
            quad_changed_count.data_ptr(), state_changed_count.data_ptr(), int(nworld),
            int(torch.cuda.current_stream(old_state.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_newton_changed_rows")


def converged(alpha, improvement, grad_dot, newton_decrement, opt_tolerance, stat_meaninertia, nv: int, maxiter: int,
              niter, done, *, overflow=None, overflow_bit: int = 0, nsolving=None) -> None:  # fmt: skip
    """Counts the iteration and marks the worlds that converged (or ran out of iterations) done,
    with the reference's four criteria; ``nsolving`` (one int32) is decremented once per such
    world."""
    import torch

    nworld = alpha.numel()
    for t, name in ((alpha, "alpha"), (improvement, "improvement"), (grad_dot, "grad_dot"), (newton_decrement, "newton_decrement")):
        _per_world(t, nworld, (torch.float32,), name)
    for t in (opt_tolerance, stat_meaninertia):
        if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous() or t.numel() == 0:
            raise TypeError("opt_tolerance and stat_meaninertia must be non-empty contiguous float32 CUDA tensors")
    _per_world(niter, nworld, (torch.int32,), "niter")
    _per_world(done, nworld, (torch.bool, torch.uint8), "done")
    if overflow is not None:
        _per_world(overflow, nworld, (torch.int32,), "overflow")
    if nsolving is not None and (nsolving.dtype != torch.int32 or not nsolving.is_cuda or nsolving.numel() != 1):
        raise TypeError("nsolving must be a one-element int32 CUDA tensor")
    with torch.cuda.device(alpha.device):
        status = _lib.lib().im_newton_converged(
            alpha.data_ptr(), improvement.data_ptr(), grad_dot.data_ptr(), newton_decrement.data_ptr(),
            opt_tolerance.data_ptr(), int(opt_tolerance.numel()), stat_meaninertia.data_ptr(), int(stat_meaninertia.numel()),
            int(nv), int(maxiter), int(overflow_bit), niter.data_ptr(), None if overflow is None else overflow.data_ptr(),
            done.data_ptr(), None if nsolving is None else nsolving.data_ptr(), int(nworld),
            int(torch.cuda.current_stream(alpha.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_newton_converged")


def init_empty_worlds(nefc, qacc_smooth, solver_niter, search_dot, done, qacc) -> None:
    """``solver_niter = 0``, ``search_dot = 0``, ``done = nefc == 0`` and ``qacc = qacc_smooth``
    for the worlds without constraint rows."""
    import torch

    nworld, nv = qacc.shape
    _per_world(nefc, nworld, (torch.int32,), "nefc")
    _per_world(solver_niter, nworld, (torch.int32,), "solver_niter")
    _per_world(search_dot, nworld, (torch.float32,), "search_dot")
    _per_world(done, nworld, (torch.bool, torch.uint8), "done")
    _rows(qacc_smooth, nworld, nv, torch.float32, "qacc_smooth")
    _rows(qacc, nworld, nv, torch.float32, "qacc")
    with torch.cuda.device(qacc.device):
        status = _lib.lib().im_newton_init_empty_worlds(
            nefc.data_ptr(), qacc_smooth.data_ptr(), qacc_smooth.stride(0), solver_niter.data_ptr(), search_dot.data_ptr(),
            done.data_ptr(), qacc.data_ptr(), qacc.stride(0), int(nv), int(nworld),
            int(torch.cuda.current_stream(qacc.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_newton_init_empty_worlds")


def qfrc_constraint_from_grad(nefc, qfrc_smooth, efc_Ma, grad, grad_scale, qfrc_constraint) -> None:
    """``qfrc_constraint = efc_Ma - qfrc_smooth - grad_scale grad``; zero where ``nefc == 0``."""
    import torch

    nworld, nv = grad.shape
    _per_world(nefc, nworld, (torch.int32,), "nefc")
    _per_world(grad_scale, nworld, (torch.float32,), "grad_scale")
    for t, name in ((qfrc_smooth, "qfrc_smooth"), (efc_Ma, "efc_Ma"), (grad, "grad"), (qfrc_constraint, "qfrc_constraint")):
        _rows(t, nworld, nv, torch.float32, name)
    with torch.cuda.device(grad.device):
        status = _lib.lib().im_qfrc_constraint_from_grad(
            nefc.data_ptr(), qfrc_smooth.data_ptr(), qfrc_smooth.stride(0), efc_Ma.data_ptr(), efc_Ma.stride(0),
            grad.data_ptr(), grad.stride(0), grad_scale.data_ptr(), qfrc_constraint.data_ptr(), qfrc_constraint.stride(0),
            int(nv), int(nworld), int(torch.cuda.current_stream(grad.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_qfrc_constraint_from_grad")


def linesearch(opt_tolerance, opt_ls_tolerance, stat_meaninertia, ne, nf, nefc, qfrc_smooth, efc_D, efc_frictionloss, Jaref,
               search, search_dot, mv, jv_in, efc_Ma, done, alpha, improvement, ls_exhausted, *, ls_iterations: int,
               overflow=None, overflow_bit: int = 0) -> None:  # fmt: skip
    """The scalar search of the line-search stage (newton_stages.py:179-372): ``alpha``,
    ``improvement`` and ``ls_exhausted`` per world from ``Jaref``, ``jv = J search``,
    ``mv = M search`` and the rows' weights.  ``ne`` / ``nf`` / ``nefc`` int32 per world or None."""
    import torch

    nworld, nv = search.shape
    njmax = efc_D.shape[1]
    for t, width, name in ((qfrc_smooth, nv, "qfrc_smooth"), (search, nv, "search"), (mv, nv, "mv"), (efc_Ma, nv, "efc_Ma"),
                           (efc_D, njmax, "efc_D"), (Jaref, njmax, "Jaref"), (jv_in, njmax, "jv")):  # fmt: skip
        _rows(t, nworld, width, torch.float32, name)
    if efc_frictionloss is not None:
        _rows(efc_frictionloss, nworld, njmax, torch.float32, "efc_frictionloss")
    for t, name in ((search_dot, "search_dot"), (alpha, "alpha"), (improvement, "improvement")):
        _per_world(t, nworld, (torch.float32,), name)
    _per_world(ls_exhausted, nworld, (torch.bool, torch.uint8), "ls_exhausted")
    for t, name in ((ne, "ne"), (nf, "nf"), (nefc, "nefc"), (overflow, "overflow")):
        if t is not None:
            _per_world(t, nworld, (torch.int32,), name)
    if done is not None:
        _per_world(done, nworld, (torch.bool, torch.uint8), "done")
    for t in (opt_tolerance, opt_ls_tolerance, stat_meaninertia):
        if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous() or t.numel() < 1:
            raise TypeError("tolerances and meaninertia must be contiguous float32 CUDA tensors")
    ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    with torch.cuda.device(search.device):
        status = _lib.lib().im_newton_linesearch(
            opt_tolerance.data_ptr(), int(opt_tolerance.numel()), opt_ls_tolerance.data_ptr(), int(opt_ls_tolerance.numel()),
            stat_meaninertia.data_ptr(), int(stat_meaninertia.numel()), ptr(ne), ptr(nf), ptr(nefc), int(njmax),
            qfrc_smooth.data_ptr(), qfrc_smooth.stride(0), efc_D.data_ptr(), efc_D.stride(0), ptr(efc_frictionloss),
            0 if efc_frictionloss is None else efc_frictionloss.stride(0), Jaref.data_ptr(), Jaref.stride(0),
            search.data_ptr(), search.stride(0), search_dot.data_ptr(), mv.data_ptr(), mv.stride(0), jv_in.data_ptr(),
            jv_in.stride(0), efc_Ma.data_ptr(), efc_Ma.stride(0), ptr(done), int(ls_iterations), int(overflow_bit),
            alpha.data_ptr(), improvement.data_ptr(), ls_exhausted.data_ptr(), ptr(overflow), int(nv), int(nworld),
            int(torch.cuda.current_stream(search.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_newton_linesearch")


def eval_constraints(Jaref, efc_D, efc_frictionloss, ne, nf, nefc, done, ls_exhausted, efc_force, efc_state, quad_changed_ids,
                     quad_changed_count, state_changed_count) -> None:  # fmt: skip
    """Force and state of every row from the advanced ``Jaref`` (in place), the ascending list of
    the rows whose being QUADRATIC flipped and the two counts (newton_stages.py:385-444)."""
    import torch

    nworld, njmax = efc_D.shape
    for t, name in ((Jaref, "Jaref"), (efc_D, "efc_D"), (efc_force, "efc_force")):
        _rows(t, nworld, njmax, torch.float32, name)
    if efc_frictionloss is not None:
        _rows(efc_frictionloss, nworld, njmax, torch.float32, "efc_frictionloss")
    _rows(efc_state, nworld, njmax, torch.int32, "efc_state")
    if quad_changed_ids.dtype != torch.int32 or not quad_changed_ids.is_contiguous() or quad_changed_ids.dim() != 2 or quad_changed_ids.shape[0] != nworld:
        raise TypeError("quad_changed_ids must be a contiguous int32 CUDA tensor (nworld, width)")
    for t, name in ((ne, "ne"), (nf, "nf"), (nefc, "nefc")):
        if t is not None:
            _per_world(t, nworld, (torch.int32,), name)
    _per_world(quad_changed_count, nworld, (torch.int32,), "quad_changed_count")
    _per_world(state_changed_count, nworld, (torch.int32,), "state_changed_count")
    for t, name in ((done, "done"), (ls_exhausted, "ls_exhausted")):
        if t is not None:
            _per_world(t, nworld, (torch.bool, torch.uint8), name)
    ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    with torch.cuda.device(efc_D.device):
        status = _lib.lib().im_newton_eval_constraints(
            Jaref.data_ptr(), Jaref.stride(0), efc_D.data_ptr(), efc_D.stride(0), ptr(efc_frictionloss),
            0 if efc_frictionloss is None else efc_frictionloss.stride(0), ptr(ne), ptr(nf), ptr(nefc), int(njmax),
            ptr(done), ptr(ls_exhausted), efc_force.data_ptr(), efc_force.stride(0), efc_state.data_ptr(),
            efc_state.stride(0), quad_changed_ids.data_ptr(), int(quad_changed_ids.shape[1]), quad_changed_count.data_ptr(),
            state_changed_count.data_ptr(), int(nworld), int(torch.cuda.current_stream(efc_D.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_newton_eval_constraints")


OVERFLOW_LS_ITERATIONS = 4  # bits of d.overflow: the caller's OverflowType where it differs
OVERFLOW_ITERATIONS = 8
DISABLE_WARMSTART = 1 << 8  # MuJoCo's mjDSBL_WARMSTART, matched by value when the model carries plain integers


def init_jaref(nefc, qacc, efc_J, efc_aref, Jaref) -> None:
    """``Jaref = J qacc - aref`` for the rows below ``nefc`` (upstream's ``_solve_init_jaref_kernel``
    as newton_fusion.py:451-468 launches it)."""
    import torch

    if efc_J.dim() != 3 or not efc_J.is_contiguous() or efc_J.dtype != torch.float32 or not efc_J.is_cuda:
        raise TypeError("efc_J must be a contiguous float32 CUDA tensor (nworld, njmax, nv)")
    nworld, njmax, nv = efc_J.shape
    _rows(qacc, nworld, nv, torch.float32, "qacc")
    _rows(efc_aref, nworld, njmax, torch.float32, "efc_aref")
    _rows(Jaref, nworld, njmax, torch.float32, "Jaref")
    if nefc is not None:
        _per_world(nefc, nworld, (torch.int32,), "nefc")
    with torch.cuda.device(efc_J.device):
        status = _lib.lib().im_newton_init_jaref(
            efc_J.data_ptr(), int(njmax), None if nefc is None else nefc.data_ptr(), qacc.data_ptr(), qacc.stride(0),
            efc_aref.data_ptr(), efc_aref.stride(0), Jaref.data_ptr(), Jaref.stride(0), int(nv), int(nworld),
            int(torch.cuda.current_stream(efc_J.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_newton_init_jaref")


def dense_from_csr(M, elemid, out) -> None:
    """``out[w]`` (rows x rows, rows >= nv) = the dense symmetric M of world w, zero outside M's
    pattern and in the padding; ``elemid`` (nv, nv) int32 names the CSR element of every pair."""
    import torch

    nv = int(elemid.shape[0])
    if elemid.dtype != torch.int32 or tuple(elemid.shape) != (nv, nv) or not elemid.is_contiguous() or not elemid.is_cuda:
        raise TypeError("elemid must be a contiguous (nv, nv) int32 CUDA tensor")
    nworld = int(M.shape[0])
    if out.dim() != 3 or out.shape[0] != nworld or out.shape[1] != out.shape[2] or out.shape[1] < nv or not out.is_contiguous():
        raise ValueError("out must be a contiguous (nworld, rows, rows) tensor with rows >= nv")
    for t in (M, out):
        if t.dtype != torch.float32 or not t.is_cuda:
            raise TypeError("M and out must be float32 CUDA tensors")
    if M.dim() != 2 or (M.shape[1] > 1 and M.stride(1) != 1):
        raise ValueError("M needs rows of contiguous floats")
    with torch.cuda.device(M.device):
        status = _lib.lib().im_dense_from_csr(M.data_ptr(), M.stride(0), elemid.data_ptr(), nv, int(out.shape[1]),
                                              out.data_ptr(), nworld, int(torch.cuda.current_stream(M.device).cuda_stream))  # fmt: skip
    _lib.check(status, "im_dense_from_csr")


def elemid_table(rowadr, rownnz, colind) -> np.ndarray:
    """(nv, nv) int32: the CSR element of M at (i, j) and (j, i), -1 outside the tree pattern (the
    layout of the reference's ``m.M_elemid``)."""
    rowadr, rownnz, colind = (np.asarray(a, np.int64) for a in (rowadr, rownnz, colind))
    nv = rowadr.size
    out = np.full((nv, nv), -1, np.int32)
    for i in range(nv):
        for k in range(rowadr[i], rowadr[i] + rownnz[i]):
            out[i, colind[k]] = out[colind[k], i] = k
    return out


def default_mul_m_call(m, d, out, vec) -> None:
    """``out = M vec`` over the model's row tables: the ``mul_m_call`` of the reference's scratch
    (src/instantmimic/utils/mjw_step_optimized.py:2595, 2709) for callers that have none."""
    mul_m(d.M, vec, out, m.M_mulm_rowadr, m.M_mulm_col, m.M_mulm_madr)


def _fused_plan(ctx):
    plan = getattr(ctx, "sparse_hessian_plan", None)
    return plan if plan is not None and plan.path == "fused" else None


def _tree_scratch(ctx):
    """The opt-in tree stage: a scratch of ``tree_ldl.create_tree_factor_solve_scratch`` that the
    caller has put on ``ctx.newton_tree_scratch`` (for models whose constraint rows stay on single
    root-to-leaf chains; the reference has no such stage)."""
    return getattr(ctx, "newton_tree_scratch", None) if ctx is not None else None


def attach_scratch(m, d, ctx, device=None) -> None:
    """Persistent per-world scratch of the fused iteration on ``ctx`` (newton_fusion.py:301-304:
    the dofs the changed rows touch, ``nv`` slots and their count); the dense path's first factor
    also keeps a dense copy of M, the M-pattern table and two constant count arrays here."""
    import torch

    dev = device if device is not None else d.qacc.device
    nworld, nv = int(d.nworld), int(m.nv)
    ctx.newton_dof_union = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=dev)
    if _fused_plan(ctx) is None and _tree_scratch(ctx) is None:
        ctx.newton_mdense = torch.zeros((nworld, nv, nv), dtype=torch.float32, device=dev)
        ctx.newton_refactor = torch.full((nworld,), -1, dtype=torch.int32, device=dev)
        ctx.newton_every = torch.ones((nworld,), dtype=torch.int32, device=dev)
        elemid = getattr(m, "M_elemid", None)
        if elemid is None:
            host = lambda a: a.cpu().numpy() if hasattr(a, "cpu") else np.asarray(a)  # noqa: E731
            elemid = torch.from_numpy(elemid_table(host(m.M_rowadr), host(m.M_rownnz), host(m.M_colind))).to(dev)
        ctx.newton_elemid = elemid.to(dtype=torch.int32).reshape(nv, nv).contiguous()
        ctx.newton_next_world = torch.zeros(1, dtype=torch.int32, device=dev)  # the resident kernel's world counter


def _stage(m, ctx):
    from . import newton_stages

    return newton_stages.factor_factory(int(m.nv), int(m.nv_pad), _fused_plan(ctx), tree_scratch=_tree_scratch(ctx),
                                        block=newton_block_dim(m))  # fmt: skip


def _launch_stage(stage, m, d, ctx) -> None:
    if _tree_scratch(ctx) is not None:
        stage(d.efc.J, d.efc.D, d.efc.state, None, None, None, ctx.done, ctx.grad, None, None, ctx.search, ctx.search_dot,
              ctx.newton_decrement, None, M=d.M, nefc=d.nefc, skip=ctx.search_unchanged)  # fmt: skip
        return
    sparse = _fused_plan(ctx) is not None
    stage(d.efc.J, d.efc.D, d.efc.state, ctx.quad_changed_ids, ctx.quad_changed_count, ctx.state_changed_count, ctx.done,
          ctx.grad, None if sparse else ctx.h, ctx.hfactor, ctx.search, ctx.search_dot, ctx.newton_decrement, ctx.newton_dof_union)  # fmt: skip


def _update_constraint(m, d, ctx) -> None:
    """Force and state of every row from ``ctx.Jaref`` (upstream's ``solver._update_constraint`` as
    newton_fusion.py:469 calls it; ``qfrc_constraint = J' force`` is formed with the gradient)."""
    eval_constraints(ctx.Jaref, d.efc.D, d.efc.frictionloss, d.ne, d.nf, d.nefc, ctx.done, None, d.efc.force, d.efc.state,
                     ctx.quad_changed_ids, ctx.quad_changed_count, ctx.state_changed_count)  # fmt: skip


def _first_gradient(m, d, ctx) -> None:
    """``qfrc_constraint``, ``grad`` and ``grad . grad`` of every world that is not done, with
    ``newton_decrement = 0``, ``grad_scale = 1`` and ``search_unchanged = done`` (upstream's
    ``_update_gradient_zero_grad_dot`` and ``_update_gradient_grad``, newton_fusion.py:487-500)."""
    nv = int(m.nv)
    gradient(d.nefc, d.efc.J, d.efc.force, d.qfrc_smooth, d.efc.Ma, None, ctx.alpha, ctx.done, d.qfrc_constraint,
             ctx.grad[:, :nv], ctx.grad_dot, ctx.newton_decrement, ctx.grad_scale, ctx.search_unchanged,
             block=newton_block_dim(m))  # fmt: skip


def _update_gradient_sparse(m, d, ctx, plan, *, gradient_done: bool = False) -> None:
    """The first gradient, then H assembled on the sparse pattern, factored and solved
    (newton_fusion.py:481-519)."""
    from . import sparse_hessian

    if not gradient_done:
        _first_gradient(m, d, ctx)
    sparse_hessian.init_factor_kernel(plan)(ctx.done, d.nefc, d.efc.J, d.efc.D, d.efc.state, d.M, ctx.grad, ctx.hfactor,
                                            ctx.search, ctx.search_dot, ctx.newton_decrement)  # fmt: skip


def _update_gradient_tree(m, d, ctx, *, gradient_done: bool = False) -> None:
    """The first gradient, then the tree stage for every world that is not done (``search_unchanged``
    is ``done`` at this point)."""
    if not gradient_done:
        _first_gradient(m, d, ctx)
    _launch_stage(_stage(m, ctx), m, d, ctx)


def _update_gradient(m, d, ctx, *, gradient_done: bool = False) -> None:
    """The dense first factor (upstream's ``solver._update_gradient`` for the dense Newton,
    newton_fusion.py:470): ``ctx.h = M + J' D_act J`` on the matrix cores, then the augmented
    blocked Cholesky of the per-iteration stage without an update."""
    from . import blocked_dense

    if not hasattr(ctx, "newton_mdense"):
        raise RuntimeError("the dense first factor needs attach_scratch(m, d, ctx)")
    if not gradient_done:
        _first_gradient(m, d, ctx)
    # one launch where the shape has one (up to 63 dofs); IMHIP_NEWTON=stages keeps the three
    if os.environ.get("IMHIP_NEWTON") != "stages" and blocked_dense.dense_init_factor(
            d.M, ctx.newton_elemid, d.efc.J, d.efc.D, d.efc.state, d.nefc, ctx.done, ctx.grad, ctx.h, ctx.hfactor, ctx.search,
            ctx.search_dot, ctx.newton_decrement, ctx.newton_dof_union):  # fmt: skip
        return
    dense_from_csr(d.M, ctx.newton_elemid, ctx.newton_mdense)
    blocked_dense.dense_hessian(ctx.newton_mdense, d.efc.J, d.efc.D, d.efc.state, d.nefc, ctx.h)
    stage = _stage(m, ctx)
    stage(d.efc.J, d.efc.D, d.efc.state, ctx.quad_changed_ids, ctx.newton_refactor, ctx.newton_every, ctx.done, ctx.grad,
          ctx.h, ctx.hfactor, ctx.search, ctx.search_dot, ctx.newton_decrement, ctx.newton_dof_union)  # fmt: skip


def init_context(m, d, ctx, mul_m_call=None) -> None:
    """``init_context`` of the fused path (newton_fusion.py:431-478): worlds without constraint rows
    finish at once with ``qacc = qacc_smooth``; ``Jaref = J qacc - aref``; ``Ma = M qacc`` for every
    world; forces and states; the first gradient, Hessian, factor and search direction through the
    sparse plan, the tree stage or the dense path, whichever ``ctx`` carries."""
    first = _init_before_factor(m, d, ctx) if mul_m_call is None else False
    if not first:
        init_empty_worlds(d.nefc, d.qacc_smooth, d.solver_niter, ctx.search_dot, ctx.done, d.qacc)
        init_jaref(d.nefc, d.qacc, d.efc.J, d.efc.aref, ctx.Jaref)
        (mul_m_call or default_mul_m_call)(m, d, d.efc.Ma, d.qacc)
        _update_constraint(m, d, ctx)
    plan = _fused_plan(ctx)
    if plan is not None:
        _update_gradient_sparse(m, d, ctx, plan, gradient_done=first)
    elif _tree_scratch(ctx) is not None:
        _update_gradient_tree(m, d, ctx, gradient_done=first)
    else:
        _update_gradient(m, d, ctx, gradient_done=first)


def _init_before_factor(m, d, ctx) -> bool:
    """Everything of ``init_context`` before the first Hessian in one launch, a wavefront per world
    (``im_newton_init_context``: the same values as the five launches it stands for).  False, with
    nothing done, under ``IMHIP_NEWTON=stages``, for arrays the one launch does not take (rows of
    ``qacc_smooth`` or ``efc.aref`` that are not contiguous) and for sizes beyond a workgroup's LDS."""
    import ctypes as C

    import torch

    if os.environ.get("IMHIP_NEWTON") == "stages":
        return False
    # the one launch takes the argument block of the resident loop: a context without the loop's own
    # arrays (a caller that only wants the start of a solve) keeps the five launches
    if any(getattr(ctx, name, None) is None for name in ("mv", "jv", "alpha", "improvement", "ls_exhausted", "search")):
        return False
    smooth, aref = d.qacc_smooth, d.efc.aref
    nworld, nv = int(d.nworld), int(m.nv)
    dev = d.efc.J.device
    for t, width in ((smooth, nv), (aref, int(d.efc.J.shape[1]))):
        if t.dtype != torch.float32 or t.device != dev or t.dim() != 2 or t.shape[0] != nworld or t.shape[1] < width or (
            t.shape[1] > 1 and t.stride(1) != 1
        ):
            return False
    a = _resident_args(m, d, ctx, None)
    with torch.cuda.device(dev):
        status = _lib.lib().im_newton_init_context(
            C.byref(a), smooth.data_ptr(), smooth.stride(0), aref.data_ptr(), aref.stride(0), nv, int(d.M.shape[1]),
            int(torch.cuda.current_stream(dev).cuda_stream))  # fmt: skip
    if status == _lib.IM_ERR_UNSUPPORTED:
        return False
    _lib.check(status, "im_newton_init_context")
    return True


def iteration(m, d, ctx, nsolving=None, *, stage=None) -> None:
    """One iteration of the fused Newton loop for every world that is not done, as eight launches in
    the reference kernel's order (newton_fusion.py:151-296): M search, J search, the scalar search,
    the step, the constraints' new forces and states, the gradient, the factor stage, the
    convergence test."""
    nv = int(m.nv)
    if stage is None:
        stage = _stage(m, ctx)
    mul_m(d.M, ctx.search, ctx.mv, m.M_mulm_rowadr, m.M_mulm_col, m.M_mulm_madr, skip_world=ctx.search_unchanged)
    jv(d.efc.J, ctx.search, ctx.jv, nefc=d.nefc, skip_world=ctx.search_unchanged)
    linesearch(m.opt.tolerance, m.opt.ls_tolerance, m.stat.meaninertia, d.ne, d.nf, d.nefc, d.qfrc_smooth, d.efc.D,
               d.efc.frictionloss, ctx.Jaref, ctx.search, ctx.search_dot, ctx.mv, ctx.jv, d.efc.Ma, ctx.done, ctx.alpha,
               ctx.improvement, ctx.ls_exhausted, ls_iterations=int(m.opt.ls_iterations), overflow=d.overflow,
               overflow_bit=OVERFLOW_LS_ITERATIONS)  # fmt: skip
    advance(ctx.alpha, ctx.search, ctx.mv, ctx.jv, d.qacc, d.efc.Ma, ctx.Jaref, nefc=d.nefc, done=ctx.done)
    eval_constraints(ctx.Jaref, d.efc.D, d.efc.frictionloss, d.ne, d.nf, d.nefc, ctx.done, ctx.ls_exhausted, d.efc.force,
                     d.efc.state, ctx.quad_changed_ids, ctx.quad_changed_count, ctx.state_changed_count)  # fmt: skip
    gradient(d.nefc, d.efc.J, d.efc.force, d.qfrc_smooth, d.efc.Ma, ctx.state_changed_count, ctx.alpha, ctx.done,
             d.qfrc_constraint, ctx.grad[:, :nv], ctx.grad_dot, ctx.newton_decrement, ctx.grad_scale, ctx.search_unchanged,
             block=newton_block_dim(m))  # fmt: skip
    _launch_stage(stage, m, d, ctx)
    converged(ctx.alpha, ctx.improvement, ctx.grad_dot, ctx.newton_decrement, m.opt.tolerance, m.stat.meaninertia, nv,
              int(m.opt.iterations), d.solver_niter, ctx.done, overflow=d.overflow, overflow_bit=OVERFLOW_ITERATIONS,
              nsolving=nsolving)  # fmt: skip


def _resident_args(m, d, ctx, nsolving):
    """The arrays of ``run`` as the C ABI's ``im_newton_args``, after the checks that no pointer may
    leave Python without: one device, float32 / int32 / bytes, rows of the expected length."""
    import torch

    nworld, nv = int(d.nworld), int(m.nv)
    J = d.efc.J
    if J.dim() != 3 or not J.is_contiguous() or J.dtype != torch.float32 or not J.is_cuda or J.shape[0] != nworld or J.shape[2] != nv:
        raise TypeError("efc_J must be a contiguous float32 CUDA tensor (nworld, njmax, nv)")
    njmax = int(J.shape[1])
    dev = J.device

    def rows(t, width, dtype, name):
        if t.dtype != dtype or t.device != dev or tuple(t.shape) != (nworld, width) or not t.is_contiguous():
            raise TypeError(f"{name} must be a contiguous ({nworld}, {width}) tensor of {dtype} on {dev}")
        return t.data_ptr()

    def per_world(t, dtypes, name, optional=False):
        if t is None and optional:
            return None
        if t.dtype not in dtypes or t.device != dev or t.numel() != nworld or not t.is_contiguous():
            raise TypeError(f"{name} must be a contiguous tensor with one element per world on {dev}")
        return t.data_ptr()

    def table(t, name):
        if t.dtype != torch.int32 or t.device != dev or not t.is_contiguous():
            raise TypeError(f"{name} must be a contiguous int32 tensor on {dev}")
        return t.data_ptr()

    f32, i32, byte = torch.float32, torch.int32, (torch.bool, torch.uint8)
    a = _lib.NewtonArgs()
    for name, t in (("opt_tolerance", m.opt.tolerance), ("opt_ls_tolerance", m.opt.ls_tolerance), ("stat_meaninertia", m.stat.meaninertia)):
        if t.dtype != f32 or t.device != dev or not t.is_contiguous() or t.numel() < 1:
            raise TypeError(f"{name} must be a non-empty contiguous float32 tensor on {dev}")
        setattr(a, name, t.data_ptr())
    a.ntolerance, a.nls_tolerance, a.nmeaninertia = m.opt.tolerance.numel(), m.opt.ls_tolerance.numel(), m.stat.meaninertia.numel()
    a.ls_iterations, a.iterations = int(m.opt.ls_iterations), int(m.opt.iterations)
    a.block, a.quad = newton_block_dim(m), 1
    a.ls_overflow_bit, a.iterations_overflow_bit = OVERFLOW_LS_ITERATIONS, OVERFLOW_ITERATIONS
    if m.M_mulm_rowadr.numel() != nv + 1 or m.M_mulm_col.numel() != m.M_mulm_madr.numel():
        raise ValueError("the row tables of M v do not match the model")
    a.M_mulm_rowadr, a.M_mulm_col, a.M_mulm_madr = (table(t, "M_mulm_*") for t in (m.M_mulm_rowadr, m.M_mulm_col, m.M_mulm_madr))
    a.nterm = int(m.M_mulm_col.numel())
    a.ne, a.nf, a.nefc = (per_world(t, (i32,), n, optional=True) for t, n in ((d.ne, "ne"), (d.nf, "nf"), (d.nefc, "nefc")))
    M = d.M
    if M.dtype != f32 or M.device != dev or M.dim() != 2 or M.shape[0] != nworld or (M.shape[1] > 1 and M.stride(1) != 1):
        raise TypeError("M must be a float32 (nworld, nM) tensor with contiguous rows")
    a.M, a.ldM = M.data_ptr(), M.stride(0)
    a.efc_J, a.njmax = J.data_ptr(), njmax
    a.efc_D = rows(d.efc.D, njmax, f32, "efc_D")
    a.efc_frictionloss = None if d.efc.frictionloss is None else rows(d.efc.frictionloss, njmax, f32, "efc_frictionloss")
    a.qfrc_smooth = rows(d.qfrc_smooth, nv, f32, "qfrc_smooth")
    a.qacc, a.efc_Ma = rows(d.qacc, nv, f32, "qacc"), rows(d.efc.Ma, nv, f32, "efc_Ma")
    a.efc_force, a.efc_state = rows(d.efc.force, njmax, f32, "efc_force"), rows(d.efc.state, njmax, i32, "efc_state")
    a.Jaref, a.jv = rows(ctx.Jaref, njmax, f32, "Jaref"), rows(ctx.jv, njmax, f32, "jv")
    a.search, a.mv = rows(ctx.search.reshape(nworld, -1), nv, f32, "search"), rows(ctx.mv, nv, f32, "mv")
    a.qfrc_constraint = rows(d.qfrc_constraint, nv, f32, "qfrc_constraint")
    grad = ctx.grad.reshape(nworld, -1)
    if grad.dtype != f32 or grad.device != dev or grad.shape[1] < nv or not grad.is_contiguous():
        raise TypeError("grad must be a contiguous float32 (nworld, >= nv) tensor")
    a.grad, a.ld_grad = grad.data_ptr(), grad.shape[1]
    for name, t in (("search_dot", ctx.search_dot), ("alpha", ctx.alpha), ("improvement", ctx.improvement), ("grad_dot", ctx.grad_dot),
                    ("grad_scale", ctx.grad_scale), ("newton_decrement", ctx.newton_decrement)):  # fmt: skip
        setattr(a, name, per_world(t, (f32,), name))
    ids = ctx.quad_changed_ids
    if ids.dtype != i32 or ids.device != dev or ids.dim() != 2 or ids.shape[0] != nworld or not ids.is_contiguous():
        raise TypeError("quad_changed_ids must be a contiguous int32 (nworld, width) tensor")
    a.quad_changed_ids, a.ld_ids = ids.data_ptr(), ids.shape[1]
    a.quad_changed_count = per_world(ctx.quad_changed_count, (i32,), "quad_changed_count")
    a.state_changed_count = per_world(ctx.state_changed_count, (i32,), "state_changed_count")
    a.solver_niter = per_world(d.solver_niter, (i32,), "solver_niter")
    a.overflow = per_world(getattr(d, "overflow", None), (i32,), "overflow", optional=True)
    if nsolving is not None and (nsolving.dtype != i32 or nsolving.device != dev or nsolving.numel() != 1):
        raise TypeError("nsolving must be a one-element int32 tensor")
    a.nsolving = None if nsolving is None else nsolving.data_ptr()
    a.done = per_world(ctx.done, byte, "done")
    a.ls_exhausted = per_world(ctx.ls_exhausted, byte, "ls_exhausted")
    a.search_unchanged = per_world(ctx.search_unchanged, byte, "search_unchanged")
    a.nworld = nworld
    return a


def run_resident(m, d, ctx, nsolving) -> bool:
    """The whole loop as one resident kernel (a wavefront per world until it is done): for a ``ctx``
    with a fused sparse plan, with the tree stage whose plan carries generated kernels, or for a
    dense model of up to 63 dofs (the single-tile stage up to 32, the blocked stage on a wavefront
    per world for a padded size of 48 or 64).  False when there is no such kernel for
    this model (the caller then launches the stages one by one)."""
    import ctypes as C

    import torch

    scratch, plan = _tree_scratch(ctx), _fused_plan(ctx)
    dense = scratch is None and plan is None and getattr(ctx, "newton_next_world", None) is not None
    dense_tile = dense and int(m.nv) <= 32
    dense_column = dense and int(m.nv) > 32 and int(m.nv_pad) in (48, 64)
    if (scratch is None and plan is None and not (dense_tile or dense_column)) or os.environ.get("IMHIP_NEWTON") == "stages":
        return False
    a = _resident_args(m, d, ctx, nsolving)
    dev = d.efc.J.device
    stream = int(torch.cuda.current_stream(dev).cuda_stream)
    with torch.cuda.device(dev):
        if dense_tile or dense_column:
            nworld, nv, pad = int(d.nworld), int(m.nv), int(m.nv_pad)
            h, uni, counter = ctx.h, ctx.newton_dof_union, ctx.newton_next_world
            if h.dtype != torch.float32 or h.device != dev or tuple(h.shape) != (nworld, pad, pad) or not h.is_contiguous():
                raise TypeError("h must be a contiguous float32 (nworld, nv_pad, nv_pad) tensor")
            if uni.dtype != torch.int32 or uni.device != dev or tuple(uni.shape) != (nworld, nv + 1) or not uni.is_contiguous():
                raise TypeError("newton_dof_union must be a contiguous int32 (nworld, nv + 1) tensor")
            if counter.dtype != torch.int32 or counter.device != dev or counter.numel() != 1:
                raise TypeError("newton_next_world must be a one-element int32 tensor")
            if dense_tile:
                status = _lib.lib().im_newton_solve_dense_tile(C.byref(a), h.data_ptr(), uni.data_ptr(), nv, pad, int(d.M.shape[1]),
                                                               counter.data_ptr(), stream)  # fmt: skip
                where = "im_newton_solve_dense_tile"
            else:
                hf = ctx.hfactor
                if hf.dtype != torch.float32 or hf.device != dev or tuple(hf.shape) != (nworld, pad, pad) or not hf.is_contiguous():
                    raise TypeError("hfactor must be a contiguous float32 (nworld, nv_pad, nv_pad) tensor")
                status = _lib.lib().im_newton_solve_dense_column(C.byref(a), h.data_ptr(), hf.data_ptr(), uni.data_ptr(), nv, pad,
                                                                 int(d.M.shape[1]), counter.data_ptr(), stream)  # fmt: skip
                where = "im_newton_solve_dense_column"
        elif plan is not None:
            nworld, nv, pad = int(d.nworld), int(m.nv), int(m.nv_pad)
            hf, uni = ctx.hfactor, ctx.newton_dof_union
            if hf.dtype != torch.float32 or hf.device != dev or tuple(hf.shape) != (nworld, pad, pad) or not hf.is_contiguous():
                raise TypeError("hfactor must be a contiguous float32 (nworld, nv_pad, nv_pad) tensor")
            if uni.dtype != torch.int32 or uni.device != dev or tuple(uni.shape) != (nworld, nv + 1) or not uni.is_contiguous():
                raise TypeError("newton_dof_union must be a contiguous int32 (nworld, nv + 1) tensor")
            if plan.handle is None or plan.nv != nv or plan.nv_pad != pad:
                raise ValueError("the sparse plan has no device state or belongs to another model")
            status = _lib.lib().im_newton_solve_sparse(plan.ptr, C.byref(a), hf.data_ptr(), uni.data_ptr(), stream)
            where = "im_newton_solve_sparse"
        else:
            status = _lib.lib().im_newton_solve_tree(scratch.kernel.ptr, C.byref(a), stream)
            where = "im_newton_solve_tree"
    if status == _lib.IM_ERR_UNSUPPORTED:
        return False
    _lib.check(status, where)
    return True


def run(m, d, ctx, nsolving, *, check_every: int | None = None, graph: bool = False) -> int:
    """The fused Newton solve with the reference's signature (newton_fusion.py:330-409): iterates
    until every world is done or ``m.opt.iterations`` is reached.  The reference keeps a world in
    one resident block for the whole loop; here an iteration is eight launches over all worlds and
    finished worlds drop out of each through ``ctx.done``, so launching all ``m.opt.iterations``
    of them is correct whatever the worlds need, touches the host nowhere and can be captured in a
    caller's graph: that is what happens under stream capture and with ``check_every=0``.  With
    the tree stage on ``ctx`` and neither ``check_every`` nor ``graph`` given, the loop is one
    resident kernel (:func:`run_resident`: the same results, no launch per stage).
    Outside a capture the host by default reads ``ctx.done`` every fourth iteration and stops early
    (``check_every``).  ``graph``: the first iteration runs as plain launches, the second is
    captured in a graph that the later ones replay (the arrays of ``d`` and ``ctx`` must then stay
    where they are for the whole solve).  Returns the number of iterations launched."""
    import torch

    if check_every is None and not graph and run_resident(m, d, ctx, nsolving):
        return int(m.opt.iterations)
    capturing = torch.cuda.is_current_stream_capturing()
    if check_every is None:
        check_every = 0 if capturing else 4
    if capturing and (check_every or graph):
        raise RuntimeError("under stream capture the solve runs without host checks and without a graph of its own")
    stage = _stage(m, ctx)
    limit = int(m.opt.iterations)
    captured = None
    launched = 0
    for it in range(limit):
        if not graph or it == 0:
            iteration(m, d, ctx, nsolving, stage=stage)
        elif captured is None:
            captured = torch.cuda.CUDAGraph()
            with torch.cuda.graph(captured):
                iteration(m, d, ctx, nsolving, stage=stage)
            captured.replay()  # capturing records the launches without running them
        else:
            captured.replay()
        launched += 1
        if check_every > 0 and (it + 1) % check_every == 0 and bool(ctx.done.all().item()):
            break
    return launched


def solve(m, d, ctx, nsolving, *, mul_m_call=None) -> None:
    """The constraint solve around the fused loop, in the order of ``_solve_monolithic_with_scratch``
    for an eligible model (src/instantmimic/utils/mjw_step_optimized.py:2588-2683): the start point
    (warm start unless disabled), ``init_context``, the loop, the constraint force from the last
    gradient.  No step reads anything back, so the whole solve can sit in a caller's graph."""
    flags = getattr(m.opt, "disableflags", 0)
    warmstart = not (int(flags) & DISABLE_WARMSTART) and getattr(d, "qacc_warmstart", None) is not None
    d.qacc.copy_(d.qacc_warmstart if warmstart else d.qacc_smooth)
    d.qfrc_constraint.zero_()
    init_context(m, d, ctx, mul_m_call)
    ctx.search_unchanged.zero_()
    nsolving.fill_(int(d.nworld))
    run(m, d, ctx, nsolving)
    nv = int(m.nv)
    qfrc_constraint_from_grad(d.nefc, d.qfrc_smooth, d.efc.Ma, ctx.grad[:, :nv], ctx.grad_scale, d.qfrc_constraint)
