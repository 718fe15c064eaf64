"""A whole constraint solve chained from the oracle's pieces, for the tests of the Newton drop-in:
the order of ``_solve_monolithic_with_scratch`` for an eligible model
(src/instantmimic/utils/mjw_step_optimized.py:2588-2683): start point, ``init_context``
(src/instantmimic/utils/mjw_kernels/newton_fusion.py:431-519), the iterations of the resident
kernel (:151-296), the constraint force from the last gradient (:522-539).  Helper module, not
collected by pytest.

Three factor stages: ``"dense"`` (incremental update of the dense H and the augmented blocked
Cholesky), ``"sparse"`` (the static-pattern L'DL of a fused plan), ``"tree"`` (fresh assembly on
M's pattern and the tree L'DL)."""

from __future__ import annotations

from types import SimpleNamespace

import numpy as np

from instantmimic_amd import synth
from instantmimic_amd.mjw_kernels import newton_fusion as NF
from oracle import planner as P
from oracle import ref as R


def problem(name: str, nworld: int, stage: str, *, seed: int = 21, maxiter: int = 30, ls_iterations: int = 50,
            empty_every: int = 0, warmstart: bool = False):
    """The model and one step's inputs on the tree of ``name``: 2 equality rows, 3 friction-loss
    rows, the rest one-sided; every ``empty_every``-th world has no constraint row at all."""
    shape = synth.SHAPES[name]
    b = synth.make_batch(shape, nworld, ragged_nefc=True)
    rng = np.random.default_rng(seed)
    nv, njmax = shape.nv, shape.nefc
    m = synth.model_from_parents(shape.parents)
    p = SimpleNamespace(b=b, name=name, nv=nv, njmax=njmax, pad=int(m.nv_pad), nworld=nworld, stage=stage, model=m)
    p.block = 64 if p.pad >= 64 else 32
    p.nefc = np.maximum(b.nefc, 8).astype(np.int32)
    if empty_every:
        p.nefc[3::empty_every] = 0
    p.ne = np.where(p.nefc > 0, 2, 0).astype(np.int32)
    p.nf = np.where(p.nefc > 0, 3, 0).astype(np.int32)
    p.J, p.M = b.J, b.M
    p.D = (10.0 ** rng.uniform(0, 3, (nworld, njmax))).astype(np.float32)
    p.frictionloss = rng.uniform(0.1, 1.0, (nworld, njmax)).astype(np.float32)
    p.aref = rng.normal(scale=2.0, size=(nworld, njmax)).astype(np.float32)
    p.qacc_smooth = rng.normal(size=(nworld, nv)).astype(np.float32)
    p.qacc_warmstart = (p.qacc_smooth + rng.normal(scale=0.1, size=(nworld, nv))).astype(np.float32) if warmstart else None
    p.tables = [np.asarray(a) for a in NF.mul_m_tables(b.rowadr, b.rownnz, b.colind)]
    p.smooth = R.mul_m_sparse(b.M, p.qacc_smooth, *p.tables)
    p.tol, p.ls_tol, p.mi = np.array([1e-7], np.float32), np.array([0.01], np.float32), np.array([1.0], np.float32)
    p.maxiter, p.ls_iterations = maxiter, ls_iterations
    p.st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    if stage == "tree":
        p.tree_plan = P.best_tree_ldl_plan(*p.st)
    if stage == "sparse":
        p.oplan = R.sparse_plan(m, [], p.block)
    return p


def oracle_init(p):
    """The solver's state after the start point and ``init_context``."""
    b, nworld, nv, njmax = p.b, p.nworld, p.nv, p.njmax
    s = SimpleNamespace()
    s.done = (p.nefc == 0).astype(np.uint8)
    start = p.qacc_smooth if p.qacc_warmstart is None else p.qacc_warmstart
    s.qacc = np.where((s.done != 0)[:, None], p.qacc_smooth, start).astype(np.float32)
    s.niter = np.zeros(nworld, np.int32)
    s.Jaref = R.newton_init_jaref(p.J, s.qacc, p.aref, nefc=p.nefc)
    s.Ma = R.mul_m_sparse(b.M, s.qacc, *p.tables)
    old = np.zeros((nworld, njmax), np.int32)
    s.force, s.state, s.ids, s.qc, s.sc = R.newton_eval_constraints(s.Jaref, p.D, p.frictionloss, p.ne, p.nf, p.nefc, old, done=s.done)
    s.alpha, s.improvement = np.zeros(nworld, np.float32), np.zeros(nworld, np.float32)
    zero, one = np.zeros(nworld, np.float32), np.ones(nworld, np.float32)
    every = np.ones(nworld, np.int32)
    s.qfc, s.grad, s.grad_dot, s.decrement, s.grad_scale, s.unchanged = R.newton_gradient(
        p.J, s.force, p.smooth, s.Ma, every, s.alpha, zero, zero, one, nefc=p.nefc, done=s.done, block=p.block)
    live = s.done == 0
    s.search, s.search_dot = np.zeros((nworld, nv), np.float32), np.zeros(nworld, np.float32)
    if p.stage == "dense":
        Md = synth.dense_from_csr(b.M, b.rowadr, b.rownnz, b.colind).astype(np.float32)
        H = R.jtdj_dense(Md.reshape(nworld, -1), p.J, p.D, s.state, p.nefc, p.pad)
        s.H, s.U, s.uni, search, sdot, decr = R.dense_update_factor(every, -every, s.ids, p.J, p.D, s.state, s.grad, H,
                                                                    np.zeros_like(H), done=s.done)  # fmt: skip
    elif p.stage == "sparse":
        s.hf, search, sdot, decr = R.sparse_init_factor(p.oplan, p.nefc, p.J, p.D, s.state, b.M, s.grad, done=s.done)
    else:
        search, sdot, decr = R.newton_tree_stage(*p.st, p.tree_plan, b.M, p.J, p.D, s.state, p.nefc, s.grad, s.done,
                                                 s.search, s.search_dot, s.decrement, block=p.block)  # fmt: skip
    s.search = np.where(live[:, None], search, s.search)
    s.search_dot, s.decrement = np.where(live, sdot, s.search_dot), np.where(live, decr, s.decrement)
    s.unchanged = np.zeros(nworld, np.uint8)  # ctx.search_unchanged.zero_() after init_context
    s.mv, s.jv = np.zeros((nworld, nv), np.float32), np.zeros((nworld, njmax), np.float32)
    s.exhausted, s.overflow = np.zeros(nworld, np.uint8), np.zeros(nworld, np.int32)
    return s


def oracle_iteration(p, s):
    b = p.b
    live = s.done == 0
    s.mv = np.where((s.unchanged != 0)[:, None], s.mv, R.mul_m_sparse(b.M, s.search, *p.tables))
    s.jv = R.newton_jv(p.J, s.search, nefc=p.nefc, skip=s.unchanged, out=s.jv.copy())
    a, imp, ex, ov = R.newton_linesearch(p.tol, p.ls_tol, p.mi, p.ne, p.nf, p.nefc, p.smooth, p.D, p.frictionloss, s.Jaref, s.search,
                                         s.search_dot, s.mv, s.jv, s.Ma, done=s.done, ls_iterations=p.ls_iterations)  # fmt: skip
    s.alpha, s.improvement, s.exhausted = np.where(live, a, s.alpha), np.where(live, imp, s.improvement), np.where(live, ex, s.exhausted)
    s.overflow |= ov
    s.qacc, s.Ma, s.Jaref = R.newton_advance(s.alpha, s.search, s.mv, s.jv, s.qacc, s.Ma, s.Jaref, nefc=p.nefc, done=s.done)
    force, state, ids, s.qc, s.sc = R.newton_eval_constraints(s.Jaref, p.D, p.frictionloss, p.ne, p.nf, p.nefc, s.state, done=s.done, exhausted=s.exhausted)
    s.force, s.state = np.where(live[:, None], force, s.force), state
    s.ids = np.where(live[:, None], ids, s.ids)
    qfc, grad, s.grad_dot, s.decrement, s.grad_scale, s.unchanged = R.newton_gradient(
        p.J, s.force, p.smooth, s.Ma, s.sc, s.alpha, s.grad_dot, s.decrement, s.grad_scale, nefc=p.nefc, done=s.done, block=p.block)
    ran = live & (s.sc != 0)
    s.grad, s.qfc = np.where(ran[:, None], grad, s.grad), np.where(ran[:, None], qfc, s.qfc)
    if p.stage == "dense":
        s.H, s.U, _, search, sdot, decr = R.dense_update_factor(s.sc, s.qc, s.ids, p.J, p.D, s.state, s.grad, s.H, s.U, done=s.done)
    elif p.stage == "sparse":
        s.hf, _, search, sdot, decr = R.sparse_update_factor(p.oplan, s.sc, s.qc, s.ids, p.J, p.D, s.state, s.grad, s.hf, done=s.done)
    else:
        search, sdot, decr = R.newton_tree_stage(*p.st, p.tree_plan, b.M, p.J, p.D, s.state, p.nefc, s.grad, s.unchanged,
                                                 s.search, s.search_dot, s.decrement, block=p.block)  # fmt: skip
    s.search = np.where(ran[:, None], search, s.search)
    s.search_dot, s.decrement = np.where(ran, sdot, s.search_dot), np.where(ran, decr, s.decrement)
    s.niter, s.done, ov2, _ = R.newton_converged(s.alpha, s.improvement, s.grad_dot, s.decrement, p.tol, p.mi, p.nv, p.maxiter, s.niter, s.done, overflow_bit=8)
    s.overflow |= ov2


def oracle_finish(p, s):
    """qfrc_constraint = Ma - qfrc_smooth - grad_scale grad, zero where nefc == 0 (newton_fusion.py:522-539)."""
    g = s.grad_scale[:, None] * s.grad
    out = (s.Ma - p.smooth) - g
    return np.where((p.nefc == 0)[:, None], np.float32(0.0), out).astype(np.float32)


def oracle_solve(p):
    s = oracle_init(p)
    for _ in range(p.maxiter):
        if s.done.all():
            break
        oracle_iteration(p, s)
    s.qfrc_constraint = oracle_finish(p, s)
    return s


def device_objects(p, device, *, poison: bool = True):
    """(m, d, ctx, nsolving) as the reference's step hands them to the solve: inputs filled, every
    array the solve writes poisoned (NaN / -7) so that nothing is taken from a previous step."""
    import torch

    from instantmimic_amd.mjw_kernels import sparse_hessian as S
    from instantmimic_amd.mjw_kernels import tree_ldl as T

    b, nworld, nv, njmax, pad = p.b, p.nworld, p.nv, p.njmax, p.pad
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    nan = float("nan") if poison else 0.0
    f = lambda *shape: torch.full(shape, nan, device=device)  # noqa: E731
    i = lambda *shape: torch.full(shape, -7 if poison else 0, dtype=torch.int32, device=device)  # noqa: E731
    u8 = lambda: torch.full((nworld,), 1 if poison else 0, dtype=torch.uint8, device=device)  # noqa: E731
    m = p.model
    m.M_mulm_rowadr, m.M_mulm_col, m.M_mulm_madr = (t(a) for a in p.tables)
    m.opt = SimpleNamespace(solver=2, cone=0, integrator=3, iterations=p.maxiter, ls_iterations=p.ls_iterations,
                            tolerance=t(p.tol), ls_tolerance=t(p.ls_tol), disableflags=0 if p.qacc_warmstart is not None else 256)  # fmt: skip
    m.stat = SimpleNamespace(meaninertia=t(p.mi))
    d = SimpleNamespace(nworld=nworld, njmax=njmax, M=t(b.M), ne=t(p.ne), nf=t(p.nf), nefc=t(p.nefc), qfrc_smooth=t(p.smooth),
                        qacc_smooth=t(p.qacc_smooth), qacc_warmstart=None if p.qacc_warmstart is None else t(p.qacc_warmstart),
                        qacc=f(nworld, nv), qfrc_constraint=f(nworld, nv), solver_niter=i(nworld),
                        overflow=torch.zeros(nworld, dtype=torch.int32, device=device),
                        efc=SimpleNamespace(J=t(p.J), D=t(p.D), frictionloss=t(p.frictionloss), aref=t(p.aref), Ma=f(nworld, nv),
                                            force=f(nworld, njmax), state=i(nworld, njmax)))  # fmt: skip
    ctx = SimpleNamespace(search=f(nworld, nv), search_dot=f(nworld), mv=f(nworld, nv), jv=f(nworld, njmax), Jaref=f(nworld, njmax),
                          done=u8(), alpha=f(nworld), improvement=f(nworld), ls_exhausted=torch.zeros(nworld, dtype=torch.uint8, device=device),
                          quad_changed_ids=i(nworld, njmax), quad_changed_count=i(nworld), state_changed_count=i(nworld),
                          search_unchanged=u8(), grad=torch.zeros((nworld, pad), device=device), grad_dot=f(nworld),
                          grad_scale=f(nworld), newton_decrement=f(nworld), h=f(nworld, pad, pad),
                          hfactor=torch.zeros((nworld, pad, pad), device=device))  # fmt: skip
    if p.stage == "tree":
        ctx.newton_tree_scratch = T.create_tree_factor_solve_scratch(m, device)
        assert ctx.newton_tree_scratch is not None
    elif p.stage == "sparse":
        plan, reason = S.plan_for_model(m, ctx, [], S.block_width(m.nv_pad), device=device)
        assert plan is not None and plan.path == "fused", reason
        ctx.sparse_hessian_plan = plan
    NF.attach_scratch(m, d, ctx, device)
    nsolving = torch.zeros(1, dtype=torch.int32, device=device)
    return m, d, ctx, nsolving


def compare(p, s, d, ctx) -> None:
    """Every array the solve leaves behind against the oracle's, bit for bit."""
    c = lambda tns: tns.cpu().numpy()  # noqa: E731
    np.testing.assert_array_equal(c(ctx.done), s.done)
    np.testing.assert_array_equal(c(d.solver_niter), s.niter)
    np.testing.assert_array_equal(c(d.qacc), s.qacc)
    np.testing.assert_array_equal(c(d.efc.Ma), s.Ma)
    np.testing.assert_array_equal(c(d.overflow), s.overflow)
    has = p.nefc > 0
    for w_rows, got, want in ((has, c(d.efc.state), s.state), (has, c(d.efc.force), s.force), (has, c(ctx.Jaref), s.Jaref)):
        rows = np.arange(p.njmax)[None, :] < p.nefc[:, None]
        np.testing.assert_array_equal(got[rows], want[rows])
    np.testing.assert_array_equal(c(ctx.grad)[has][:, : p.nv], s.grad[has])
    np.testing.assert_array_equal(c(ctx.search)[has], s.search[has])
    np.testing.assert_array_equal(c(ctx.grad_scale)[has], s.grad_scale[has])
    np.testing.assert_array_equal(c(d.qfrc_constraint), s.qfrc_constraint)
