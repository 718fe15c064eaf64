"""Per-kernel timings of the library on the configured shapes, one JSON line per kernel:

    python -m instantmimic_amd.rowbench [--launches N] [--only trees,generated,stress,muscles,walks,iteration,bodies] [--no-graph]

Every line names the kernel, the workload, the mean time of one launch (event-timed hipGraph
replay over rotating input sets), the algorithmic bytes or flops of that launch and the
fraction of the MI355X roofline that bounds it (HBM 8 TB/s; fp32 matrix cores 157.3 TFLOP/s).
Algorithmic bytes count every input and output array once.
"""

from __future__ import annotations

import argparse
import json
from types import SimpleNamespace

import numpy as np

HBM_GBS = 8000.0
MFMA_F32_TFLOPS = 157.3


GRAPH = True  # False (--no-graph): plain launches, which is what a counter run of rocprofv3 sees per dispatch


def _timeit(torch, fn, nsets: int, launches: int, prime: bool = True) -> float:
    """prime=False: no extra fn(0) ahead of the capture, for a fn that changes its own input (the
    launches of a replay must then leave that input as they found it)."""
    for i in range(min(nsets, 4)):
        fn(i)
    torch.cuda.synchronize()
    if not GRAPH:
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(launches):
            fn(i % nsets)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / launches * 1e-3
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        if prime:
            fn(0)
        with torch.cuda.graph(g, stream=s):
            for i in range(launches):
                fn(i % nsets)
    torch.cuda.current_stream().wait_stream(s)
    g.replay()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(5):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b) / launches * 1e-3)
    return best


def _line(kernel, workload, seconds, *, bytes_=None, flops=None, nworld=None):
    out = {"kernel": kernel, "workload": workload, "us_per_launch": round(seconds * 1e6, 2)}
    if nworld:
        out["worlds_per_s"] = round(nworld / seconds)
    if bytes_ is not None:
        gbs = bytes_ / seconds / 1e9
        out.update(bound="hbm", algorithmic_bytes=int(bytes_), achieved_GBs=round(gbs, 1), frac=round(gbs / HBM_GBS, 4))
    if flops is not None:
        tf = flops / seconds / 1e12
        out.update(bound="mfma", algorithmic_flops=int(flops), achieved_TFLOPs=round(tf, 2), frac=round(tf / MFMA_F32_TFLOPS, 4))
    print(json.dumps(out), flush=True)


def newton_case(name, stage, seed=21, maxiter=10, device="cuda:0"):
    """(m, d, ctx, nsolving) of one step on the tree of `name`: 2 equality rows, 3 friction-loss rows, the
    rest one-sided; everything the solve writes starts as it happens to lie there."""
    import torch

    from . import synth
    from .mjw_kernels import newton_fusion as NF
    from .mjw_kernels import sparse_hessian as SH
    from .mjw_kernels import tree_ldl as T

    dev = torch.device(device)

    def t(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    shape = synth.SHAPES[name]
    b = synth.make_batch(shape, ragged_nefc=True)
    rng = np.random.default_rng(seed)
    nworld, nv, njmax = b.nworld, shape.nv, shape.nefc
    m = synth.model_from_parents(shape.parents)
    pad = int(m.nv_pad)
    nefc = np.maximum(b.nefc, 8).astype(np.int32)
    tables = [t(a) for a in NF.mul_m_tables(b.rowadr, b.rownnz, b.colind)]
    m.M_mulm_rowadr, m.M_mulm_col, m.M_mulm_madr = tables
    m.opt = SimpleNamespace(solver=2, cone=0, integrator=3, iterations=maxiter, ls_iterations=50, disableflags=256,
                            tolerance=torch.full((1,), 1e-7, device=dev), ls_tolerance=torch.full((1,), 0.01, device=dev))  # fmt: skip
    m.stat = SimpleNamespace(meaninertia=torch.ones(1, device=dev))
    f = lambda *shape_: torch.zeros(shape_, device=dev)  # noqa: E731
    i = lambda *shape_: torch.zeros(shape_, dtype=torch.int32, device=dev)  # noqa: E731
    u8 = lambda: torch.zeros(nworld, dtype=torch.uint8, device=dev)  # noqa: E731
    qs = t(rng.normal(size=(nworld, nv)).astype(np.float32))
    M_ = t(b.M)
    smooth = f(nworld, nv)
    NF.mul_m(M_, qs, smooth, *tables)
    d = SimpleNamespace(nworld=nworld, njmax=njmax, M=M_, ne=t(np.full(nworld, 2, np.int32)), nf=t(np.full(nworld, 3, np.int32)),
                        nefc=t(nefc), qfrc_smooth=smooth, qacc_smooth=qs, qacc_warmstart=None, qacc=f(nworld, nv),
                        qfrc_constraint=f(nworld, nv), solver_niter=i(nworld), overflow=i(nworld),
                        efc=SimpleNamespace(J=t(b.J), D=t((10.0 ** rng.uniform(0, 3, (nworld, njmax))).astype(np.float32)),
                                            frictionloss=t(rng.uniform(0.1, 1.0, (nworld, njmax)).astype(np.float32)),
                                            aref=t(rng.normal(scale=2.0, size=(nworld, njmax)).astype(np.float32)),
                                            Ma=f(nworld, nv), force=f(nworld, njmax), state=i(nworld, njmax)))  # fmt: skip
    ctx = SimpleNamespace(search=f(nworld, nv), search_dot=f(nworld), mv=f(nworld, nv), jv=f(nworld, njmax), Jaref=f(nworld, njmax),
                          done=u8(), alpha=f(nworld), improvement=f(nworld), ls_exhausted=u8(), quad_changed_ids=i(nworld, njmax),
                          quad_changed_count=i(nworld), state_changed_count=i(nworld), search_unchanged=u8(), grad=f(nworld, pad),
                          grad_dot=f(nworld), grad_scale=f(nworld), newton_decrement=f(nworld), h=f(nworld, pad, pad),
                          hfactor=f(nworld, pad, pad))  # fmt: skip
    if stage == "tree":
        ctx.newton_tree_scratch = T.create_tree_factor_solve_scratch(m, dev)
    elif stage == "sparse":
        ctx.sparse_hessian_plan, why = SH.plan_for_model(m, ctx, [], SH.block_width(pad), device=dev)
        assert ctx.sparse_hessian_plan is not None, why
    NF.attach_scratch(m, d, ctx, dev)
    return m, d, ctx, torch.zeros(1, dtype=torch.int32, device=dev)


def run(launches: int = 32, only: str | None = None) -> None:
    """``only``: comma-separated section names out of trees, generated, stress, muscles, walks, iteration, solve, implicit, bodies."""
    import torch

    from . import synth
    from .mjw_kernels import blocked_dense as BD
    from .mjw_kernels import newton_fusion as NF
    from .mjw_kernels import newton_stages as NS
    from .mjw_kernels import sparse_hessian as SH
    from .mjw_kernels import tree_fusion as TF
    from .mjw_kernels import tree_ldl as T
    from .muscle import muscle_qfrc_projector as Q
    from .muscle import wrench_projection as WP
    from .muscle.muscle_dynamics import MuscleDynamicsLayer

    dev = torch.device("cuda:0")

    def t(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    def sets_of(arrays, nsets):
        return [[t(a) for a in arrays] for _ in range(nsets)]

    wanted = None if only is None else {w.strip() for w in only.split(",")}

    def section(name):
        return wanted is None or name in wanted

    # ---- a 64 MiB device copy, for scaling the FETCH_SIZE / WRITE_SIZE counters of a profiler run (only when asked for)
    if wanted is not None and "calibration" in wanted:
        src, dst = torch.ones(16 << 20, device=dev), torch.zeros(16 << 20, device=dev)
        sec = _timeit(torch, lambda i: dst.copy_(src), 1, 8)
        _line("64 MiB device copy", "16 Mi floats", sec, bytes_=2 * (64 << 20))
        del src, dst

    # ---- fused assemble + tree L'DL + solve and solve-only on every tree shape
    if section("trees"):
        for name, nsets in (("ant", 8), ("humanoid", 16), ("g1", 8), ("snu", 8)):
            b = synth.make_batch(name)
            nv, nM, nefc, nworld = b.shape.nv, int(b.colind.size), b.shape.nefc, b.nworld
            m = SimpleNamespace(nv=nv, M_rowadr=b.rowadr, M_rownnz=b.rownnz, M_colind=b.colind)
            sc = T.create_tree_factor_solve_scratch(m, dev)
            S = sets_of((b.M, b.J, b.D, b.state[0], b.nefc, b.grad), nsets)
            X = [torch.zeros(b.grad.shape, device=dev) for _ in range(nsets)]
            wl = f"{name} nv={nv} nM={nM} nefc={nefc} x {nworld} worlds"
            sec = _timeit(torch, lambda i: T.assemble_tree_factor_solve(sc, *S[i], X[i]), nsets, launches)
            _line("im_assemble_tree_ldl_solve", wl, sec, bytes_=nworld * 4 * (nM + nefc * nv + 2 * nefc + 2 * nv), nworld=nworld)
            if name != "ant":
                # a step's three Newton iterations in one launch: M and J once, states / gradients / x per iteration
                St = [torch.stack([s[3], 1 - s[3], s[3]]).contiguous() for s in S]
                G3 = [torch.stack([s[5], -s[5], 2 * s[5]]).contiguous() for s in S]
                X3 = [torch.zeros((3,) + tuple(b.grad.shape), device=dev) for _ in range(nsets)]
                sec = _timeit(torch, lambda i: T.assemble_tree_factor_solve_iters(sc, S[i][0], S[i][1], S[i][2], St[i], S[i][4], G3[i], X3[i]), nsets, launches)
                _line("im_assemble_tree_ldl_solve_iters (3 iterations, bytes of three separate solves)", wl, sec,
                      bytes_=3 * nworld * 4 * (nM + nefc * nv + 2 * nefc + 2 * nv), nworld=3 * nworld)  # fmt: skip
                del St, G3, X3
            sec = _timeit(torch, lambda i: T.tree_factor_solve(sc, S[i][0], X[i], S[i][5]), nsets, launches)
            _line("im_tree_factor_solve", wl, sec, bytes_=nworld * 4 * (nM + 2 * nv), nworld=nworld)
            if nv <= 32:
                # the same solve through one Cholesky tile gathered from M's structure (no factor kept)
                ids = synth.matrix_elemid(b.rowadr, b.rownnz, b.colind)
                tile = SimpleNamespace(size=nv, adr=torch.zeros(1, dtype=torch.int32, device=dev), elemid=t(np.where(ids < 0, nM, ids).astype(np.int32).reshape(-1)))
                mt = SimpleNamespace(M_tiles=[tile], nv=nv, qLD_block_total=0)
                dt = SimpleNamespace(nworld=nworld, qLD=torch.zeros((nworld, 0), device=dev))
                sec = _timeit(torch, lambda i: BD._factor_solve_i_dense(mt, dt, S[i][0], X[i], S[i][5]), nsets, launches)
                _line("im_tile_cholesky_solve_m", wl, sec, bytes_=nworld * 4 * (nM + 2 * nv), nworld=nworld)
            if name != "ant":
                # the dense Newton's first Hessian and factor as one launch (M through the element table, J'DJ, the stage)
                pad = (nv // 16 + 1) * 16
                eid = t(NF.elemid_table(b.rowadr, b.rownnz, b.colind))
                Hd, Ud = torch.zeros((nworld, pad, pad), device=dev), torch.zeros((nworld, pad, pad), device=dev)
                un = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=dev)
                se = torch.zeros((nworld, nv), device=dev)
                sd_, de_ = torch.zeros(nworld, device=dev), torch.zeros(nworld, device=dev)
                ok = BD.dense_init_factor(S[0][0], eid, S[0][1], S[0][2], S[0][3], S[0][4], None, S[0][5], Hd, Ud, se, sd_, de_, un)
                assert ok, "no one-launch dense first factor for this shape"
                sec = _timeit(torch, lambda i: BD.dense_init_factor(S[i][0], eid, S[i][1], S[i][2], S[i][3], S[i][4], None, S[i][5], Hd, Ud, se, sd_, de_, un), nsets, launches)
                _line("im_dense_init_factor (M + J'DJ, factor, solve)", wl, sec,
                      bytes_=nworld * 4 * (nM + nefc * nv + 2 * nefc + 2 * nv + pad * pad + (pad * pad if nv > 32 else 0) + 2), nworld=nworld)  # fmt: skip
                del Hd, Ud
            if name in ("g1", "snu"):
                # the same Hessians through the blocked dense factor and the static-pattern sparse L'DL
                Md = synth.dense_from_csr(b.M, b.rowadr, b.rownnz, b.colind).astype(np.float32).reshape(nworld, -1)
                mm = SimpleNamespace(nv=nv, M_tiles=[SimpleNamespace(size=nv, elemid=np.arange(nv * nv))])
                for B in (8, 16):
                    Mt = [t(Md) for _ in range(4)]
                    d = SimpleNamespace(nworld=nworld, M=Mt[0])
                    bs = BD.create_blocked_dense_factor_solve_scratch(mm, d, dev, block_size=B)
                    Y = t(b.grad).reshape(nworld, nv, 1)
                    Xb = torch.zeros_like(Y)
                    sec = _timeit(torch, lambda i: BD._blocked_dense_factor_solve(d, Mt[i], Xb, Y, bs), 4, launches)
                    _line(f"im_blocked_factor_solve B={B}", wl, sec, bytes_=nworld * 4 * (nv * nv + 2 * nv + bs.pad * bs.pad), nworld=nworld)
                model = synth.model_from_parents(b.shape.parents)
                plan, _ = SH.plan_for_model(model, None, [], SH.block_width(model.nv_pad), device=dev)
                if plan is not None:
                    launch = SH.init_factor_kernel(plan)
                    hf = torch.zeros((nworld, plan.nv_pad, plan.nv_pad), device=dev)
                    search = torch.zeros((nworld, nv, 1), device=dev)
                    sd, de = torch.zeros(nworld, device=dev), torch.zeros(nworld, device=dev)
                    G = [s[5][:, :, None].contiguous() for s in S]
                    sec = _timeit(torch, lambda i: launch(None, S[i][4], S[i][1], S[i][2], S[i][3], S[i][0], G[i], hf, search, sd, de), nsets, launches)
                    used = 2 * plan.nfac + nv
                    _line("im_sparse_init_factor", wl, sec, bytes_=nworld * 4 * (nM + nefc * nv + 2 * nefc + 2 * nv + used + 2), nworld=nworld)
                    # per-iteration stage: a tenth of the rows change state.  The stage updates the packed H
                    # in hfactor in place, so launches alternate between the mask the factor was made
                    # with and the one with those rows flipped: H goes there and back and stays a Hessian.
                    rng = np.random.default_rng(1)
                    ids = np.zeros((nworld, nefc), np.int32)
                    k = max(nefc // 10, 1)
                    for w in range(nworld):
                        ids[w, :k] = np.sort(rng.choice(nefc, k, replace=False))
                    chg = t(np.full(nworld, k, np.int32))
                    uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=dev)
                    stage = NS.factor_factory(nv, plan.nv_pad, plan)
                    s2 = search.reshape(nworld, nv)
                    idt = t(ids)
                    st0 = b.state[0]
                    flip = np.zeros((nworld, nefc), bool)
                    np.put_along_axis(flip, ids[:, :k], True, axis=1)
                    st1 = t(np.where(flip, np.where(st0 == synth.QUADRATIC, 0, synth.QUADRATIC), st0).astype(np.int32))
                    launch(None, S[0][4], S[0][1], S[0][2], S[0][3], S[0][0], G[0], hf, search, sd, de)  # the factor of the first mask
                    sec = _timeit(torch, lambda i: stage(S[i][1], S[i][2], st1 if i % 2 == 0 else S[i][3], idt, chg, chg, None, S[i][5], None, hf, s2, sd, de, uni),
                                  nsets, launches, prime=False)
                    assert bool(torch.isfinite(s2).all()), "the stage's matrices left the solver's range"
                    _line("im_sparse_update_factor", wl + f", {k} changed rows", sec, bytes_=nworld * 4 * (k * nv + 2 * used + 2 * nv + nv + 1 + 2), nworld=nworld)
            del S, X
            torch.cuda.empty_cache()

    # ---- trees beside the benchmark shapes: kernels generated and compiled when the plan is created
    if section("generated"):
        import os

        for name, parents in synth.extra_trees().items():
            if name not in ("limbs", "branched", "limbs62", "limbs70", "limbs78"):
                continue
            shape = synth.Shape(name, tuple(parents), 64, 4096, (0.5, 8.0), 0.02, (-4.0, 4.0), 0.6, 3, 1001)
            b = synth.make_batch(shape)
            nv, nM, nefc, nworld = b.shape.nv, int(b.colind.size), b.shape.nefc, b.nworld
            m = SimpleNamespace(nv=nv, M_rowadr=b.rowadr, M_rownnz=b.rownnz, M_colind=b.colind)
            S = sets_of((b.M, b.J, b.D, b.state[0], b.nefc, b.grad), 8)
            X = [torch.zeros(b.grad.shape, device=dev) for _ in range(8)]
            wl = f"{name} nv={nv} nM={nM} nefc={nefc} x {nworld} worlds"
            for kind in ("generated", "table-driven") if nv <= 64 else ("generated",):  # beyond 64 dofs: generated kernels only
                if kind == "table-driven":
                    os.environ["IMHIP_TREE_KERNEL"] = "generic"
                try:
                    sc = T.create_tree_factor_solve_scratch(m, dev)
                finally:
                    os.environ.pop("IMHIP_TREE_KERNEL", None)
                sec = _timeit(torch, lambda i: T.assemble_tree_factor_solve(sc, *S[i], X[i]), 8, launches)
                _line(f"im_assemble_tree_ldl_solve ({kind} kernel)", wl, sec, bytes_=nworld * 4 * (nM + nefc * nv + 2 * nefc + 2 * nv), nworld=nworld)
            if nv > 64:
                # the same assemble + factor + solve on the static sparse pattern and on the dense matrix:
                # the sizes at which the reference's sparse path is its fastest (sparse_hessian.py:179-183)
                model = synth.model_from_parents(list(parents))
                pad = int(model.nv_pad)
                plan, why = SH.plan_for_model(model, None, [], SH.block_width(pad), device=dev)
                if plan is not None:
                    launch = SH.init_factor_kernel(plan)
                    hf = torch.zeros((nworld, plan.nv_pad, plan.nv_pad), device=dev)
                    search = torch.zeros((nworld, nv, 1), device=dev)
                    sd, de = torch.zeros(nworld, device=dev), torch.zeros(nworld, device=dev)
                    G = [s_[5][:, :, None].contiguous() for s_ in S]
                    sec = _timeit(torch, lambda i: launch(None, S[i][4], S[i][1], S[i][2], S[i][3], S[i][0], G[i], hf, search, sd, de), 8, launches)
                    _line("im_sparse_init_factor (workgroup per world: beyond 64 dofs)", wl, sec,
                          bytes_=nworld * 4 * (nM + nefc * nv + 2 * nefc + 2 * nv + 2 * plan.nfac + nv + 2), nworld=nworld)  # fmt: skip
                    del hf, G
                else:
                    print(json.dumps({"kernel": "im_sparse_init_factor", "workload": wl, "refused": why}), flush=True)
                Md = [t(synth.dense_from_csr(b.M, b.rowadr, b.rownnz, b.colind).astype(np.float32).reshape(nworld, -1)) for _ in range(2)]
                Hd = torch.zeros((nworld, pad, pad), device=dev)
                padU = -(-nv // 16) * 16
                Ud = torch.zeros((nworld, padU, padU), device=dev)
                sec = _timeit(torch, lambda i: BD.dense_hessian_factor_solve(Md[i % 2], S[i][1], S[i][2], S[i][3], S[i][4], Hd, S[i][5], X[i], factor=Ud), 8, launches)
                _line("im_jtdj_factor_solve (dense J'DJ + blocked factor + solve)", wl, sec,
                      bytes_=nworld * 4 * (nv * nv + nefc * nv + 2 * nefc + 2 * nv + pad * pad + padU * padU), nworld=nworld)  # fmt: skip
                del Md, Hd, Ud
            del S, X
            torch.cuda.empty_cache()

    # ---- stress: dense J'DJ on the matrix cores, blocked factor, dense per-iteration stage
    if section("stress"):
        b = synth.make_batch("stress", 16384)
        nv, nefc, nworld = b.shape.nv, b.shape.nefc, b.nworld
        pad = ((nv + 1 + 15) // 16) * 16
        Md = t(synth.dense_from_csr(b.M, b.rowadr, b.rownnz, b.colind).astype(np.float32).reshape(nworld, -1))
        J, D, st, ne, g = (t(a) for a in (b.J, b.D, b.state[0], b.nefc, b.grad))
        H = torch.zeros((nworld, pad, pad), device=dev)
        wl = f"stress nv={nv} nefc={nefc} x {nworld} worlds"
        sec = _timeit(torch, lambda i: BD.dense_hessian(Md, J, D, st, ne, H), 1, 8)
        # the product the matrix cores execute: the 16 x 16 tiles on and right of the diagonal blocks, over the first 32 rows
        # and the contributing rows behind them in chunks of 32 (the full square over every row would be 2 nv^2 nefc)
        tail = ((b.state[0][:, 32:] == synth.QUADRATIC) & (np.arange(32, nefc)[None, :] < b.nefc[:, None])).sum(1)
        chunks = np.where(b.nefc > 0, 1 + (tail + 31) // 32, 0)
        nb16 = (nv + 15) // 16
        _line("im_jtdj_mfma (flops executed on the matrix cores)", wl, sec, flops=float(chunks.sum()) * 32 * (nb16 * (nb16 + 1) // 2) * 512, nworld=nworld)
        _line("im_jtdj_mfma (as bytes)", wl, sec, bytes_=nworld * 4 * (nv * nv + nefc * nv + 2 * nefc + pad * pad), nworld=nworld)
        mm = SimpleNamespace(nv=nv, M_tiles=[SimpleNamespace(size=nv, elemid=np.arange(nv * nv))])
        Hc = H[:, :nv, :nv].contiguous().reshape(nworld, -1)
        d = SimpleNamespace(nworld=nworld, M=Hc)
        bs = BD.create_blocked_dense_factor_solve_scratch(mm, d, dev, block_size=16)
        Y = g.reshape(nworld, nv, 1)
        Xb = torch.zeros_like(Y)
        sec = _timeit(torch, lambda i: BD._blocked_dense_factor_solve(d, Hc, Xb, Y, bs), 1, 8)
        _line("im_blocked_factor_solve B=16", wl, sec, bytes_=nworld * 4 * (nv * nv + 2 * nv + bs.pad * bs.pad), nworld=nworld)
        Uf, xf = torch.zeros((nworld, bs.pad, bs.pad), device=dev), torch.zeros((nworld, nv), device=dev)
        sec = _timeit(torch, lambda i: BD.dense_hessian_factor_solve(Md, J, D, st, ne, H, g, xf, factor=Uf), 1, 8)
        _line("im_jtdj_factor_solve (J'DJ + blocked factor + solve in one launch)", wl, sec,
              bytes_=nworld * 4 * (nv * nv + nefc * nv + 2 * nefc + pad * pad + bs.pad * bs.pad + 2 * nv), nworld=nworld)  # fmt: skip
        # The stage updates H in place, so a launch's input is the launch before's output.  Launches
        # alternate between two active masks that differ in the changed rows: rows enter and leave,
        # H goes from the Hessian of one mask to that of the other and back, and stays what a solver
        # would hand over.  (With one mask applied over and over the rows that left are subtracted
        # again and again, H stops being positive definite, and every diagonal tile falls back to the
        # library square root.)
        rng = np.random.default_rng(2)
        uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=dev)
        U = torch.zeros((nworld, pad, pad), device=dev)
        g3 = torch.zeros((nworld, pad, 1), device=dev)
        g3[:, :nv, 0] = g
        search = torch.zeros((nworld, pad, 1), device=dev)
        sd, de = torch.zeros(nworld, device=dev), torch.zeros(nworld, device=dev)
        stage = NS.factor_factory(nv, pad)
        st0 = b.state[0]
        for label in ("flip", "fresh"):
            if label == "flip":  # a tenth of the rows change state
                k = nefc // 10
                flip = np.zeros((nworld, nefc), bool)
                np.put_along_axis(flip, rng.permuted(np.tile(np.arange(nefc), (nworld, 1)), axis=1)[:, :k], True, axis=1)
                st1 = np.where(flip, np.where(st0 == synth.QUADRATIC, 0, synth.QUADRATIC), st0).astype(np.int32)
            else:  # a fresh active mask
                st1 = np.where(rng.uniform(size=st0.shape) < b.shape.p_active, synth.QUADRATIC, 0).astype(np.int32)
            differ = (st1 == synth.QUADRATIC) != (st0 == synth.QUADRATIC)
            counts = differ.sum(1).astype(np.int32)
            ids = np.zeros((nworld, nefc), np.int32)
            order = np.argsort(~differ, axis=1, kind="stable")  # the differing rows first, ascending
            ids[:] = np.where(np.arange(nefc)[None, :] < counts[:, None], order, 0)
            idt, chg, masks = t(ids), t(counts), [t(st1), st]
            BD.dense_hessian(Md, J, D, st, ne, H)  # H of the first mask, whatever ran before
            sec = _timeit(torch, lambda i: stage(J, D, masks[i % 2], idt, chg, chg, None, g3, H, U, search, sd, de, uni), 2, 8, prime=False)
            assert bool(torch.isfinite(search[:, :nv]).all()), "the stage's matrices left the solver's range"
            kmean = float(counts.mean())
            note = f", {kmean:.0f} changed rows" + (" (a fresh active mask)" if label == "fresh" else "")
            _line("im_dense_update_factor", wl + note, sec, bytes_=nworld * 4 * (kmean * nv + 2 * pad * pad + 2 * nv), nworld=nworld)
        del J, H, U, Md, Hc
        torch.cuda.empty_cache()

    # ---- muscles on the SNU-like tree
    if section("muscles"):
        nworld = 4096
        mb = synth.make_muscles(nworld)
        rowadr, rownnz, colind = synth.csr_from_parents(synth.snu_parents())
        nv, nM = len(rowadr), int(colind.size)
        ent = Q.entries_from_muscle_dofs(mb.muscle_dofs, mb.nmuscle)
        ne_ = len(ent.muscle_dof_torque_idx)
        offsets, order = Q.torque_sorted_entries(ent.muscle_dof_torque_idx, nv - mb.root_dof_count)
        nsets = 8
        mom = [t(mb.moment) for _ in range(nsets)]
        frc = [t(mb.force) for _ in range(nsets)]
        slope = [t(mb.slope) for _ in range(nsets)]
        qfrc = torch.zeros((nworld, nv), device=dev)
        off_d, ord_d, em_d = t(offsets), t(order), t(ent.muscle_dof_muscle_idx.astype(np.int32))
        wl = f"snu nv={nv} muscles={mb.nmuscle} entries={ne_} x {nworld} worlds"
        sec = _timeit(torch, lambda i: Q.project_muscle_sparse_moment_qfrc(mom[i], frc[i], off_d, ord_d, em_d, mb.root_dof_count, qfrc), nsets, launches)
        _line("im_muscle_project", wl, sec, bytes_=nworld * 4 * (ne_ + mb.nmuscle + nv - mb.root_dof_count), nworld=nworld)
        prepared = Q.prepare_muscle_implicit_qderiv_pairs(
            pair_entry_i=ent.pair_entry_i, pair_entry_j=ent.pair_entry_j, pair_muscle_idx=ent.pair_muscle_idx,
            muscle_dof_torque_idx=ent.muscle_dof_torque_idx, matrix_elemid=synth.matrix_elemid(rowadr, rownnz, colind),
            root_dof_count=mb.root_dof_count,
        )  # fmt: skip
        gather = Q.build_muscle_implicit_qderiv_gather(prepared, ent.muscle_dof_muscle_idx, dev)
        qd = torch.zeros((nworld, nM), device=dev)
        sec = _timeit(torch, lambda i: Q.apply_muscle_implicit_qderiv_gather(gather, mom[i], slope[i], mb.timestep, qd), nsets, launches)
        touched = int(gather.elem_ids.numel())
        _line("im_muscle_implicit_gather", wl, sec, bytes_=nworld * 4 * (ne_ + mb.nmuscle + 2 * touched), nworld=nworld)
        # the muscle terms into the fused solve: h A'sA into M, tau = A'f out of the right-hand side, solve
        b = synth.make_batch("snu")
        sc = T.create_tree_factor_solve_scratch(SimpleNamespace(nv=nv, M_rowadr=b.rowadr, M_rownnz=b.rownnz, M_colind=b.colind), dev)
        S = sets_of((b.M, b.J, b.D, b.state[0], b.nefc, b.grad), nsets)
        Mq = [torch.empty_like(s[0]) for s in S]
        rhs, xs = torch.zeros((nworld, nv), device=dev), torch.zeros((nworld, nv), device=dev)
        nefc = b.shape.nefc

        def chain(i):
            Mq[i].copy_(S[i][0])
            Q.apply_muscle_implicit_qderiv_gather(gather, mom[i], slope[i], mb.timestep, Mq[i])
            Q.project_muscle_sparse_moment_qfrc(mom[i], frc[i], off_d, ord_d, em_d, mb.root_dof_count, qfrc)
            torch.sub(S[i][5], qfrc, out=rhs)
            T.assemble_tree_factor_solve(sc, Mq[i], S[i][1], S[i][2], S[i][3], S[i][4], rhs, xs)

        sec = _timeit(torch, chain, nsets, launches)
        _line("muscle terms + fused solve: copy M, im_muscle_implicit_gather, im_muscle_project, subtract, im_assemble_tree_ldl_solve (five launches)",
              wl + f" nefc={nefc}", sec, bytes_=nworld * 4 * (2 * ne_ + 2 * mb.nmuscle + nM + nefc * nv + 2 * nefc + 2 * nv), nworld=nworld)  # fmt: skip
        # the slope's producer
        ws = np.concatenate([[0], np.cumsum(np.full(mb.nmuscle, 4))]).astype(np.int32)
        rngm = np.random.default_rng(4)
        wps = [torch.randn((nworld, int(ws[-1]), 3), device=dev) for _ in range(4)]
        par = t(np.stack([rngm.uniform(100, 3000, mb.nmuscle), rngm.uniform(0.5, 1.5, mb.nmuscle), rngm.uniform(0, 0.5, mb.nmuscle), rngm.uniform(0, 0.5, mb.nmuscle)], 1).astype(np.float32))
        rest, scale = t(rngm.uniform(2, 6, mb.nmuscle).astype(np.float32)), t(rngm.uniform(0.1, 0.5, mb.nmuscle).astype(np.float32))
        actv, qv = torch.rand((nworld, mb.nmuscle), device=dev), torch.randn((nworld, nv), device=dev)
        outs = [torch.zeros((nworld, mb.nmuscle), device=dev) for _ in range(5)]
        ws_d = t(ws)
        dof_off, dof_tq = t(ent.muscle_dof_offsets.astype(np.int32)), t(ent.muscle_dof_torque_idx.astype(np.int32))
        sec = _timeit(
            torch,
            lambda i: Q.eval_muscle_force_velocity_state(
                wps[i], ws_d, par, rest, scale, actv, qv, mom[i], dof_off, dof_tq, mb.root_dof_count,
                muscle_force_scale=1.0, muscle_length_norm_min=0.4, muscle_length_norm_max=1.6, vmax=1.5, fvmax=1.4,
                clamp_activation=True, include_active=True, active_force_model_params=np.array([1.0, 0.5, 1.6], np.float32),
                muscle_length=outs[0], effective_activation=outs[1], length_velocity=outs[2],
                force_velocity_multiplier=outs[3], force_velocity_slope=outs[4],
            ),
            4, launches,
        )  # fmt: skip
        _line("im_muscle_force_velocity_state", wl + f", {int(ws[-1])} waypoints", sec,
              bytes_=nworld * 4 * (3 * int(ws[-1]) + ne_ + nv + mb.nmuscle + 5 * mb.nmuscle), nworld=nworld)  # fmt: skip
        del S, Mq
        rig = synth.make_muscle_rig()
        layer = MuscleDynamicsLayer(rig.topology, **rig.dims(), device=dev)
        ctx = [t(synth.make_muscle_context(rig, nworld, seed=s)) for s in range(4)]
        act = torch.rand((nworld, rig.muscle_count), device=dev)
        gout = torch.randn((nworld, rig.torque_dim), device=dev)
        wl = (f"snu rig: {rig.muscle_count} muscles, {layer.waypoint_count} waypoints, {len(layer.segments_host[0])} applied "
              f"segments, {len(layer.torque_entries_host[2])} torque entries x {nworld} worlds")  # fmt: skip
        cbytes = 4 * layer.context_dim
        sec = _timeit(torch, lambda i: layer._warp_muscle_dynamics_from_activation_forward(act, ctx[i], include_passive_force=True), 4, launches)
        _line("torque_forward (waypoints + force magnitudes + im_muscle_torque_forward)", wl, sec,
              bytes_=nworld * (cbytes + 4 * (3 * layer.waypoint_count * 2 + 3 * rig.muscle_count + rig.muscle_count + rig.torque_dim)), nworld=nworld)  # fmt: skip
        sec = _timeit(torch, lambda i: layer._warp_muscle_dynamics_from_activation_backward(ctx[i], gout), 4, launches)
        _line("torque_backward (waypoints + force magnitudes + im_muscle_activation_grad)", wl, sec,
              bytes_=nworld * (cbytes + 4 * (3 * layer.waypoint_count * 2 + 2 * rig.muscle_count + rig.muscle_count + rig.torque_dim)), nworld=nworld)  # fmt: skip
        sec = _timeit(torch, lambda i: layer.eval_muscle_sparse_moment(ctx[i]), 4, launches)
        _line("eval_muscle_sparse_moment (waypoints + im_muscle_sparse_moment)", wl, sec,
              bytes_=nworld * (cbytes + 4 * (3 * layer.waypoint_count * 2 + len(layer.sparse_entries.muscle_dof_torque_idx))), nworld=nworld)  # fmt: skip

    # ---- the tree walks either side of the solve
    if section("walks"):
        for name, nsets in (("humanoid", 16), ("snu", 8)):
            b = synth.make_batch(name)
            nv, nM, nworld = b.shape.nv, int(b.colind.size), b.nworld
            tables = [t(a) for a in NF.mul_m_tables(b.rowadr, b.rownnz, b.colind)]
            Ms, Vs = [t(b.M) for _ in range(nsets)], [t(b.grad) for _ in range(nsets)]
            out = torch.zeros((nworld, nv), device=dev)
            sec = _timeit(torch, lambda i: NF.mul_m(Ms[i], Vs[i], out, *tables), nsets, launches)
            _line("im_mul_m_sparse", f"{name} nv={nv} nM={nM} x {nworld} worlds", sec, bytes_=nworld * 4 * (nM + 2 * nv), nworld=nworld)
        for name, nsets in (("humanoid", 16), ("g1", 8), ("snu", 8)):
            b = synth.make_batch(name)
            nv, nefc, nworld = b.shape.nv, b.shape.nefc, b.nworld
            # a constraint's force is zero unless its state is quadratic, as after the reference's update of the constraints
            quad_rows = t(b.state[0] == synth.QUADRATIC)
            Js, Fs = [t(b.J) for _ in range(nsets)], [torch.randn((nworld, nefc), device=dev) * quad_rows for _ in range(nsets)]
            ne, sm, ma = t(b.nefc), t(b.grad), torch.randn((nworld, nv), device=dev)
            chg, al = torch.ones(nworld, dtype=torch.int32, device=dev), torch.zeros(nworld, device=dev)
            qc, gr = torch.zeros((nworld, nv), device=dev), torch.zeros((nworld, nv), device=dev)
            gd, de, sc = (torch.zeros(nworld, device=dev) for _ in range(3))
            un = torch.zeros(nworld, dtype=torch.uint8, device=dev)
            sec = _timeit(torch, lambda i: NF.gradient(ne, Js[i], Fs[i], sm, ma, chg, al, None, qc, gr, gd, de, sc, un), nsets, launches)
            _line("im_newton_gradient", f"{name} nv={nv} nefc={nefc} x {nworld} worlds", sec,
                  bytes_=nworld * 4 * (nefc * nv + nefc + 4 * nv + 6), nworld=nworld)  # fmt: skip
            jvo = torch.zeros((nworld, nefc), device=dev)
            sec = _timeit(torch, lambda i: NF.jv(Js[i], sm, jvo, nefc=ne), nsets, launches)
            _line("im_newton_jv", f"{name} nv={nv} nefc={nefc} x {nworld} worlds", sec, bytes_=nworld * 4 * (nefc * nv + nefc + nv), nworld=nworld)

    # ---- one Newton iteration from the library's pieces, tree path, humanoid
    if section("iteration"):
        b = synth.make_batch("humanoid")
        nv, nM, nefc, nworld = b.shape.nv, int(b.colind.size), b.shape.nefc, b.nworld
        sc_tree = T.create_tree_factor_solve_scratch(SimpleNamespace(nv=nv, M_rowadr=b.rowadr, M_rownnz=b.rownnz, M_colind=b.colind), dev)
        nsets = 16
        S = sets_of((b.M, b.J, b.D, b.state[0], b.state[1], b.nefc), nsets)
        f32 = lambda *shape: torch.randn(shape, device=dev)  # noqa: E731
        i32 = lambda: torch.zeros(nworld, dtype=torch.int32, device=dev)  # noqa: E731
        search, mvv, qacc, Ma, smooth, force = f32(nworld, nv), f32(nworld, nv), f32(nworld, nv), f32(nworld, nv), f32(nworld, nv), f32(nworld, nefc)
        jvv, jaref, alpha = torch.zeros((nworld, nefc), device=dev), f32(nworld, nefc), torch.rand(nworld, device=dev)
        ids, qcnt, scnt, nit = torch.zeros((nworld, nefc), dtype=torch.int32, device=dev), i32(), i32(), i32()
        qc, gr = torch.zeros((nworld, nv), device=dev), torch.zeros((nworld, nv), device=dev)
        gd, de, gs, imp = (torch.ones(nworld, device=dev) for _ in range(4))
        un, dn = torch.zeros(nworld, dtype=torch.uint8, device=dev), torch.zeros(nworld, dtype=torch.uint8, device=dev)
        tol, inertia = torch.full((1,), 1e-30, device=dev), torch.ones(1, device=dev)

        def iteration(i):
            M_, J_, D_, s0, s1, ne_ = S[i]
            NF.jv(J_, search, jvv, nefc=ne_, skip_world=dn)
            NF.advance(alpha, search, mvv, jvv, qacc, Ma, jaref, nefc=ne_, done=dn)
            NF.changed_rows(s0, s1, ids, qcnt, scnt, nefc=ne_, done=dn)
            NF.gradient(ne_, J_, force, smooth, Ma, scnt, alpha, dn, qc, gr, gd, de, gs, un)
            T.assemble_tree_factor_solve(sc_tree, M_, J_, D_, s1, ne_, gr, search, negate=True)
            NF.converged(alpha, imp, gd, de, tol, inertia, nv, 1 << 30, nit, dn)

        sec = _timeit(torch, iteration, nsets, launches)
        _line("one Newton iteration: jv, step, changed rows, gradient, fused tree solve, convergence test (six launches)",
              f"humanoid nv={nv} nefc={nefc} x {nworld} worlds", sec,
              bytes_=nworld * 4 * (3 * nefc * nv + nM + 8 * nefc + 12 * nv + 10), nworld=nworld)  # fmt: skip

        # the line search on a consistent problem: search = -H^-1 grad of the first iteration, mv = M search and
        # jv = J search from the library's own kernels, one-sided rows only; then the whole iteration of
        # newton_fusion.iteration (eight launches: M search, J search, scalar search, step, constraints, gradient,
        # fused tree solve, convergence test)
        tables = [t(a) for a in NF.mul_m_tables(b.rowadr, b.rownnz, b.colind)]
        M0, J0, D0, st0, _, ne0 = S[0]
        qacc0 = 0.1 * f32(nworld, nv)
        Ma0, jar0, sr0 = torch.zeros((nworld, nv), device=dev), torch.zeros((nworld, nefc), device=dev), torch.zeros((nworld, nv), device=dev)
        NF.mul_m(M0, qacc0, Ma0, *tables)
        NF.jv(J0, qacc0, jar0, nefc=ne0)
        jar0 += 0.3 * f32(nworld, nefc)  # J qacc - aref
        grad0 = t(b.grad)
        T.assemble_tree_factor_solve(sc_tree, M0, J0, D0, st0, ne0, grad0, sr0, negate=True)
        sdot0 = (sr0 * sr0).sum(1)
        mv0, jv0 = torch.zeros((nworld, nv), device=dev), torch.zeros((nworld, nefc), device=dev)
        NF.mul_m(M0, sr0, mv0, *tables)
        NF.jv(J0, sr0, jv0, nefc=ne0)
        smooth0 = Ma0 - grad0  # so that the unconstrained gradient is the batch's
        ls_tol, tol8 = torch.full((1,), 0.01, device=dev), torch.full((1,), 1e-8, device=dev)
        al, im_, ex = torch.zeros(nworld, device=dev), torch.zeros(nworld, device=dev), torch.zeros(nworld, dtype=torch.uint8, device=dev)
        ovf = torch.zeros(nworld, dtype=torch.int32, device=dev)
        sec = _timeit(torch, lambda i: NF.linesearch(tol8, ls_tol, inertia, None, None, ne0, smooth0, D0, None, jar0, sr0, sdot0, mv0, jv0, Ma0, None,
                                                     al, im_, ex, ls_iterations=50, overflow=ovf, overflow_bit=4), 1, launches)  # fmt: skip
        _line("im_newton_linesearch (up to 50 rounds of three candidates)", f"humanoid nv={nv} nefc={nefc} x {nworld} worlds", sec,
              bytes_=nworld * 4 * (4 * nefc + 5 * nv + 6), nworld=nworld)  # fmt: skip
        frc, est = torch.zeros((nworld, nefc), device=dev), torch.zeros((nworld, nefc), dtype=torch.int32, device=dev)
        sec = _timeit(torch, lambda i: NF.eval_constraints(jar0, D0, None, None, None, ne0, None, ex, frc, est, ids, qcnt, scnt), 1, launches)
        _line("im_newton_eval_constraints", f"humanoid nv={nv} nefc={nefc} x {nworld} worlds", sec,
              bytes_=nworld * 4 * (5 * nefc + 3), nworld=nworld)  # fmt: skip
        mm = SimpleNamespace(nv=nv, nv_pad=(nv + 1 + 15) // 16 * 16, M_mulm_rowadr=tables[0], M_mulm_col=tables[1], M_mulm_madr=tables[2],
                             opt=SimpleNamespace(tolerance=tol8, ls_tolerance=ls_tol, iterations=1 << 30, ls_iterations=50),
                             stat=SimpleNamespace(meaninertia=inertia), block_dim=SimpleNamespace(linesearch_iterative=32))  # fmt: skip

        def tree_stage(J_, D_, state_, ids_, qcnt_, scnt_, done_, grad_, h_, hfactor_, search_, sdot_, decr_, union_):
            T.assemble_tree_factor_solve(sc_tree, M0, J_, D_, state_, ne0, grad_[:, :nv], search_, negate=True)

        def whole(i):
            M_, J_, D_, s0, _, ne_ = S[i]
            dd = SimpleNamespace(nworld=nworld, M=M_, ne=None, nf=None, nefc=ne_, qfrc_smooth=smooth0, qacc=qacc0,
                                 efc=SimpleNamespace(J=J_, D=D_, frictionloss=None, Ma=Ma0, force=frc, state=est),
                                 qfrc_constraint=qc, solver_niter=nit, overflow=ovf)  # fmt: skip
            cx = SimpleNamespace(search=sr0, search_dot=sdot0, mv=mv0, jv=jv0, Jaref=jar0, done=dn, alpha=al, improvement=im_,
                                 ls_exhausted=ex, quad_changed_ids=ids, quad_changed_count=qcnt, state_changed_count=scnt,
                                 search_unchanged=un, grad=gr, grad_dot=gd, grad_scale=gs, newton_decrement=de, h=None, hfactor=None,
                                 newton_dof_union=None)  # fmt: skip
            NF.iteration(mm, dd, cx, None, stage=tree_stage)

        sec = _timeit(torch, whole, nsets, launches)
        _line("newton_fusion.iteration: M search, J search, line search, step, constraints, gradient, fused tree solve, convergence test (eight launches)",
              f"humanoid nv={nv} nefc={nefc} x {nworld} worlds", sec,
              bytes_=nworld * 4 * (3 * nefc * nv + 2 * nM + 14 * nefc + 20 * nv + 16), nworld=nworld)  # fmt: skip

    # ---- whole constraint solves with dependent iterations: init_context, the Newton loop, the force recovery
    if section("solve"):
        import os


        for name, stage, loop in (("humanoid", "tree", "resident"), ("humanoid", "tree", "stages"), ("humanoid", "dense", "resident"), ("humanoid", "dense", "stages"),
                                  ("g1", "dense", "resident"), ("g1", "dense", "stages"), ("g1", "tree", "resident"), ("g1", "tree", "stages"), ("g1", "sparse", "resident"), ("g1", "sparse", "stages"),
                                  ("snu", "dense", "resident"), ("snu", "dense", "stages"), ("snu", "tree", "resident"), ("snu", "sparse", "resident"), ("snu", "sparse", "stages")):  # fmt: skip
            if loop == "stages":
                os.environ["IMHIP_NEWTON"] = "stages"
            else:
                os.environ.pop("IMHIP_NEWTON", None)
            nsets = 8
            cases = [newton_case(name, stage, seed=21 + k) for k in range(nsets)]
            m0, d0, _, _ = cases[0]
            nworld, nv, njmax, nM = d0.nworld, m0.nv, d0.njmax, int(d0.M.shape[1])
            NF.solve(*cases[0])
            torch.cuda.synchronize()
            its = cases[0][1].solver_niter.cpu().numpy()
            unfinished = int((cases[0][2].done.cpu().numpy() == 0).sum())

            def start(k):  # what precedes the loop: the start point, init_context, the counters
                m_, d_, c_, n_ = cases[k]
                d_.qacc.copy_(d_.qacc_smooth)
                d_.qfrc_constraint.zero_()
                NF.init_context(m_, d_, c_)
                c_.search_unchanged.zero_()
                n_.fill_(nworld)

            sec_all = _timeit(torch, lambda k: NF.solve(*cases[k]), nsets, max(launches // 4, 4), prime=False)
            sec_init = _timeit(torch, start, nsets, max(launches // 4, 4), prime=False)
            rounds = int(its.max())  # dependent iterations the slowest world takes: the length of the loop
            issued = rounds if loop == "resident" else int(m0.opt.iterations)
            loop_s = sec_all - sec_init
            out = {"kernel": f"newton_fusion.solve, {stage} stage, iterations as {'one resident kernel' if loop == 'resident' else 'eight launches each'}",
                   "workload": f"{name} nv={nv} nefc={njmax} x {nworld} worlds, tolerance 1e-7, at most {m0.opt.iterations} iterations",
                   "us_per_solve": round(sec_all * 1e6, 1), "us_init_context": round(sec_init * 1e6, 1), "us_loop": round(loop_s * 1e6, 1),
                   "iterations_mean": round(float(its.mean()), 2), "iterations_max": rounds, "iterations_issued": issued,
                   "us_per_issued_iteration": round(loop_s * 1e6 / max(issued, 1), 2), "worlds_unfinished": unfinished,
                   "world_iterations_per_s": round(float(its.sum()) / loop_s)}  # fmt: skip
            # one pass over M, J, D and the per-row and per-dof vectors per iteration a world takes
            per_it = 4 * (njmax * nv + nM + 6 * njmax + 10 * nv)
            out.update(bound="hbm", algorithmic_bytes=int(per_it * its.sum()), achieved_GBs=round(per_it * float(its.sum()) / loop_s / 1e9, 1),
                       frac=round(per_it * float(its.sum()) / loop_s / 1e9 / HBM_GBS, 4))  # fmt: skip
            print(json.dumps(out), flush=True)
            del cases
        os.environ.pop("IMHIP_NEWTON", None)

    # ---- implicit-fast integrator matrix and its solve; the upstream-iteration sparse factor from the dense Hessian
    if section("implicit"):
        from .mjw_kernels import implicit_qh as IQ

        nworld = 4096
        m, d, st, _ = synth.make_implicit_case(nworld)
        dd = SimpleNamespace(nworld=nworld, M=t(d.M), moment_rownnz=d.moment_rownnz, moment_rowadr=d.moment_rowadr, moment_colind=d.moment_colind,
                             actuator_moment=t(d.actuator_moment), ten_J=t(d.ten_J), ctrl=t(d.ctrl), actuator_force=t(d.actuator_force),
                             efc=SimpleNamespace(Ma=t(d.efc.Ma)))  # fmt: skip
        scratch = IQ.create_implicit_qh_scratch(m, dd, dev)
        nM, nmom, nten, nu = int(st[2].size), int(d.moment_colind.size), int(m.ten_J_colind.size), int(m.nactuator)
        wl = f"snu + a free body nv={m.nv} nM={nM}, {nu} actuators ({nmom} moment entries), {m.ntendon} tendons ({nten} entries) x {nworld} worlds"
        sec = _timeit(torch, lambda i: IQ.deriv_smooth_vel(m, dd, scratch.implicit_qderiv, scratch), 1, launches)
        _line("im_implicit_qh: qH = M - h dF/dv in one launch (damping, actuator gains and pair sums, tendon pair sums)", wl, sec,
              bytes_=nworld * 4 * (2 * nM + nmom + nten + 3 * nu), nworld=nworld)  # fmt: skip
        sec = _timeit(torch, lambda i: IQ.deriv_smooth_vel(m, dd, scratch.implicit_qderiv, scratch, fused=False), 1, launches)
        _line("the same as separate launches: im_implicit_qh_base, im_actuator_velocity_gain, two entry permutations, two gathers", wl, sec,
              bytes_=nworld * 4 * (2 * nM + nmom + nten + 3 * nu), nworld=nworld)  # fmt: skip
        scratch.tree_factor_solve = T.create_tree_factor_solve_scratch(m, dev)
        sec = _timeit(torch, lambda i: IQ.implicit_factor_optimized(m, dd, scratch), 1, launches)
        _line("implicit_factor_optimized: qH and the tree L'DL solve on it", wl, sec,
              bytes_=nworld * 4 * (2 * nM + nmom + nten + 3 * nu + nM + 2 * m.nv), nworld=nworld)  # fmt: skip
        del dd, scratch
        torch.cuda.empty_cache()
        # non-fused sparse factor on a model the fused loop does not take (84 dofs), H = M + J'DJ from the dense assembly
        parents = tuple(synth.limbs_parents(6, 13))
        model = synth.model_from_parents(parents)
        b = synth.make_batch(synth.Shape("limbs84", parents, 48, nworld, (0.5, 8.0), 0.02, (-3.0, 3.0), 0.6, 2, 11), nworld)
        nv = model.nv
        plan, reason = SH.plan_for_model(model, SimpleNamespace(hfactor=np.zeros((1, model.nv_pad, model.nv_pad), np.float32)), [], 64, device=dev)
        if plan is not None and plan.path == "nonfused":
            Md = t(synth.dense_from_csr(b.M, b.rowadr, b.rownnz, b.colind).astype(np.float32).reshape(nworld, -1))
            H = torch.zeros((nworld, model.nv_pad, model.nv_pad), device=dev)
            BD.dense_hessian(Md, t(b.J), t(b.D), t(b.state[0]), t(b.nefc), H)
            hf = torch.zeros_like(H)
            g3, s3 = t(b.grad).reshape(nworld, nv, 1), torch.zeros((nworld, nv, 1), device=dev)
            sd, de = torch.zeros(nworld, device=dev), torch.zeros(nworld, device=dev)
            refactor = SH.nonfused_kernel(plan, False, False)
            sec = _timeit(torch, lambda i: refactor(None, g3, H, None, None, hf, s3, sd, de), 1, launches)
            used = plan.nfac + nv
            _line("im_sparse_dense_factor (refactor from the dense H)", f"limbs84 nv={nv} nfac={plan.nfac} x {nworld} worlds", sec,
                  bytes_=nworld * 4 * (2 * used + 2 * nv + 2), nworld=nworld)  # fmt: skip
            zero = torch.zeros(nworld, dtype=torch.int32, device=dev)
            one = torch.ones(nworld, dtype=torch.int32, device=dev)
            solve_only = SH.nonfused_kernel(plan, True, True)
            sec = _timeit(torch, lambda i: solve_only(None, g3, H, zero, one, hf, s3, sd, de), 1, launches)
            _line("im_sparse_dense_factor (solve with the stored factor)", f"limbs84 nv={nv} nfac={plan.nfac} x {nworld} worlds", sec,
                  bytes_=nworld * 4 * (used + 2 * nv + 2), nworld=nworld)  # fmt: skip

    # ---- body-tree accumulations and the wrench projection
    if section("bodies"):
        rig = synth.make_muscle_rig()
        topo = rig.topology
        nworld = 4096
        nb, nvf = rig.body_count, rig.full_torque_dim
        parent = np.asarray(topo.body_parentid, np.int32)
        order, offsets, _, _ = WP.tree_levels(parent)
        model = SimpleNamespace(body_parentid=parent, body_tree=[order[offsets[i] : offsets[i + 1]] for i in range(len(offsets) - 1)])
        scratch = TF.create_tree_reduction_scratch(model, deterministic=True, device=dev)
        for comp, skip, what in ((3, False, "subtree_com"), (10, True, "crb")):
            vals = [torch.randn((nworld, nb, comp), device=dev) for _ in range(8)]
            sec = _timeit(torch, lambda i: TF.accumulate(model, None, vals[i], comp, skip, scratch), 8, launches)
            _line(f"im_tree_accumulate ({what}: {comp} components)", f"snu rig body tree: {nb} bodies, {len(offsets) - 1} levels x {nworld} worlds", sec,
                  bytes_=nworld * 4 * 2 * nb * comp, nworld=nworld)  # fmt: skip
        wt = WP.build_wrench_projection_topology(t(parent), t(np.asarray(topo.dof_bodyid, np.int32)), nb, dev)
        rootid = t(np.asarray(topo.body_rootid, np.int32))
        ins = [[torch.randn((nworld, nb, 3), device=dev) for _ in range(4)] + [torch.randn((nworld, nvf, 6), device=dev)] for _ in range(8)]
        mean = torch.zeros((nworld, rig.torque_dim), device=dev)
        root = nvf - rig.torque_dim
        sec = _timeit(
            torch,
            lambda i: WP.launch_project_body_wrench_to_torque(
                wt, body_force=ins[i][0], body_torque=ins[i][1], xipos=ins[i][2], subtree_com=ins[i][3], cdof=ins[i][4],
                body_rootid=rootid, mean=mean, body_count=nb, torque_dim=rig.torque_dim, root_dof_count=root,
                output_dof_offset=0, batch_size=nworld,
            ),
            8, launches,
        )  # fmt: skip
        _line("im_project_body_wrenches", f"snu rig: {nb} bodies, {rig.torque_dim} torque dofs x {nworld} worlds", sec,
              bytes_=nworld * 4 * (12 * nb + 6 * nvf + rig.torque_dim), nworld=nworld)  # fmt: skip


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--launches", type=int, default=32)
    ap.add_argument("--only", default=None, help="comma-separated sections: trees, generated, stress, muscles, walks, iteration, solve, implicit, bodies")
    ap.add_argument("--no-graph", action="store_true", help="plain launches instead of a hipGraph replay")
    args = ap.parse_args()
    GRAPH = not args.no_graph
    run(args.launches, args.only)
