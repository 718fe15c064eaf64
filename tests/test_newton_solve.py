"""The constraint solve as the reference's step calls it: ``init_context``, the fused Newton loop
and the force recovery (src/instantmimic/utils/mjw_step_optimized.py:2588-2683,
src/instantmimic/utils/mjw_kernels/newton_fusion.py:330-539), started from poisoned solver state,
captured in a graph without any read-back, against the oracle's pieces chained in the same order."""

import numpy as np
import pytest

import newton_chain as NC
from instantmimic_amd import synth
from instantmimic_amd.mjw_kernels import newton_fusion as NF
from oracle import ref as R


# ---------------------------------------------------------------- oracle pinning (CPU)


def test_oracle_search_sums_and_init_jaref():
    rng = np.random.default_rng(2)
    for nv, block in ((27, 32), (56, 64), (70, 32), (14, 64)):
        g, s = rng.normal(size=(9, nv)).astype(np.float32), rng.normal(size=(9, nv)).astype(np.float32)
        skip = np.zeros(9, np.uint8)
        skip[4] = 1
        sd, de = R.newton_search_sums(g, s, block=block, skip=skip, sdot=np.full(9, 5.0, np.float32), decr=np.full(9, 6.0, np.float32))
        assert sd[4] == 5.0 and de[4] == 6.0
        live = skip == 0
        np.testing.assert_allclose(sd[live], (s.astype(np.float64) ** 2).sum(1)[live], rtol=1e-6)
        np.testing.assert_allclose(de[live], -(g.astype(np.float64) * s).sum(1)[live], rtol=1e-5, atol=1e-5)
    # one dof per lane: the sum is the 32-lane shuffle-down tree over the squares, folds in order
    v = rng.normal(size=(1, 32)).astype(np.float32)
    sq = (v[0] * v[0]).astype(np.float32)  # fma(v, v, 0) = the rounded square
    for off in (16, 8, 4, 2, 1):
        sq = (sq[:off] + sq[off : 2 * off]).astype(np.float32)
    assert R.newton_search_sums(np.zeros_like(v), v, block=32)[0][0] == np.float32(0.0) + sq[0]
    # Jaref = J qacc - aref
    J, q, a = rng.normal(size=(5, 12, 27)).astype(np.float32), rng.normal(size=(5, 27)).astype(np.float32), rng.normal(size=(5, 12)).astype(np.float32)
    nefc = np.array([12, 0, 5, 12, 1], np.int32)
    out = R.newton_init_jaref(J, q, a, nefc=nefc)
    want = np.einsum("wrj,wj->wr", J.astype(np.float64), q) - a
    rows = np.arange(12)[None, :] < nefc[:, None]
    np.testing.assert_allclose(out[rows], want[rows], rtol=1e-5, atol=1e-5)
    assert not out[~rows].any()


def test_oracle_dense_first_factor_is_the_factor_of_h():
    """A negative count of changed rows: H as it lies there is factored with the gradient as the
    augmented column, and U'U gives it back (beyond 32 dofs: below, no factor is kept)."""
    shape = synth.SHAPES["g1"]
    b = synth.make_batch(shape, 6, ragged_nefc=True)
    nv, pad = shape.nv, 48
    Md = synth.dense_from_csr(b.M, b.rowadr, b.rownnz, b.colind).astype(np.float32)
    H = R.jtdj_dense(Md.reshape(6, -1), b.J, b.D, b.state[0], b.nefc, pad)
    every = np.ones(6, np.int32)
    ids = np.zeros((6, shape.nefc), np.int32)
    H2, U, uni, search, sdot, decr = R.dense_update_factor(every, -every, ids, b.J, b.D, b.state[0], b.grad, H, np.zeros_like(H))
    np.testing.assert_array_equal(H2, H)
    assert not uni[:, nv].any()
    Hd = H[:, :nv, :nv].astype(np.float64)
    Hd = np.triu(Hd) + np.triu(Hd, 1).transpose(0, 2, 1)
    x64 = R.solve64(Hd, b.grad)
    err = np.linalg.norm(-search - x64, axis=1) / np.linalg.norm(x64, axis=1)
    assert (err / (np.linalg.cond(Hd) * 6e-8)).max() < 4.0
    Uf = np.triu(U[:, :nv, :nv].astype(np.float64))
    back = np.einsum("wki,wkj->wij", Uf, Uf)
    assert np.abs(back - Hd).max() / np.abs(Hd).max() < 2e-6
    np.testing.assert_allclose(decr, (b.grad * x64).sum(1), rtol=5e-3)


def test_elemid_table_matches_the_csr():
    rowadr, rownnz, colind = synth.csr_from_parents(synth.humanoid_parents())
    table = NF.elemid_table(rowadr, rownnz, colind)
    np.testing.assert_array_equal(table, synth.matrix_elemid(rowadr, rownnz, colind))
    assert (table == table.T).all() and (np.diag(table) == rowadr + rownnz - 1).all()


@pytest.mark.parametrize("stage", ["dense", "tree", "sparse"])
def test_oracle_solve_converges_to_the_fp64_minimum(stage):
    """The chained oracle from init_context on: every world finishes, no overflow, and at the end
    the gradient of the fp64 cost vanishes against the problem's scale -- on all three factor
    stages, with worlds that have no constraint rows and with a warm start."""
    name = "g1" if stage == "sparse" else "humanoid"
    p = NC.problem(name, 24, stage, empty_every=7, warmstart=(stage == "tree"))
    s = NC.oracle_solve(p)
    assert s.done.all() and not (s.overflow & 8).any() and s.niter.max() < 25
    assert (s.niter[p.nefc == 0] == 0).all() and (s.niter[p.nefc > 0] > 0).all()
    np.testing.assert_array_equal(s.qacc[p.nefc == 0], p.qacc_smooth[p.nefc == 0])
    b = p.b
    M64 = synth.dense_from_csr(b.M.astype(np.float64), b.rowadr, b.rownnz, b.colind)
    x = np.einsum("wrj,wj->wr", p.J.astype(np.float64), s.qacc.astype(np.float64)) - p.aref
    g = np.einsum("wij,wj->wi", M64, s.qacc.astype(np.float64) - p.qacc_smooth)
    for w in range(p.nworld):
        ne, nf, nefc = int(p.ne[w]), int(p.nf[w]), int(p.nefc[w])
        D, fl = p.D[w].astype(np.float64), p.frictionloss[w].astype(np.float64)
        slope = np.zeros(p.njmax)
        slope[:ne] = D[:ne] * x[w, :ne]
        fr = slice(ne, ne + nf)
        slope[fr] = np.clip(D[fr] * x[w, fr], -fl[fr], fl[fr])
        rest = slice(ne + nf, nefc)
        slope[rest] = D[rest] * np.minimum(x[w, rest], 0.0)
        g[w] += slope[:nefc] @ p.J[w, :nefc].astype(np.float64)
        # the recovered constraint force is minus that slope pulled back: J' force = -J' slope
        np.testing.assert_allclose(s.qfrc_constraint[w], -(slope[:nefc] @ p.J[w, :nefc].astype(np.float64)), rtol=2e-3, atol=2e-3 * max(1.0, np.abs(s.qfrc_constraint[w]).max()))
    g0 = np.linalg.norm(np.einsum("wrj,wr->wj", p.J.astype(np.float64), p.D * np.abs(p.aref)), axis=1)
    has = p.nefc > 0
    assert (np.linalg.norm(g, axis=1)[has] / g0[has]).max() < 1e-4


# ---------------------------------------------------------------- GPU


def _solve_on_gpu(p, device, *, graph: bool):
    import torch

    m, d, ctx, nsolving = NC.device_objects(p, device)
    if graph:
        # the whole solve as one graph of the caller's: nothing in it may touch the host
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            NF.solve(m, d, ctx, nsolving)  # first use outside the capture (lazy initialisations)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        m, d, ctx, nsolving = NC.device_objects(p, device)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            NF.solve(m, d, ctx, nsolving)
        g.replay()
    else:
        NF.solve(m, d, ctx, nsolving)
    torch.cuda.synchronize()
    return m, d, ctx, nsolving


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld,stage,graph,loop", [
    ("humanoid", 300, "dense", False, "stages"), ("humanoid", 300, "tree", False, "stages"), ("g1", 200, "sparse", False, "stages"),
    ("humanoid", 4096, "tree", True, "stages"), ("humanoid", 4096, "dense", True, "stages"), ("g1", 8192, "sparse", True, "stages"),
    ("snu", 4096, "sparse", True, "stages"), ("ant", 64, "tree", True, "stages"), ("snu", 130, "tree", False, "stages"),
    ("humanoid", 301, "tree", False, "resident"), ("humanoid", 4096, "tree", True, "resident"), ("ant", 67, "tree", True, "resident"),
    ("g1", 203, "sparse", False, "resident"), ("g1", 8192, "sparse", True, "resident"), ("snu", 4096, "sparse", True, "resident"),
    ("g1", 8192, "tree", True, "resident"), ("snu", 131, "tree", False, "resident"), ("snu", 4096, "tree", True, "resident"),
    ("humanoid", 303, "dense", False, "resident"), ("humanoid", 4096, "dense", True, "resident"), ("ant", 69, "dense", True, "resident"),
    ("g1", 205, "dense", False, "resident"), ("g1", 8192, "dense", True, "resident"), ("g1", 207, "dense", False, "stages"),
    ("snu", 133, "dense", False, "resident"), ("snu", 4096, "dense", True, "resident"), ("snu", 135, "dense", False, "stages"),
])  # fmt: skip
def test_gpu_solve_from_init_context_matches_the_oracle_chain(device, monkeypatch, name, nworld, stage, graph, loop):
    """``loop``: the iterations as eight launches each (``stages``) or as one resident kernel with a
    wavefront per world (``resident``: the tree stage with generated kernels, the sparse stage, the
    dense single-tile stage up to 32 dofs, the dense blocked stage for a padded size of 48 or 64): the same
    arrays at the end either way."""
    small = nworld <= 301
    p = NC.problem(name, nworld, stage, empty_every=11 if small else 97, warmstart=small, maxiter=12)
    s = NC.oracle_solve(p)
    taken = []
    inner = NF.run_resident
    monkeypatch.setattr(NF, "run_resident", lambda *a: taken.append(inner(*a)) or taken[-1])
    if loop == "stages":
        monkeypatch.setenv("IMHIP_NEWTON", "stages")
    m, d, ctx, nsolving = _solve_on_gpu(p, device, graph=graph)
    assert all(taken) == (loop == "resident") and len(taken) > 0
    NC.compare(p, s, d, ctx)
    assert int(nsolving.item()) == int((p.nefc == 0).sum())  # every world that had rows has reported done


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld,stage", [("humanoid", 301, "tree"), ("g1", 203, "sparse"), ("snu", 131, "tree"), ("ant", 67, "dense"),
                                               ("humanoid", 299, "dense"), ("g1", 201, "dense"), ("snu", 129, "dense")])  # fmt: skip
def test_gpu_init_context_in_one_launch_leaves_what_the_five_launches_leave(device, monkeypatch, name, nworld, stage):
    """Everything before the first Hessian as one launch (a wavefront per world) against the same
    steps as launches of their own: every array of ``d``, ``d.efc`` and ``ctx`` bit for bit, poison
    included where neither writes.  On the dense stage the first Hessian and its factor are one
    launch as well (``im_dense_init_factor``: a single tile up to 32 dofs, 48 or 64 columns beyond)
    against dense M, ``J' D J`` and the stage as three; the dense copy of M is scratch of the three."""
    import torch

    p = NC.problem(name, nworld, stage, empty_every=7, warmstart=True, maxiter=12)
    taken = []
    inner = NF._init_before_factor
    monkeypatch.setattr(NF, "_init_before_factor", lambda *a: taken.append(inner(*a)) or taken[-1])
    got = []
    for env in ("stages", None):
        if env:
            monkeypatch.setenv("IMHIP_NEWTON", env)
        else:
            monkeypatch.delenv("IMHIP_NEWTON")
        m, d, ctx, _ = NC.device_objects(p, device)
        d.qacc.copy_(d.qacc_warmstart)
        NF.init_context(m, d, ctx)
        torch.cuda.synchronize()
        got.append({f"{where}.{k}": v.cpu().numpy() for where, ns in (("d", d), ("efc", d.efc), ("ctx", ctx))
                    for k, v in vars(ns).items() if isinstance(v, torch.Tensor)})  # fmt: skip
    assert taken == [False, True]
    assert got[0].keys() == got[1].keys() and "ctx.grad" in got[0] and "efc.Ma" in got[0]
    for key in got[0]:
        if key == "ctx.newton_mdense":
            continue
        a, b = got[0][key], got[1][key]
        assert a.tobytes() == b.tobytes(), key
    if stage == "dense":
        assert "ctx.h" in got[0] and "ctx.hfactor" in got[0] and np.nanmax(np.abs(got[1]["ctx.h"])) > 0


def _floating_chain(nv: int, limbs: int = 1):
    """A free body and hinges behind it (the reference's layout-boundary models,
    tests/test_mjw_newton_fusion.py:100-131): ``nv`` dofs, one chain or ``limbs`` chains off the
    free body's last dof."""
    parents = [-1, 0, 1, 2, 3, 4]
    tips = [5] * limbs
    for k in range(6, nv):
        parents.append(tips[k % limbs])
        tips[k % limbs] = k
    return tuple(parents[:nv])


# (dofs, stage, chains): one chain on the dense stage; chains off the free body on the tree stage (a single
# chain's M is dense: the tree factor declines it)
_BOUNDARY = [(13, "dense", 1), (16, "dense", 1), (17, "dense", 1), (29, "dense", 1), (31, "dense", 1), (32, "dense", 1),
             (33, "dense", 1), (35, "dense", 1), (48, "dense", 1), (49, "dense", 1), (56, "dense", 1), (60, "dense", 1),
             (61, "dense", 1), (62, "dense", 1), (63, "dense", 1), (64, "dense", 1), (70, "dense", 1), (79, "dense", 1),
             (17, "tree", 3), (33, "tree", 3), (49, "tree", 3), (40, "tree", 2), (45, "tree", 3), (68, "tree", 4), (72, "tree", 4)]  # fmt: skip
# (79 dofs in four or five chains behind a free body have more than the 1024 elements of M that the tree kernels take:
# such a model gets no tree scratch and solves on the dense stage)


@pytest.mark.gpu
@pytest.mark.parametrize("maxiter,ls_iterations,warmstart", [(12, 50, False), (4, 4, True)])
@pytest.mark.parametrize("nv,stage,chains", _BOUNDARY)
def test_gpu_solve_at_layout_boundaries(device, monkeypatch, nv, stage, chains, maxiter, ls_iterations, warmstart):
    """Dof counts on both sides of the padded layouts' boundaries (16, 32, 48, 64, 80: the single tile up
    to 32 dofs, the blocked factor beyond, as stage launches from 64 dofs on; kernels generated on the
    spot on the tree stage, also where the rows touch few dofs: two to four chains), with a budget
    that lets every world converge and with one of four iterations and four line-search rounds from a
    warm start, as the reference checks its captured solve there (tests/test_mjw_newton_fusion.py
    :257-288)."""
    name = f"chain{nv}x{chains}"
    parents = _floating_chain(nv, chains)
    monkeypatch.setitem(synth.SHAPES, name, synth.Shape(name, parents, 40, 64, (0.5, 8.0), 0.02, (-4.0, 4.0), 0.6, 1, 1100 + nv))
    p = NC.problem(name, 37, stage, empty_every=9, maxiter=maxiter, ls_iterations=ls_iterations, warmstart=warmstart)
    s = NC.oracle_solve(p)
    assert s.done.all()
    m, d, ctx, nsolving = _solve_on_gpu(p, device, graph=True)
    NC.compare(p, s, d, ctx)
