"""The steps either side of the solve that walk a world's small trees: M v over the tree
CSR, bottom-up accumulation of per-body values, body wrenches onto joint torques.  Oracle
pinning and host tables on the CPU, bit-for-bit parity of the HIP kernels on the GPU."""

import numpy as np
import pytest

from instantmimic_amd import synth
from instantmimic_amd.mjw_kernels import newton_fusion as NF
from instantmimic_amd.mjw_kernels import tree_fusion as TF
from instantmimic_amd.muscle import wrench_projection as WP
from instantmimic_amd.muscle.muscle_dynamics import build_dof_subtree_mask
from oracle import ref as R

TREES = {"ant": synth.ant_parents, "humanoid": synth.humanoid_parents, "snu": synth.snu_parents, "stress": synth.stress_parents}


def _body_tree(nbody: int, seed: int):
    """A random body tree with body 0 the world: parents reference earlier bodies."""
    rng = np.random.default_rng(seed)
    parent = np.zeros(nbody, np.int32)
    for b in range(1, nbody):
        parent[b] = rng.integers(max(0, b - 4), b)
    return parent


def _levels(parent):
    order, offsets, _, _ = WP.tree_levels(parent)
    return order, offsets


def _ancestor_or_self(parent):
    n = len(parent)
    anc = np.zeros((n, n), bool)  # anc[b, a]: a is b or an ancestor of b
    for b in range(n):
        p = b
        while True:
            anc[b, p] = True
            if p == 0:
                break
            p = int(parent[p])
    return anc


# ---------------------------------------------------------------- M v
@pytest.mark.parametrize("tree", list(TREES))
def test_mul_m_tables_and_oracle_against_dense_fp64(tree):
    rowadr, rownnz, colind = synth.csr_from_parents(TREES[tree]())
    nv, nM = len(rowadr), len(colind)
    adr, col, madr = NF.mul_m_tables(rowadr, rownnz, colind)
    # every element of the symmetric matrix exactly once, at its CSR address
    elem = synth.matrix_elemid(rowadr, rownnz, colind)
    assert adr[0] == 0 and adr[-1] == 2 * nM - nv
    for i in range(nv):
        cols = col[adr[i] : adr[i + 1]]
        assert len(set(cols.tolist())) == len(cols)
        assert sorted(cols.tolist()) == np.nonzero(elem[i] >= 0)[0].tolist()
        np.testing.assert_array_equal(madr[adr[i] : adr[i + 1]], elem[i, cols])
    rng = np.random.default_rng(5)
    M = rng.normal(size=(9, nM)).astype(np.float32)
    v = rng.normal(size=(9, nv)).astype(np.float32)
    out = R.mul_m_sparse(M, v, adr, col, madr)
    dense = synth.dense_from_csr(M.astype(np.float64), rowadr, rownnz, colind)
    want = np.einsum("wij,wj->wi", dense, v.astype(np.float64))
    assert R.rel_l2(out, want) < 1e-6
    # scaling by a power of two is exact; skipped worlds keep their rows
    np.testing.assert_array_equal(R.mul_m_sparse(M, 4 * v, adr, col, madr), 4 * out)
    skip = np.zeros(9, np.uint8)
    skip[[2, 7]] = 1
    kept = R.mul_m_sparse(M, v, adr, col, madr, skip=skip, out=np.full((9, nv), 7.0, np.float32))
    assert (kept[[2, 7]] == 7.0).all()
    np.testing.assert_array_equal(np.delete(kept, [2, 7], 0), np.delete(out, [2, 7], 0))


# ---------------------------------------------------------------- accumulation
@pytest.mark.parametrize("nbody,components,skip", [(1, 3, False), (2, 3, False), (17, 3, False), (17, 10, True), (60, 6, False), (300, 10, True)])
def test_oracle_accumulate_against_subtree_sums(nbody, components, skip):
    parent = _body_tree(nbody, seed=nbody)
    order, offsets = _levels(parent)
    rng = np.random.default_rng(11)
    vals = rng.normal(size=(5, nbody, components)).astype(np.float32)
    got = R.tree_accumulate(vals, components, parent, order, offsets, skip)
    anc = _ancestor_or_self(parent)
    want = np.einsum("ba,wbc->wac", anc.astype(np.float64), vals.astype(np.float64))
    # body 0 is never a child; with skip the children of body 0 are not added to it
    want[:, 0] = vals[:, 0] if skip else vals[:, 0] + want[:, 1:][:, parent[1:] == 0].sum(1)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 1e-6 * scale * max(1, np.log2(nbody))
    # integers: every order of additions gives the same bits
    ints = rng.integers(-8, 9, size=(3, nbody, components)).astype(np.float32)
    wi = np.einsum("ba,wbc->wac", anc.astype(np.float64), ints.astype(np.float64))
    wi[:, 0] = ints[:, 0] if skip else ints[:, 0] + wi[:, 1:][:, parent[1:] == 0].sum(1)
    np.testing.assert_array_equal(R.tree_accumulate(ints, components, parent, order, offsets, skip), wi.astype(np.float32))


def test_accumulate_scratch_mirrors_the_reference_fields():
    class M:
        body_tree = [np.array([0]), np.array([1, 4]), np.array([2, 3, 5])]
        body_parentid = np.array([0, 0, 1, 1, 0, 4])

    class Empty:
        body_tree = []
        body_parentid = np.zeros(1, np.int32)

    assert TF.create_tree_reduction_scratch(Empty(), device="cpu") is None
    s = TF.create_tree_reduction_scratch(M(), deterministic=True, device="cpu")
    assert s.levels == 3 and s.deterministic and s.cooperative and s.nbody == 6
    assert s.bodies.tolist() == [0, 1, 4, 2, 3, 5] and s.offsets.tolist() == [0, 1, 3, 6]
    order, offsets, child_bodies, child_offsets = WP.tree_levels(M.body_parentid)
    assert order.tolist() == s.bodies.tolist() and offsets.tolist() == s.offsets.tolist()
    assert child_bodies.tolist() == [1, 4, 2, 3, 5] and child_offsets.tolist() == [0, 2, 4, 4, 4, 5, 5]
    with pytest.raises(ValueError):
        WP.tree_levels(np.array([0, 2, 1]))


# ---------------------------------------------------------------- wrench projection
def _wrench_case(nworld, seed=1003):
    rig = synth.make_muscle_rig(nmuscle=40, seed=seed)
    topo = rig.topology
    nb, nv = rig.body_count, rig.full_torque_dim
    ctx = synth.make_muscle_context(rig, nworld, seed=seed + 1)
    xipos = ctx[:, 7 * nb : 10 * nb].reshape(nworld, nb, 3)
    com = ctx[:, 10 * nb : 13 * nb].reshape(nworld, nb, 3)
    cdof = ctx[:, 13 * nb : 13 * nb + 6 * nv].reshape(nworld, nv, 6)
    rng = np.random.default_rng(seed + 2)
    force = rng.normal(0, 50, (nworld, nb, 3)).astype(np.float32)
    torque = rng.normal(0, 5, (nworld, nb, 3)).astype(np.float32)
    return rig, topo, force, torque, np.ascontiguousarray(xipos), np.ascontiguousarray(com), np.ascontiguousarray(cdof)


def test_oracle_wrench_projection_against_the_masked_sum_fp64():
    nworld = 6
    rig, topo, force, torque, xipos, com, cdof = _wrench_case(nworld)
    nb, root, nt = rig.body_count, rig.full_torque_dim - rig.torque_dim, rig.torque_dim
    parent, rootid, dof_body = (np.asarray(a, np.int32) for a in (topo.body_parentid, topo.body_rootid, topo.dof_bodyid))
    order, offsets = _levels(parent)
    got = R.project_body_wrenches(force, torque, xipos, com, cdof, rootid, dof_body, parent, order, offsets, root, nt, out_offset=2,
                                  mean=np.full((nworld, nt + 5), 7.0, np.float32))  # fmt: skip
    assert (got[:, :2] == 7.0).all() and (got[:, nt + 2 :] == 7.0).all()
    # the per-dof kernel of the reference: total += mask * (lin . f + ang . (t + (x - c_root) x f))
    mask = build_dof_subtree_mask(parent, dof_body, nb, rig.full_torque_dim).astype(np.float64)
    f64, t64 = force.astype(np.float64), torque.astype(np.float64)
    arm = xipos.astype(np.float64) - com.astype(np.float64)[:, rootid]
    moment = t64 + np.cross(arm, f64)
    per_body = np.einsum("wdk,wbk->wdb", cdof[:, :, 3:].astype(np.float64), f64) + np.einsum(
        "wdk,wbk->wdb", cdof[:, :, :3].astype(np.float64), moment
    )
    want = np.einsum("db,wdb->wd", mask, per_body)[:, root : root + nt]
    assert R.rel_l2(got[:, 2 : nt + 2], want) < 1e-6


# ---------------------------------------------------------------- GPU
@pytest.mark.gpu
@pytest.mark.parametrize("tree,nworld", [("ant", 64), ("humanoid", 4096), ("snu", 333), ("stress", 67)])
def test_gpu_mul_m_bitwise(device, tree, nworld):
    import torch

    rowadr, rownnz, colind = synth.csr_from_parents(TREES[tree]())
    nv, nM = len(rowadr), len(colind)
    tables = NF.mul_m_tables(rowadr, rownnz, colind)
    rng = np.random.default_rng(7)
    M = rng.normal(size=(nworld, nM)).astype(np.float32)
    v = rng.normal(size=(nworld, nv)).astype(np.float32)
    skip = (rng.uniform(size=nworld) < 0.2).astype(np.uint8)
    t = lambda a: torch.from_numpy(a).to(device)  # noqa: E731
    td = [t(a) for a in tables]
    Md = torch.zeros((nworld, nM + 3), device=device)
    Md[:, :nM] = t(M)
    out = torch.full((nworld, nv + 2), 7.0, device=device)
    NF.mul_m(Md[:, :nM], t(v), out[:, :nv], *td)
    torch.cuda.synchronize()
    want = R.mul_m_sparse(M, v, *tables)
    got = out.cpu().numpy()
    np.testing.assert_array_equal(got[:, :nv], want)
    assert (got[:, nv:] == 7.0).all()
    out.fill_(7.0)
    NF.mul_m(Md[:, :nM], t(v), out[:, :nv], *td, skip_world=t(skip))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert (got[skip == 1] == 7.0).all()
    np.testing.assert_array_equal(got[skip == 0][:, :nv], want[skip == 0])


@pytest.mark.gpu
@pytest.mark.parametrize("nbody,components,skip,nworld", [(2, 3, False, 5), (17, 3, False, 4096), (17, 10, True, 1000), (60, 6, False, 333), (300, 10, True, 65), (1200, 10, False, 9)])
def test_gpu_accumulate_bitwise(device, nbody, components, skip, nworld):
    import torch

    parent = _body_tree(nbody, seed=nbody)
    order, offsets = _levels(parent)

    class M:
        body_parentid = parent
        body_tree = [order[offsets[i] : offsets[i + 1]] for i in range(len(offsets) - 1)]

    scratch = TF.create_tree_reduction_scratch(M(), deterministic=True, device=device)
    vals = np.random.default_rng(3).normal(size=(nworld, nbody, components)).astype(np.float32)
    vd = torch.from_numpy(vals).to(device)
    TF.accumulate(M(), None, vd, components, skip, scratch)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(vd.cpu().numpy(), R.tree_accumulate(vals, components, parent, order, offsets, skip))


@pytest.mark.gpu
@pytest.mark.parametrize("nworld", [1, 67, 4096])
def test_gpu_wrench_projection_bitwise(device, nworld):
    import torch

    rig, topo, force, torque, xipos, com, cdof = _wrench_case(nworld)
    nb, root, nt = rig.body_count, rig.full_torque_dim - rig.torque_dim, rig.torque_dim
    parent, rootid, dof_body = (np.asarray(a, np.int32) for a in (topo.body_parentid, topo.body_rootid, topo.dof_bodyid))
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    topology = WP.build_wrench_projection_topology(t(parent), t(dof_body), nb, device)
    assert topology is not None and topology.levels == len(_levels(parent)[1]) - 1
    mean = torch.full((nworld, nt + 5), 7.0, device=device)
    WP.launch_project_body_wrench_to_torque(
        topology, body_force=t(force), body_torque=t(torque), xipos=t(xipos), subtree_com=t(com), cdof=t(cdof),
        body_rootid=t(rootid), dof_subtree_mask=None, mean=mean, body_count=nb, torque_dim=nt, root_dof_count=root,
        output_dof_offset=2, batch_size=nworld, device=str(device),
    )  # fmt: skip
    torch.cuda.synchronize()
    order, offsets = _levels(parent)
    want = R.project_body_wrenches(force, torque, xipos, com, cdof, rootid, dof_body, parent, order, offsets, root, nt, out_offset=2,
                                   mean=np.full((nworld, nt + 5), 7.0, np.float32))  # fmt: skip
    np.testing.assert_array_equal(mean.cpu().numpy(), want)


@pytest.mark.gpu
def test_gpu_tree_walks_replay_in_a_graph(device):
    """The three launchers captured in one graph: every replay, with eager work on the same
    buffers between the replays, gives the eager results bit for bit."""
    import torch

    nworld = 257
    rig, topo, force, torque, xipos, com, cdof = _wrench_case(nworld)
    nb, root, nt = rig.body_count, rig.full_torque_dim - rig.torque_dim, rig.torque_dim
    parent, rootid, dof_body = (np.asarray(a, np.int32) for a in (topo.body_parentid, topo.body_rootid, topo.dof_bodyid))
    order, offsets = _levels(parent)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    topology = WP.build_wrench_projection_topology(t(parent), t(dof_body), nb, device)
    model = type("M", (), dict(body_parentid=parent, body_tree=[order[offsets[i] : offsets[i + 1]] for i in range(len(offsets) - 1)]))
    scratch = TF.create_tree_reduction_scratch(model, deterministic=True, device=device)
    rowadr, rownnz, colind = synth.csr_from_parents(synth.snu_parents())
    tables = [t(a) for a in NF.mul_m_tables(rowadr, rownnz, colind)]
    rng = np.random.default_rng(4)
    M, v = t(rng.normal(size=(nworld, len(colind))).astype(np.float32)), t(rng.normal(size=(nworld, len(rowadr))).astype(np.float32))
    vals0 = t(rng.normal(size=(nworld, nb, 6)).astype(np.float32))
    ins = dict(body_force=t(force), body_torque=t(torque), xipos=t(xipos), subtree_com=t(com), cdof=t(cdof), body_rootid=t(rootid))
    vals, mean, mv = vals0.clone(), torch.zeros((nworld, nt), device=device), torch.zeros_like(v)

    def work():
        vals.copy_(vals0)
        TF.accumulate(model, None, vals, 6, False, scratch)
        WP.launch_project_body_wrench_to_torque(topology, **ins, mean=mean, body_count=nb, torque_dim=nt, root_dof_count=root,
                                                output_dof_offset=0, batch_size=nworld)  # fmt: skip
        NF.mul_m(M, v, mv, *tables)

    work()
    torch.cuda.synchronize()
    want = [a.clone() for a in (vals, mean, mv)]
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        work()
    torch.cuda.current_stream().wait_stream(s)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        work()
    for _ in range(3):
        for a in (vals, mean, mv):
            a.fill_(float("nan"))  # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for a, b in zip((vals, mean, mv), want):
            assert torch.equal(a, b)


# ---------------------------------------------------------------- Newton gradient
def _gradient_case(name, nworld, seed=9):
    b = synth.make_batch(name, nworld, ragged_nefc=True)
    rng = np.random.default_rng(seed)
    njmax, nv = b.J.shape[1], b.J.shape[2]
    force = rng.normal(0, 3, (nworld, njmax)).astype(np.float32)
    # satisfied constraints carry no force: the kernel does not read their rows of J
    idle = rng.uniform(size=force.shape)
    force[idle < 0.4] = 0.0
    force[idle < 0.05] = -0.0
    force[0] = 0.0  # a world without any force
    smooth = rng.normal(0, 1, (nworld, nv)).astype(np.float32)
    Ma = rng.normal(0, 1, (nworld, nv)).astype(np.float32)
    changed = rng.integers(0, 3, nworld).astype(np.int32)  # a third of the worlds keep their states
    done = (rng.uniform(size=nworld) < 0.15).astype(np.uint8)
    alpha = rng.uniform(0, 0.5, nworld).astype(np.float32)
    scalars = [rng.uniform(0.5, 2, nworld).astype(np.float32) for _ in range(3)]
    scalars[2][::11] = 0.0  # a zero scale: the ratio is defined as 0
    return b, force, smooth, Ma, changed, alpha, done, scalars


@pytest.mark.parametrize("name,block", [("ant", 32), ("humanoid", 64), ("snu", 32), ("stress", 64)])
def test_oracle_newton_gradient_against_fp64(name, block):
    nworld = 40
    b, force, smooth, Ma, changed, alpha, done, (gd0, de0, sc0) = _gradient_case(name, nworld)
    qc, grad, gd, de, sc, un = R.newton_gradient(b.J, force, smooth, Ma, changed, alpha, gd0, de0, sc0, nefc=b.nefc, done=done, block=block)
    np.testing.assert_array_equal(un, ((done != 0) | (changed == 0)).astype(np.uint8))
    work = (done == 0) & (changed != 0)
    rows = np.arange(b.J.shape[1])[None, :] < b.nefc[:, None]
    qc64 = np.einsum("wrd,wr->wd", b.J.astype(np.float64) * rows[:, :, None], force.astype(np.float64))
    g64 = Ma.astype(np.float64) - smooth - qc64
    assert R.rel_l2(qc[work], qc64[work]) < 1e-6 and R.rel_l2(grad[work], g64[work]) < 1e-6
    np.testing.assert_allclose(gd[work], (g64[work] ** 2).sum(1), rtol=1e-5)
    assert (de[work] == 0).all() and (sc[work] == 1).all()
    # untouched where done; rescaled where the states did not change
    d = done != 0
    assert (qc[~work] == 0).all() and (grad[~work] == 0).all()
    for got, was in ((gd, gd0), (de, de0), (sc, sc0)):
        np.testing.assert_array_equal(got[d], was[d])
    keep = (done == 0) & (changed == 0)
    new_sigma = sc0 - alpha
    ratio = np.where(sc0 != 0, new_sigma / np.where(sc0 != 0, sc0, 1), 0).astype(np.float32)
    np.testing.assert_array_equal(sc[keep], new_sigma[keep])
    np.testing.assert_array_equal(gd[keep], (gd0 * (ratio * ratio))[keep])
    np.testing.assert_array_equal(de[keep], (de0 * (ratio * ratio))[keep])


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld,block", [("ant", 64, 32), ("humanoid", 4096, 64), ("g1", 333, 32), ("snu", 130, 64), ("stress", 37, 64)])
def test_gpu_newton_gradient_bitwise(device, name, nworld, block):
    import torch

    b, force, smooth, Ma, changed, alpha, done, (gd0, de0, sc0) = _gradient_case(name, nworld)
    nv = b.J.shape[2]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    qc, grad = torch.full((nworld, nv), 7.0, device=device), torch.full((nworld, nv), 7.0, device=device)
    gd, de, sc = t(gd0), t(de0), t(sc0)
    un = torch.full((nworld,), 9, dtype=torch.uint8, device=device)
    NF.gradient(t(b.nefc), t(b.J), t(force), t(smooth), t(Ma), t(changed), t(alpha), t(done), qc, grad, gd, de, sc, un, block=block)
    torch.cuda.synchronize()
    want = R.newton_gradient(b.J, force, smooth, Ma, changed, alpha, gd0, de0, sc0, nefc=b.nefc, done=done, block=block)
    work = (done == 0) & (changed != 0)
    np.testing.assert_array_equal(qc.cpu().numpy()[work], want[0][work])
    np.testing.assert_array_equal(grad.cpu().numpy()[work], want[1][work])
    assert (qc.cpu().numpy()[~work] == 7.0).all() and (grad.cpu().numpy()[~work] == 7.0).all()
    for got, ref in zip((gd, de, sc, un), want[2:]):
        np.testing.assert_array_equal(got.cpu().numpy(), ref)
    # without the optional arrays: every row counts, no world is done
    NF.gradient(None, t(b.J), t(force), t(smooth), t(Ma), t(changed), t(alpha), None, qc, grad, t(gd0), t(de0), t(sc0), un, block=block)
    torch.cuda.synchronize()
    want = R.newton_gradient(b.J, force, smooth, Ma, changed, alpha, gd0, de0, sc0, block=block)
    np.testing.assert_array_equal(qc.cpu().numpy()[changed != 0], want[0][changed != 0])
    np.testing.assert_array_equal(un.cpu().numpy(), want[5])


# ---------------------------------------------------------------- J v of the line search
@pytest.mark.parametrize("name", ["ant", "humanoid", "snu", "stress"])
def test_oracle_newton_jv_against_fp64(name):
    nworld = 24
    b = synth.make_batch(name, nworld, ragged_nefc=True)
    rng = np.random.default_rng(2)
    search = rng.normal(size=(nworld, b.J.shape[2])).astype(np.float32)
    skip = np.zeros(nworld, np.uint8)
    skip[::5] = 1
    got = R.newton_jv(b.J, search, nefc=b.nefc, skip=skip, out=np.full(b.J.shape[:2], 7.0, np.float32))
    want = np.einsum("wrd,wd->wr", b.J.astype(np.float64), search.astype(np.float64))
    rows = np.arange(b.J.shape[1])[None, :] < b.nefc[:, None]
    live = rows & (skip == 0)[:, None]
    assert np.abs(got[live] - want[live]).max() <= 1e-5 * np.abs(want).max()
    assert (got[~live] == 7.0).all()
    # one chain up to 50 dofs: the same bits as a running fused multiply-add in numpy's float32
    if b.J.shape[2] <= 50:
        w, r = int(np.flatnonzero(skip == 0)[0]), 0
        acc = np.float32(0)
        for i in range(b.J.shape[2]):
            acc = np.float32(np.float64(b.J[w, r, i]) * np.float64(search[w, i]) + np.float64(acc))  # exact product, one rounding
        assert got[w, r] == acc


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld", [("ant", 64), ("humanoid", 4096), ("g1", 333), ("snu", 130), ("stress", 37)])
def test_gpu_newton_jv_bitwise(device, name, nworld):
    import torch

    b = synth.make_batch(name, nworld, ragged_nefc=True)
    njmax, nv = b.J.shape[1], b.J.shape[2]
    rng = np.random.default_rng(2)
    search = rng.normal(size=(nworld, nv)).astype(np.float32)
    skip = (rng.uniform(size=nworld) < 0.2).astype(np.uint8)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    out = torch.full((nworld, njmax), 7.0, device=device)
    NF.jv(t(b.J), t(search), out, nefc=t(b.nefc), skip_world=t(skip))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), R.newton_jv(b.J, search, nefc=b.nefc, skip=skip, out=np.full((nworld, njmax), 7.0, np.float32)))
    out.fill_(7.0)
    NF.jv(t(b.J), t(search), out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), R.newton_jv(b.J, search))


# ---------------------------------------------------------------- step and changed rows
def _step_case(name, nworld, seed=6):
    b = synth.make_batch(name, nworld, ragged_nefc=True)
    rng = np.random.default_rng(seed)
    njmax, nv = b.J.shape[1], b.J.shape[2]
    f = lambda *shape: rng.normal(size=shape).astype(np.float32)  # noqa: E731
    done = (rng.uniform(size=nworld) < 0.2).astype(np.uint8)
    old = rng.integers(0, 4, (nworld, njmax)).astype(np.int32)
    new = np.where(rng.uniform(size=old.shape) < 0.3, rng.integers(0, 4, old.shape), old).astype(np.int32)
    return b, (f(nworld), f(nworld, nv), f(nworld, nv), f(nworld, njmax), f(nworld, nv), f(nworld, nv), f(nworld, njmax)), done, old, new


def test_oracle_step_and_changed_rows():
    from test_newton_stages import _changes

    b, (alpha, search, mv, jv, qacc, Ma, jaref), done, old, new = _step_case("humanoid", 30)
    q, m, j = R.newton_advance(alpha, search, mv, jv, qacc, Ma, jaref, nefc=b.nefc, done=done)
    live = done == 0
    want = qacc.astype(np.float64) + alpha[:, None].astype(np.float64) * search
    assert np.abs(q[live] - want[live]).max() < 1e-6 * np.abs(want).max()
    np.testing.assert_array_equal(q[~live], qacc[~live])
    rows = np.arange(jv.shape[1])[None, :] < b.nefc[:, None]
    np.testing.assert_array_equal(j[~(rows & live[:, None])], jaref[~(rows & live[:, None])])
    assert np.abs(j - (jaref + alpha[:, None].astype(np.float64) * jv))[rows & live[:, None]].max() < 1e-6 * np.abs(jaref).max()
    # the listing against the row lists the factor-stage tests build on their own
    import dataclasses

    b3 = synth.make_batch(dataclasses.replace(synth.SHAPES["g1"], iterations=2), 40, ragged_nefc=True)
    new_s, ids, changes, _, _, _ = _changes(b3, np.random.default_rng(1))
    got_ids, qc, sc = R.newton_changed_rows(b3.state[0], new_s, quad=synth.QUADRATIC, nefc=b3.nefc)
    np.testing.assert_array_equal(qc, changes)
    for w in range(40):
        np.testing.assert_array_equal(got_ids[w, : qc[w]], ids[w, : changes[w]])
    assert (sc >= qc).all()


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld", [("ant", 64), ("humanoid", 4096), ("snu", 130), ("stress", 37)])
def test_gpu_step_and_changed_rows_bitwise(device, name, nworld):
    import torch

    b, arrays, done, old, new = _step_case(name, nworld)
    alpha, search, mv, jv, qacc, Ma, jaref = arrays
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    qd, md, jd = t(qacc), t(Ma), t(jaref)
    NF.advance(t(alpha), t(search), t(mv), t(jv), qd, md, jd, nefc=t(b.nefc), done=t(done))
    torch.cuda.synchronize()
    q, m, j = R.newton_advance(alpha, search, mv, jv, qacc, Ma, jaref, nefc=b.nefc, done=done)
    np.testing.assert_array_equal(qd.cpu().numpy(), q)
    np.testing.assert_array_equal(md.cpu().numpy(), m)
    np.testing.assert_array_equal(jd.cpu().numpy(), j)
    njmax = old.shape[1]
    ids = torch.full((nworld, njmax), -5, dtype=torch.int32, device=device)
    qc = torch.full((nworld,), -5, dtype=torch.int32, device=device)
    sc = torch.full((nworld,), -5, dtype=torch.int32, device=device)
    NF.changed_rows(t(old), t(new), ids, qc, sc, nefc=t(b.nefc), done=t(done), quad=synth.QUADRATIC)
    torch.cuda.synchronize()
    want = R.newton_changed_rows(old, new, quad=synth.QUADRATIC, nefc=b.nefc, done=done, ids=np.full((nworld, njmax), -5, np.int32),
                                 quad_count=np.full(nworld, -5, np.int32), state_count=np.full(nworld, -5, np.int32))  # fmt: skip
    for got, ref in zip((ids, qc, sc), want):
        np.testing.assert_array_equal(got.cpu().numpy(), ref)


# ---------------------------------------------------------------- convergence test
def _convergence_case(nworld, seed=8):
    rng = np.random.default_rng(seed)
    alpha = rng.uniform(0.1, 1, nworld).astype(np.float32)
    imp = rng.uniform(1, 2, nworld).astype(np.float32)
    gd = rng.uniform(1, 4, nworld).astype(np.float32)
    de = rng.uniform(1, 4, nworld).astype(np.float32)
    niter = rng.integers(0, 3, nworld).astype(np.int32)
    done = (rng.uniform(size=nworld) < 0.1).astype(np.uint8)
    # one criterion each for a few worlds; the others fail all four
    kind = rng.integers(0, 6, nworld)
    alpha[kind == 1] = 0.0
    imp[kind == 2] = 1e-9
    gd[kind == 3] = 1e-16
    de[kind == 4] = 1e-9
    imp[kind == 5] = -1.0  # a negative improvement never counts
    return alpha, imp, gd, de, niter, done, kind


def test_oracle_convergence_criteria():
    nworld, nv, maxiter = 400, 27, 3
    alpha, imp, gd, de, niter, done, kind = _convergence_case(nworld)
    tol, inertia = np.array([1e-6, 2e-6], np.float32), np.array([0.5], np.float32)
    it, dn, ov, count = R.newton_converged(alpha, imp, gd, de, tol, inertia, nv, maxiter, niter, done, overflow_bit=4)
    live = done == 0
    np.testing.assert_array_equal(it[live], niter[live] + 1)
    np.testing.assert_array_equal(it[~live], niter[~live])
    met = np.isin(kind, (1, 2, 3, 4))
    out_of_iterations = (niter + 1 == maxiter) & ~met
    np.testing.assert_array_equal(dn[live], (met | out_of_iterations)[live].astype(np.uint8))
    assert (dn[~live] == 1).all()
    np.testing.assert_array_equal(ov[live], np.where(out_of_iterations, 4, 0)[live])
    assert count == int((live & (met | out_of_iterations)).sum())


@pytest.mark.gpu
def test_gpu_convergence_bitwise(device):
    import torch

    nworld, nv, maxiter = 5000, 27, 3
    alpha, imp, gd, de, niter, done, _ = _convergence_case(nworld)
    tol, inertia = np.array([1e-6, 2e-6], np.float32), np.array([0.5, 0.7, 0.9], np.float32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    it, dn = t(niter), t(done)
    ov = torch.zeros(nworld, dtype=torch.int32, device=device)
    ns = torch.full((1,), int((done == 0).sum()), dtype=torch.int32, device=device)
    NF.converged(t(alpha), t(imp), t(gd), t(de), t(tol), t(inertia), nv, maxiter, it, dn, overflow=ov, overflow_bit=4, nsolving=ns)
    torch.cuda.synchronize()
    want = R.newton_converged(alpha, imp, gd, de, tol, inertia, nv, maxiter, niter, done, overflow_bit=4)
    np.testing.assert_array_equal(it.cpu().numpy(), want[0])
    np.testing.assert_array_equal(dn.cpu().numpy(), want[1])
    np.testing.assert_array_equal(ov.cpu().numpy(), want[2])
    assert int(ns.item()) == int((done == 0).sum()) - want[3]


@pytest.mark.gpu
def test_gpu_start_and_finish_of_the_fused_solve(device):
    """_init_efc_settling_empty_worlds and qfrc_constraint_from_grad (newton_fusion.py:412-428,
    537-555) against their statements in NumPy float32, bit for bit."""
    import torch

    nworld, nv = 777, 35
    rng = np.random.default_rng(12)
    nefc = rng.integers(0, 3, nworld).astype(np.int32)  # a third of the worlds have no rows
    f = lambda *shape: rng.normal(size=shape).astype(np.float32)  # noqa: E731
    smooth, Ma, grad, scale, qacc0 = f(nworld, nv), f(nworld, nv), f(nworld, nv), f(nworld), f(nworld, nv)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    niter = torch.full((nworld,), 9, dtype=torch.int32, device=device)
    sdot, done, qacc = torch.full((nworld,), 9.0, device=device), torch.full((nworld,), 9, dtype=torch.uint8, device=device), t(qacc0)
    NF.init_empty_worlds(t(nefc), t(smooth), niter, sdot, done, qacc)
    out = torch.full((nworld, nv), 9.0, device=device)
    NF.qfrc_constraint_from_grad(t(nefc), t(smooth), t(Ma), t(grad), t(scale), out)
    torch.cuda.synchronize()
    empty = nefc == 0
    assert not niter.any() and not sdot.any()
    np.testing.assert_array_equal(done.cpu().numpy(), empty.astype(np.uint8))
    np.testing.assert_array_equal(qacc.cpu().numpy(), np.where(empty[:, None], smooth, qacc0))
    want = np.where(empty[:, None], np.float32(0), (Ma - smooth) - scale[:, None] * grad)
    np.testing.assert_array_equal(out.cpu().numpy(), want)
