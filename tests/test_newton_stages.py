"""Per-iteration factor stage: incremental Hessian update over the changed constraint rows,
refactor or solve-only, on the static sparse pattern and on the dense Hessian with the
augmented blocked Cholesky."""

import numpy as np
import pytest

from instantmimic_amd import synth
from instantmimic_amd.mjw_kernels import newton_stages as NS
from instantmimic_amd.mjw_kernels import sparse_hessian as S
from oracle import planner as P
from oracle import ref as R

Q = synth.QUADRATIC


def _contact_case(nworld, seed):
    m, ids = synth.contact_model()
    groups = [[ids["footL"], ids["boxB"]]]
    nv = m.nv
    sup = list(synth.chain_mask(list(m.dof_parentid)))
    for g in groups:
        mask = np.zeros(nv, bool)
        for b in g:
            mask[P.body_chain(b, m.body_parentid, m.body_dofadr, m.body_dofnum)] = True
        sup += [mask] * 6
    shape = synth.Shape("contact", tuple(int(p) for p in m.dof_parentid), 40, nworld, (0.5, 8.0), 0.02, (-4.0, 4.0),
                        0.6, 2, seed)  # fmt: skip
    return m, groups, synth.make_batch(shape, nworld, ragged_nefc=True, supports=np.array(sup))


def _changes(b, rng):
    """Row lists of the second iteration: rows (below nefc) whose quadratic-ness flipped, in
    ascending order; every 5th world has none (solve-only), every 7th is untouched
    (state_changes == 0), world 3 is done."""
    nworld, njmax = b.D.shape
    new = b.state[1].copy()
    new[::5] = b.state[0][::5]
    ids = np.zeros((nworld, njmax), np.int32)
    changes = np.zeros(nworld, np.int32)
    for w in range(nworld):
        rows = np.flatnonzero((new[w] == Q) != (b.state[0][w] == Q))
        rows = rows[rows < b.nefc[w]]
        # rows at or beyond nefc keep their old contribution (none): restore their state
        keep = np.ones(njmax, bool)
        keep[rows] = False
        new[w, keep] = b.state[0][w, keep]
        ids[w, : len(rows)] = rows
        changes[w] = len(rows)
    state_changes = np.maximum(changes, 1).astype(np.int32)
    state_changes[::7] = 0
    done = np.zeros(nworld, np.uint8)
    done[3] = 1
    grad = rng.standard_normal(b.grad.shape).astype(np.float32)
    return new, ids, changes, state_changes, done, grad


def _live(state_changes, done):
    return (state_changes != 0) & (done == 0)


# ---------------------------------------------------------------- oracle pinning (CPU)


def test_oracle_sparse_stage_against_fp64():
    m, groups, b = _contact_case(36, 21)
    rng = np.random.default_rng(4)
    for block in (32, 64):
        plan = R.sparse_plan(m, groups, block)
        hf0, *_ = R.sparse_init_factor(plan, b.nefc, b.J, b.D, b.state[0], b.M, b.grad)
        new, ids, changes, sc, done, grad = _changes(b, rng)
        hf, uni, search, sdot, decr = R.sparse_update_factor(plan, sc, changes, ids, b.J, b.D, new, grad, hf0, done=done)
        live = _live(sc, done)
        st = (b.rowadr, b.rownnz, b.colind)
        Hd = R.assemble_dense64(*st, b.M, b.J, b.D, new, b.nefc)
        sa, sb = plan.tables["SH_SA"], plan.tables["SH_SB"]
        nfac = plan.nfac
        packed = hf.reshape(len(hf), -1)[:, :nfac]
        # the incrementally updated H equals a fresh assembly with the new states
        # (to the rounding of the larger of the two: removed rows cancel)
        Hold = R.assemble_dense64(*st, b.M, b.J, b.D, b.state[0], b.nefc)
        scale = np.maximum(np.abs(Hd).max(axis=(1, 2)), np.abs(Hold).max(axis=(1, 2)))[:, None]
        assert (np.abs(packed - Hd[:, sa, sb]) / scale)[live].max() < 2e-6
        assert (hf[:, -1, -1] == 0).all()
        # untouched worlds keep their buffers
        np.testing.assert_array_equal(hf[~live], hf0[~live])
        assert not search[~live].any()
        # dof union = ascending dofs any changed row touches
        for w in np.flatnonzero(live & (changes > 0)):
            want = np.flatnonzero((b.J[w, ids[w, : changes[w]]] != 0).any(axis=0))
            assert uni[w, m.nv] == len(want) and np.array_equal(uni[w, : len(want)], want)
        x64 = R.solve64(Hd, grad)
        cond = np.linalg.cond(Hd)
        err = np.linalg.norm(-search - x64, axis=1) / np.linalg.norm(x64, axis=1)
        assert (err / (cond * 6e-8))[live].max() < 4.0
        np.testing.assert_allclose(decr[live], (grad * x64).sum(1)[live], rtol=2e-3, atol=2e-3 * np.abs(decr).max())
        # solve-only worlds reuse the stored factor: same answer as refactoring the same H
        solve_only = live & (changes == 0)
        assert solve_only.any()
        again, *_ = R.sparse_init_factor(plan, b.nefc, b.J, b.D, new, b.M, grad)
        _, _, s2, _, _ = R.sparse_update_factor(plan, sc, changes, ids, b.J, b.D, new, grad, again, done=done)
        assert R.rel_l2(search[solve_only], s2[solve_only]) < 1e-4


def _dense_start(b, pad):
    st = (b.rowadr, b.rownnz, b.colind)
    Md = synth.dense_from_csr(b.M, *st).astype(np.float32)
    H0 = R.jtdj_dense(Md, b.J, b.D, b.state[0], b.nefc, pad)
    return st, H0


@pytest.mark.parametrize("name,nworld", [("g1", 24), ("stress", 6)])
def test_oracle_dense_stage_against_fp64(name, nworld):
    shape = synth.SHAPES[name]
    import dataclasses

    b = synth.make_batch(dataclasses.replace(shape, iterations=2), nworld, ragged_nefc=True)
    nv = shape.nv
    pad = ((nv + 1 + 15) // 16) * 16
    rng = np.random.default_rng(8)
    st, H0 = _dense_start(b, pad)
    new, ids, changes, sc, done, grad = _changes(b, rng)
    U0 = np.zeros_like(H0)
    # first a refactor everywhere (changes as computed, solve-only worlds refactor at state 0)
    first_changes = np.where(changes == 0, 0, changes)
    H1, U1, uni, search, sdot, decr = R.dense_update_factor(
        np.ones_like(sc), np.maximum(first_changes, 0), ids, b.J, b.D, new, grad, H0, U0
    )
    refactored = first_changes > 0
    Hd = R.assemble_dense64(*st, b.M, b.J, b.D, new, b.nefc)
    iu = np.triu_indices(nv)
    Hold = R.assemble_dense64(*st, b.M, b.J, b.D, b.state[0], b.nefc)
    scale = np.maximum(np.abs(Hd).max(axis=(1, 2)), np.abs(Hold).max(axis=(1, 2)))[:, None]
    assert (np.abs(H1[:, :nv, :nv][:, iu[0], iu[1]] - Hd[:, iu[0], iu[1]]) / scale)[refactored].max() < 3e-6
    # the strict lower triangle and the padding are left alone
    il = np.tril_indices(nv, -1)
    np.testing.assert_array_equal(H1[:, il[0], il[1]], H0[:, il[0], il[1]])
    # stored factor: U'U = [[H, g], [g', 1e30]] with identity padding
    for w in np.flatnonzero(refactored)[:4]:
        U = U1[w].astype(np.float64)
        assert np.allclose(np.tril(U, -1), 0.0)
        aug = np.eye(pad)
        aug[:nv, :nv] = np.triu(H1[w, :nv, :nv].astype(np.float64)) + np.triu(H1[w, :nv, :nv].astype(np.float64), 1).T
        aug[:nv, pad - 1] = aug[pad - 1, :nv] = grad[w]
        aug[pad - 1, pad - 1] = 1e30
        got = U.T @ U
        assert np.abs(got[:nv, :nv] - aug[:nv, :nv]).max() < 1e-5 * np.abs(aug[:nv, :nv]).max()
        assert np.abs(got[:nv, pad - 1] - grad[w]).max() < 1e-5 * np.abs(grad[w]).max()
        assert abs(got[pad - 1, pad - 1] / 1e30 - 1) < 1e-6
    x64 = R.solve64(Hd, grad)
    cond = np.linalg.cond(Hd)
    err = np.linalg.norm(-search - x64, axis=1) / np.linalg.norm(x64, axis=1)
    assert (err / (cond * 6e-8))[refactored].max() < 4.0
    sd64 = (x64**2).sum(1)
    assert (np.abs(sdot - sd64) / sd64 / np.maximum(cond * 6e-8, 1e-6))[refactored].max() < 10.0
    # then a solve-only pass with a new gradient against the stored factor
    grad2 = rng.standard_normal(grad.shape).astype(np.float32)
    H2, U2, _, search2, _, decr2 = R.dense_update_factor(
        np.ones_like(sc), np.zeros_like(changes), ids, b.J, b.D, new, grad2, H1, U1
    )
    np.testing.assert_array_equal(H2, H1)
    np.testing.assert_array_equal(U2, U1)
    x64 = R.solve64(Hd, grad2)
    err = np.linalg.norm(-search2 - x64, axis=1) / np.linalg.norm(x64, axis=1)
    assert (err / (cond * 6e-8))[refactored].max() < 4.0


# ---------------------------------------------------------------- GPU parity


def _t(a, device):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


@pytest.mark.gpu
@pytest.mark.parametrize("block", [32, 64])
def test_gpu_sparse_stage_bitwise(device, block):
    import torch

    m, groups, b = _contact_case(150, 23)
    rng = np.random.default_rng(5)
    plan = S.build_plan(m, groups, block, device=device)
    oplan = R.sparse_plan(m, groups, block)
    hf0, *_ = R.sparse_init_factor(oplan, b.nefc, b.J, b.D, b.state[0], b.M, b.grad)
    new, ids, changes, sc, done, grad = _changes(b, rng)
    # one update outside the declared pattern: a changed row coupling the two arms
    w_bad = int(np.flatnonzero(_live(sc, done) & (changes > 0))[0])
    r_bad = ids[w_bad, 0]
    b.J[w_bad, r_bad, :] = 0.0
    b.J[w_bad, r_bad, [18, 21]] = 1.0
    want = R.sparse_update_factor(oplan, sc, changes, ids, b.J, b.D, new, grad, hf0, done=done)
    nworld, nv = b.nworld, m.nv
    hf = _t(hf0, device)
    uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=device)
    search = torch.zeros((nworld, nv), device=device)
    sdot, decr = torch.zeros(nworld, device=device), torch.zeros(nworld, device=device)
    stage = NS.factor_factory(nv, m.nv_pad, plan)
    stage(_t(b.J, device), _t(b.D, device), _t(new, device), _t(ids, device), _t(changes, device), _t(sc, device),
          _t(done, device), _t(grad, device), None, hf, search, sdot, decr, uni)  # fmt: skip
    torch.cuda.synchronize()
    got = (hf.cpu().numpy(), uni.cpu().numpy(), search.cpu().numpy(), sdot.cpu().numpy(), decr.cpu().numpy())
    assert got[0][w_bad, -1, -1] == 1.0 and want[0][w_bad, -1, -1] == 1.0
    n_used = 2 * plan.nfac + nv
    np.testing.assert_array_equal(got[0].reshape(nworld, -1)[:, :n_used], want[0].reshape(nworld, -1)[:, :n_used])
    np.testing.assert_array_equal(got[0][:, -1, -1], want[0][:, -1, -1])
    refactored = _live(sc, done) & (changes > 0)
    np.testing.assert_array_equal(got[1][refactored], want[1][refactored])
    for g, r in zip(got[2:], want[2:]):
        np.testing.assert_array_equal(g, r)


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld", [("g1", 130), ("snu", 70), ("stress", 20)])
def test_gpu_dense_stage_bitwise(device, name, nworld):
    import dataclasses

    import torch

    shape = synth.SHAPES[name]
    b = synth.make_batch(dataclasses.replace(shape, iterations=2), nworld, ragged_nefc=True)
    nv = shape.nv
    pad = ((nv + 1 + 15) // 16) * 16
    rng = np.random.default_rng(9)
    _, H0 = _dense_start(b, pad)
    new, ids, changes, sc, done, grad = _changes(b, rng)
    U0 = np.broadcast_to(np.eye(pad, dtype=np.float32), H0.shape).copy()
    want1 = R.dense_update_factor(sc, changes, ids, b.J, b.D, new, grad, H0, U0, done=done)
    grad2 = rng.standard_normal(grad.shape).astype(np.float32)
    zero = np.zeros_like(changes)
    want2 = R.dense_update_factor(sc, zero, ids, b.J, b.D, new, grad2, want1[0], want1[1], done=done)
    H, U = _t(H0, device), _t(U0, device)
    uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=device)
    search = torch.zeros((nworld, pad, 1), device=device)
    sdot, decr = torch.zeros(nworld, device=device), torch.zeros(nworld, device=device)
    stage = NS.factor_factory(nv, pad)
    g3 = torch.zeros((nworld, pad, 1), device=device)
    g3[:, :nv, 0] = _t(grad, device)
    common = (_t(b.J, device), _t(b.D, device), _t(new, device), _t(ids, device))
    stage(*common, _t(changes, device), _t(sc, device), _t(done, device), g3, H, U, search, sdot, decr, uni)
    torch.cuda.synchronize()
    refactored = _live(sc, done) & (changes > 0)
    np.testing.assert_array_equal(H.cpu().numpy(), want1[0])
    np.testing.assert_array_equal(U.cpu().numpy(), want1[1])
    np.testing.assert_array_equal(uni.cpu().numpy()[refactored], want1[2][refactored])
    np.testing.assert_array_equal(search.cpu().numpy()[:, :nv, 0], want1[3])
    np.testing.assert_array_equal(sdot.cpu().numpy(), want1[4])
    np.testing.assert_array_equal(decr.cpu().numpy(), want1[5])
    # solve-only against the stored factor
    g3[:, :nv, 0] = _t(grad2, device)
    stage(*common, _t(zero, device), _t(sc, device), _t(done, device), g3, H, U, search, sdot, decr, uni)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(U.cpu().numpy(), want2[1])
    live = _live(sc, done)
    np.testing.assert_array_equal(search.cpu().numpy()[live][:, :nv, 0], want2[3][live])
    np.testing.assert_array_equal(decr.cpu().numpy()[live], want2[5][live])


def _toggled(b, rng, counts):
    """World w has counts[w % len(counts)] rows whose quadratic-ness flips (rows below nefc, ascending);
    every world is live."""
    nworld, njmax = b.D.shape
    new = b.state[0].copy()
    ids = np.zeros((nworld, njmax), np.int32)
    changes = np.zeros(nworld, np.int32)
    for w in range(nworld):
        k = min(int(counts[w % len(counts)]), int(b.nefc[w]))
        rows = np.sort(rng.choice(int(b.nefc[w]), size=k, replace=False))
        new[w, rows] = np.where(b.state[0][w, rows] == Q, 0, Q)
        ids[w, :k] = rows
        changes[w] = k
    grad = rng.standard_normal(b.grad.shape).astype(np.float32)
    return new, ids, changes, np.ones(nworld, np.int32), np.zeros(nworld, np.uint8), grad


# changed rows per world: inside the staged capacities (16 and 32 rows), inside what the masks hold
# (128), and beyond, where the pairs read J row by row
_MANY = (0, 3, 16, 17, 32, 33, 64, 127, 128, 129, 150, 160)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["ant", "humanoid", "g1", "snu"])
def test_gpu_dense_stage_with_up_to_160_changed_rows(device, name):
    """The single tile (ant: 16 columns, humanoid: 32) and the 48- and 64-column stages with 160 rows per world, of which
    0 to 160 change: every form of the update (staged rows, masks, row by row) against the CPU
    restatement, bit for bit."""
    import dataclasses

    import torch

    shape = dataclasses.replace(synth.SHAPES[name], nefc=160, iterations=1)
    nworld = 2 * len(_MANY) + 1
    b = synth.make_batch(shape, nworld, ragged_nefc=False)
    nv = shape.nv
    pad = ((nv + 1 + 15) // 16) * 16
    rng = np.random.default_rng(31)
    _, H0 = _dense_start(b, pad)
    new, ids, changes, sc, done, grad = _toggled(b, rng, _MANY)
    assert changes.max() == 160 and set(_MANY) <= set(changes.tolist())
    U0 = np.broadcast_to(np.eye(pad, dtype=np.float32), H0.shape).copy()
    want = R.dense_update_factor(sc, changes, ids, b.J, b.D, new, grad, H0, U0, done=done)
    H, U = _t(H0, device), _t(U0, device)
    uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=device)
    search = torch.zeros((nworld, pad, 1), device=device)
    sdot, decr = torch.zeros(nworld, device=device), torch.zeros(nworld, device=device)
    g3 = torch.zeros((nworld, pad, 1), device=device)
    g3[:, :nv, 0] = _t(grad, device)
    NS.factor_factory(nv, pad)(_t(b.J, device), _t(b.D, device), _t(new, device), _t(ids, device), _t(changes, device),
                               _t(sc, device), _t(done, device), g3, H, U, search, sdot, decr, uni)  # fmt: skip
    torch.cuda.synchronize()
    np.testing.assert_array_equal(H.cpu().numpy(), want[0])
    np.testing.assert_array_equal(U.cpu().numpy(), want[1])
    refactored = changes > 0
    np.testing.assert_array_equal(uni.cpu().numpy()[refactored], want[2][refactored])
    np.testing.assert_array_equal(search.cpu().numpy()[:, :nv, 0], want[3])
    np.testing.assert_array_equal(sdot.cpu().numpy(), want[4])
    np.testing.assert_array_equal(decr.cpu().numpy(), want[5])


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["g1", "snu"])
def test_gpu_sparse_stage_with_up_to_160_changed_rows(device, name):
    """The same for the sparse stage on the benchmark trees' plans."""
    import dataclasses

    import torch

    shape = dataclasses.replace(synth.SHAPES[name], nefc=160, iterations=1)
    m = synth.model_from_parents(shape.parents)
    block = S.block_width(m.nv_pad)
    plan, reason = S.plan_for_model(m, None, [], block, device=device)
    assert plan is not None, reason
    oplan = R.sparse_plan(m, [], block)
    nworld = 2 * len(_MANY) + 1
    b = synth.make_batch(shape, nworld, ragged_nefc=False)
    rng = np.random.default_rng(37)
    hf0, *_ = R.sparse_init_factor(oplan, b.nefc, b.J, b.D, b.state[0], b.M, b.grad)
    new, ids, changes, sc, done, grad = _toggled(b, rng, _MANY)
    want = R.sparse_update_factor(oplan, sc, changes, ids, b.J, b.D, new, grad, hf0, done=done)
    nv = m.nv
    hf = _t(hf0, device)
    uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=device)
    search = torch.zeros((nworld, nv), device=device)
    sdot, decr = torch.zeros(nworld, device=device), torch.zeros(nworld, device=device)
    NS.factor_factory(nv, m.nv_pad, plan)(_t(b.J, device), _t(b.D, device), _t(new, device), _t(ids, device), _t(changes, device),
                                          _t(sc, device), _t(done, device), _t(grad, device), None, hf, search, sdot, decr, uni)  # fmt: skip
    torch.cuda.synchronize()
    n_used = 2 * plan.nfac + nv
    np.testing.assert_array_equal(hf.cpu().numpy().reshape(nworld, -1)[:, :n_used], want[0].reshape(nworld, -1)[:, :n_used])
    refactored = changes > 0
    np.testing.assert_array_equal(uni.cpu().numpy()[refactored], want[1][refactored])
    np.testing.assert_array_equal(search.cpu().numpy(), want[2])
    np.testing.assert_array_equal(sdot.cpu().numpy(), want[3])
    np.testing.assert_array_equal(decr.cpu().numpy(), want[4])


@pytest.mark.gpu
def test_gpu_block_per_world_sparse_kernels_agree():
    """The sparse factor has two kernels per entry point (a wavefront per world with the tables in
    LDS, and a workgroup of the plan's width per world for models it does not fit): the second
    family is forced here in a child process and must pass the same bitwise comparisons."""
    import os
    import subprocess
    import sys

    env = dict(os.environ, IMHIP_SPARSE_KERNEL="simple")
    code = (
        "import sys, torch; sys.path.insert(0, 'tests');"
        "import test_newton_stages as a, test_sparse_hessian as b; d = torch.device('cuda:0');"
        "a.test_gpu_sparse_stage_bitwise(d, 32); a.test_gpu_sparse_stage_bitwise(d, 64);"
        "b.test_gpu_contact_model_bitwise(d, 1, 32); b.test_gpu_benchmark_trees_bitwise(d, 'snu', 100);"
        "b.test_gpu_done_mask_violation_counter_and_graph_replay(d); print('block-per-world kernels ok')"
    )
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "block-per-world kernels ok" in out.stdout, out.stderr[-2000:]


@pytest.mark.gpu
def test_gpu_changed_rows_feed_the_factor_stage(device):
    """The row lists and counts of im_newton_changed_rows, taken as they are by the sparse factor
    stage, against the oracle run on the lists that _changes() builds on its own."""
    import torch

    from instantmimic_amd.mjw_kernels import newton_fusion as NF

    m, groups, b = _contact_case(150, 23)
    rng = np.random.default_rng(5)
    plan = S.build_plan(m, groups, 64, device=device)
    oplan = R.sparse_plan(m, groups, 64)
    hf0, *_ = R.sparse_init_factor(oplan, b.nefc, b.J, b.D, b.state[0], b.M, b.grad)
    new, ids, changes, _, done, grad = _changes(b, rng)
    nworld, nv, njmax = b.nworld, m.nv, b.D.shape[1]
    ids_d = torch.zeros((nworld, njmax), dtype=torch.int32, device=device)
    qc = torch.zeros(nworld, dtype=torch.int32, device=device)
    sc = torch.zeros(nworld, dtype=torch.int32, device=device)
    NF.changed_rows(_t(b.state[0], device), _t(new, device), ids_d, qc, sc, nefc=_t(b.nefc, device), quad=Q)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(qc.cpu().numpy(), changes)
    # a world whose states did not change at all is solve-only for the stage and skipped when its count is zero:
    # give every world at least the solve, as the reference's line search does through its own increments
    sc_np = np.maximum(sc.cpu().numpy(), 1).astype(np.int32)
    want = R.sparse_update_factor(oplan, sc_np, changes, ids, b.J, b.D, new, grad, hf0, done=done)
    hf = _t(hf0, device)
    uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=device)
    search = torch.zeros((nworld, nv), device=device)
    sdot, decr = torch.zeros(nworld, device=device), torch.zeros(nworld, device=device)
    stage = NS.factor_factory(nv, m.nv_pad, plan)
    stage(_t(b.J, device), _t(b.D, device), _t(new, device), ids_d, qc, _t(sc_np, device), _t(done, device),
          _t(grad, device), None, hf, search, sdot, decr, uni)  # fmt: skip
    torch.cuda.synchronize()
    n_used = 2 * plan.nfac + nv
    np.testing.assert_array_equal(hf.cpu().numpy().reshape(nworld, -1)[:, :n_used], want[0].reshape(nworld, -1)[:, :n_used])
    np.testing.assert_array_equal(search.cpu().numpy(), want[2])


@pytest.mark.gpu
def test_gpu_one_iteration_chained(device):
    """One Newton iteration with the library's pieces in the reference's order (J v, step, changed
    rows, gradient, factor stage, convergence test) against the oracle's pieces in the same order.
    The step length, the new states and the new forces come from outside, as they come from
    upstream code in the reference."""
    import torch

    from instantmimic_amd.mjw_kernels import newton_fusion as NF

    m, groups, b = _contact_case(150, 23)
    rng = np.random.default_rng(15)
    plan = S.build_plan(m, groups, 64, device=device)
    oplan = R.sparse_plan(m, groups, 64)
    nworld, nv, njmax = b.nworld, m.nv, b.D.shape[1]
    hf0, search0, sdot0, decr0 = R.sparse_init_factor(oplan, b.nefc, b.J, b.D, b.state[0], b.M, b.grad)
    new, _, _, _, done, _ = _changes(b, rng)
    f = lambda *shape: rng.normal(size=shape).astype(np.float32)  # noqa: E731
    alpha = rng.uniform(0.1, 1, nworld).astype(np.float32)
    mv, qacc, Ma, jaref, smooth, force = f(nworld, nv), f(nworld, nv), f(nworld, nv), f(nworld, njmax), f(nworld, nv), f(nworld, njmax)
    gd0, sc0 = rng.uniform(1, 2, nworld).astype(np.float32), np.ones(nworld, np.float32)
    imp = rng.uniform(0, 1e-3, nworld).astype(np.float32)
    tol, inertia = np.array([1e-6], np.float32), np.array([1.0], np.float32)
    # oracle chain
    jv = R.newton_jv(b.J, search0, nefc=b.nefc, skip=done)
    q1, Ma1, ja1 = R.newton_advance(alpha, search0, mv, jv, qacc, Ma, jaref, nefc=b.nefc, done=done)
    ids, qc, sc = R.newton_changed_rows(b.state[0], new, quad=Q, nefc=b.nefc, done=done)
    qcf, grad, gd, de, gs, un = R.newton_gradient(b.J, force, smooth, Ma1, sc, alpha, gd0, decr0, sc0, nefc=b.nefc, done=done, block=64)
    want = R.sparse_update_factor(oplan, sc, qc, ids, b.J, b.D, new, grad, hf0, done=done)
    ran = (done == 0) & (sc != 0)  # the factor stage leaves the other worlds' decrement as the gradient step left it
    it, dn, _, _ = R.newton_converged(alpha, imp, gd, np.where(ran, want[4], de), tol, inertia, nv, 5, np.zeros(nworld, np.int32), done)
    # the same on the GPU
    t = lambda a: _t(a, device)  # noqa: E731
    J, D, nefc, dn_d, al = t(b.J), t(b.D), t(b.nefc), t(done), t(alpha)
    search = t(search0)
    jv_d = torch.zeros((nworld, njmax), device=device)
    NF.jv(J, search, jv_d, nefc=nefc, skip_world=dn_d)
    q_d, Ma_d, ja_d = t(qacc), t(Ma), t(jaref)
    NF.advance(al, search, t(mv), jv_d, q_d, Ma_d, ja_d, nefc=nefc, done=dn_d)
    ids_d = torch.zeros((nworld, njmax), dtype=torch.int32, device=device)
    qc_d, sc_d = torch.zeros(nworld, dtype=torch.int32, device=device), torch.zeros(nworld, dtype=torch.int32, device=device)
    new_d = t(new)
    NF.changed_rows(t(b.state[0]), new_d, ids_d, qc_d, sc_d, nefc=nefc, done=dn_d, quad=Q)
    qcf_d, grad_d = torch.zeros((nworld, nv), device=device), torch.zeros((nworld, nv), device=device)
    gd_d, de_d, gs_d = t(gd0), t(decr0), t(sc0)
    un_d = torch.zeros(nworld, dtype=torch.uint8, device=device)
    NF.gradient(nefc, J, t(force), t(smooth), Ma_d, sc_d, al, dn_d, qcf_d, grad_d, gd_d, de_d, gs_d, un_d, block=64)
    hf = t(hf0)
    uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=device)
    sdot_d = t(sdot0)
    NS.factor_factory(nv, m.nv_pad, plan)(J, D, new_d, ids_d, qc_d, sc_d, dn_d, grad_d, None, hf, search, sdot_d, de_d, uni)
    it_d = torch.zeros(nworld, dtype=torch.int32, device=device)
    NF.converged(al, t(imp), gd_d, de_d, t(tol), t(inertia), nv, 5, it_d, dn_d)
    torch.cuda.synchronize()
    live = (done == 0) & (sc != 0)
    np.testing.assert_array_equal(q_d.cpu().numpy(), q1)
    np.testing.assert_array_equal(ja_d.cpu().numpy(), ja1)
    np.testing.assert_array_equal(grad_d.cpu().numpy()[live], grad[live])
    np.testing.assert_array_equal(search.cpu().numpy()[live], want[2][live])
    np.testing.assert_array_equal(de_d.cpu().numpy()[live], want[4][live])
    np.testing.assert_array_equal(it_d.cpu().numpy(), it)
    np.testing.assert_array_equal(dn_d.cpu().numpy(), dn)
