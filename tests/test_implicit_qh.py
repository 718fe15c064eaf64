"""The implicit-fast integrator's matrix qH = M - h dF/dv on M's pattern and the solve on it
(reference: src/instantmimic/utils/mjw_step_optimized.py:3734-3745, 3803-3900, 4936-4968).  The
upstream derivative kernels are not in the reference tree, so the checks are against the dense
fp64 statement of MuJoCo's mjd_smooth_vel for this integrator: parity with upstream's own bits is
unpinned."""

from types import SimpleNamespace

import numpy as np
import pytest

from instantmimic_amd import synth
from instantmimic_amd.mjw_kernels import implicit_qh as Q
from oracle import ref as R

H_STEP = 0.004


def _model(nworld, seed=3):
    return synth.make_implicit_case(nworld, H_STEP, seed)


def _dense64(m, d, st, nv0):
    """qH in dense fp64: M + h diag(b) - h A' diag(g) A + h Jt' diag(bt) Jt on M's pattern, the free
    body's rows equal to M."""
    rowadr, rownnz, colind = st
    nworld, nv = d.nworld, m.nv
    M64 = synth.dense_from_csr(d.M.astype(np.float64), *st)
    gain = np.where(m.actuator_biastype == 1, m.actuator_biasprm[:, 2], 0.0)[None, :] + np.where(m.actuator_gaintype == 1, m.actuator_gainprm[:, 2], 0.0)[None, :] * d.ctrl.astype(np.float64)
    out = (m.actuator_forcelimited[None, :] != 0) & ((d.actuator_force <= -1.0) | (d.actuator_force >= 1.0))
    gain = np.where(out, 0.0, gain)

    def dense_rows(nnz, adr, col, vals):
        A = np.zeros((nworld, len(nnz), nv))
        for r in range(len(nnz)):
            A[:, r, col[adr[r] : adr[r] + nnz[r]]] = vals[:, adr[r] : adr[r] + nnz[r]]
        return A

    A = dense_rows(d.moment_rownnz, d.moment_rowadr, d.moment_colind, d.actuator_moment)
    Jt = dense_rows(m.ten_J_rownnz, m.ten_J_rowadr, m.ten_J_colind, d.ten_J)
    dq = -np.einsum("wri,wr,wrj->wij", A, gain, A) + np.einsum("wri,r,wrj->wij", Jt, m.tendon_damping.astype(np.float64), Jt)
    dq[:, np.arange(nv), np.arange(nv)] += m.dof_damping.astype(np.float64)
    pattern = np.zeros((nv, nv), bool)
    rowi = np.repeat(np.arange(nv), rownnz)
    pattern[rowi, colind] = pattern[colind, rowi] = True
    pattern[nv0:, :] = pattern[:, nv0:] = False  # the free body keeps M
    return M64 + H_STEP * dq * pattern[None], gain


def _oracle_qh(m, d, st):
    """The oracle chained as the product chains its kernels."""
    from instantmimic_amd.muscle import muscle_qfrc_projector as MQ

    elemid = Q.matrix_elemid(m)
    qh = R.implicit_qh_base(d.M, Q.element_dofs(m), m.dof_damping, H_STEP)
    gain = R.actuator_velocity_gain(m.actuator_gaintype, m.actuator_biastype, m.actuator_gainprm, m.actuator_biasprm, d.ctrl,
                                    m.actuator_forcelimited, m.actuator_forcerange, d.actuator_force)  # fmt: skip
    for (nnz, adr, col), vals, weight, h in (((d.moment_rownnz, d.moment_rowadr, d.moment_colind), d.actuator_moment, gain, -H_STEP),
                                             ((m.ten_J_rownnz, m.ten_J_rowadr, m.ten_J_colind), d.ten_J, np.broadcast_to(m.tendon_damping, (d.nworld, m.ntendon)).copy(), H_STEP)):  # fmt: skip
        rows = np.repeat(np.arange(len(nnz)), nnz)
        pos = np.concatenate([np.arange(a, a + n) for a, n in zip(adr, nnz)])
        order = np.lexsort((col[pos], rows))
        ent = MQ.entries_from_muscle_dofs(np.stack([rows[order], col[pos][order]], 1), len(nnz))
        prepared = MQ.prepare_muscle_implicit_qderiv_pairs(
            pair_entry_i=ent.pair_entry_i, pair_entry_j=ent.pair_entry_j, pair_muscle_idx=ent.pair_muscle_idx,
            muscle_dof_torque_idx=ent.muscle_dof_torque_idx, matrix_elemid=elemid, root_dof_count=0)  # fmt: skip
        tables = MQ.gather_tables(prepared, ent.muscle_dof_muscle_idx)
        qh = R.muscle_implicit_gather(vals[:, pos[order]], weight, ent.muscle_dof_muscle_idx, tables[0], tables[1], tables[2], tables[4], h, qh)
    return qh, gain


def test_oracle_against_fp64():
    m, d, st, nv0 = _model(20)
    want, gain64 = _dense64(m, d, st, nv0)
    qh, gain = _oracle_qh(m, d, st)
    np.testing.assert_allclose(gain, gain64, rtol=1e-6, atol=1e-6)
    assert (gain == 0).any() and (gain != 0).any()
    got = synth.dense_from_csr(qh.astype(np.float64), *st)
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=2e-6 * np.abs(want).max())
    # the terms are there: damping, actuators and tendons each move some element, the free body none
    rowi = np.repeat(np.arange(m.nv), st[1])
    assert np.array_equal(qh[:, rowi >= nv0], d.M[:, rowi >= nv0])
    assert (qh[:, rowi < nv0] != d.M[:, rowi < nv0]).mean() > 0.05
    off = (rowi != st[2]) & (rowi < nv0)
    assert (qh[:, off] != d.M[:, off]).any()


def _with_polynomial_dampers(m, d, rng):
    m.dof_dampingpoly = (rng.uniform(0.0, 0.5, (m.nv, 2)) * (rng.random((m.nv, 1)) < 0.6)).astype(np.float32)
    m.tendon_dampingpoly = rng.uniform(0.0, 0.8, (m.ntendon, 3)).astype(np.float32)
    d.qvel = rng.normal(scale=2.0, size=(d.nworld, m.nv)).astype(np.float32)
    d.ten_velocity = rng.normal(scale=1.5, size=(d.nworld, m.ntendon)).astype(np.float32)


def test_oracle_polynomial_damping_is_the_slope_of_the_force():
    rng = np.random.default_rng(12)
    base = rng.uniform(0, 2, 9).astype(np.float32)
    poly = rng.uniform(0, 1, (9, 3)).astype(np.float32)
    v = rng.normal(scale=2.0, size=(5, 9)).astype(np.float32)
    v[0, 0] = 0.0
    got = R.polynomial_damping(base, poly, v)

    def force(x):
        a = np.abs(x)
        return -x * (base.astype(np.float64) + sum(poly[:, k].astype(np.float64) * a ** (k + 1) for k in range(3)))

    eps = 1e-6
    slope = -(force(v.astype(np.float64) + eps) - force(v.astype(np.float64) - eps)) / (2 * eps)
    np.testing.assert_allclose(got, slope, rtol=2e-6, atol=1e-6)
    assert got[0, 0] == base[0]
    np.testing.assert_array_equal(R.polynomial_damping(base, np.zeros((9, 0), np.float32), v), np.broadcast_to(base, v.shape))
    # per-world coefficients
    pw = rng.uniform(0, 1, (5, 9, 2)).astype(np.float32)
    bw = rng.uniform(0, 1, (5, 9)).astype(np.float32)
    want = bw + 2 * pw[:, :, 0].astype(np.float64) * np.abs(v) + 3 * pw[:, :, 1].astype(np.float64) * v.astype(np.float64) ** 2
    np.testing.assert_allclose(R.polynomial_damping(bw, pw, v), want, rtol=2e-6)


def test_tables():
    m, d, st, nv0 = _model(1)
    np.testing.assert_array_equal(Q.free_dofs(m), np.arange(nv0, nv0 + 6))
    ed = Q.element_dofs(m)
    rowi = np.repeat(np.arange(m.nv), st[1])
    assert (ed[rowi >= nv0] == -1).all() and (ed[(rowi == st[2]) & (rowi < nv0)] >= 0).all() and (ed[rowi != st[2]] == -1).all()
    assert (Q.element_dofs(m, damper=False) == -1).all()
    eid = Q.matrix_elemid(m)
    assert (eid[nv0:, :] == -1).all() and (eid[:, nv0:] == -1).all() and np.array_equal(eid, eid.T)
    del m.body_freeadr
    assert Q.free_dofs(m).size == 0 and (Q.matrix_elemid(m)[nv0:, nv0:] >= 0).any()


@pytest.mark.gpu
def test_gpu_qh_and_solve(device):
    import torch

    from instantmimic_amd.mjw_kernels import tree_ldl as T

    nworld = 300
    m, d, st, nv0 = _model(nworld)
    want_qh, want_gain = _oracle_qh(m, d, st)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    dd = SimpleNamespace(nworld=nworld, M=t(d.M), moment_rownnz=d.moment_rownnz, moment_rowadr=d.moment_rowadr, moment_colind=d.moment_colind,
                         actuator_moment=t(d.actuator_moment), ten_J=t(d.ten_J), ctrl=t(d.ctrl), actuator_force=t(d.actuator_force),
                         efc=SimpleNamespace(Ma=t(d.efc.Ma)))  # fmt: skip
    scratch = Q.create_implicit_qh_scratch(m, dd, device)
    assert scratch.actuators.dropped_pair_count > 0  # pairs on the free body's rows: those rows keep M
    # one launch (im_implicit_qh), then the separate launches: base, gains, one gather per term
    for fused in (True, False):
        scratch.implicit_qderiv.fill_(float("nan"))
        scratch.actuator_gain.fill_(float("nan"))
        Q.deriv_smooth_vel(m, dd, scratch.implicit_qderiv, scratch, fused=fused)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(scratch.actuator_gain.cpu().numpy(), want_gain)
        np.testing.assert_array_equal(scratch.implicit_qderiv.cpu().numpy(), want_qh)
    # the whole step: qH, then the tree L'DL (the model is a forest: 56 + 6 dofs)
    scratch.tree_factor_solve = T.create_tree_factor_solve_scratch(m, device)
    assert scratch.tree_factor_solve is not None
    qacc = Q.implicit_factor_optimized(m, dd, scratch)
    torch.cuda.synchronize()
    x_ref = R.tree_ldl_solve(*st, __import__("oracle.planner", fromlist=["x"]).best_tree_ldl_plan(*st), want_qh, d.efc.Ma)
    np.testing.assert_array_equal(qacc.cpu().numpy(), x_ref)
    want64, _ = _dense64(m, d, st, nv0)
    x64 = np.linalg.solve(want64, d.efc.Ma.astype(np.float64)[:, :, None])[:, :, 0]
    err = np.linalg.norm(qacc.cpu().numpy() - x64, axis=1) / np.linalg.norm(x64, axis=1)
    assert (err / (np.linalg.cond(want64) * 6e-8)).max() < 2.0
    # a contributor rides on top (the muscles' h A'sA enters this way)
    class Twice:
        def apply(self, qh):
            qh.mul_(2.0)

    scratch.implicit_qh_contributors = (Twice(),)
    q2 = Q.implicit_factor_optimized(m, dd, scratch).clone()
    torch.cuda.synchronize()
    np.testing.assert_array_equal(scratch.implicit_qderiv.cpu().numpy(), 2.0 * want_qh)
    np.testing.assert_allclose(q2.cpu().numpy(), 0.5 * x_ref, rtol=1e-3, atol=1e-4 * np.abs(x_ref).max())


@pytest.mark.gpu
def test_gpu_qh_with_polynomial_dampers(device):
    """dof_dampingpoly and tendon_dampingpoly: the slope of each damper at the current velocity takes
    the place of its constant coefficient; both forms of the assembly, against the oracle chained
    the same way and against the dense fp64 matrix with those slopes."""
    import torch

    nworld = 130
    m, d, st, nv0 = _model(nworld, seed=5)
    _with_polynomial_dampers(m, d, np.random.default_rng(6))
    dof_eff = R.polynomial_damping(m.dof_damping, m.dof_dampingpoly, d.qvel)
    ten_eff = R.polynomial_damping(m.tendon_damping, m.tendon_dampingpoly, d.ten_velocity)
    assert (dof_eff > m.dof_damping).any() and (ten_eff > m.tendon_damping).all()
    plain_dof, plain_ten = m.dof_damping, m.tendon_damping
    want = []
    for w in range(nworld):  # the oracle's chain takes one set of coefficients: world by world
        m.dof_damping, m.tendon_damping = dof_eff[w], ten_eff[w]
        one = SimpleNamespace(**{k: (v[w : w + 1] if isinstance(v, np.ndarray) and v.ndim > 1 and v.shape[0] == nworld else v) for k, v in vars(d).items()})
        one.nworld = 1
        want.append(_oracle_qh(m, one, st)[0][0])
    want = np.stack(want)
    m.dof_damping, m.tendon_damping = plain_dof, plain_ten
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    dd = SimpleNamespace(nworld=nworld, M=t(d.M), moment_rownnz=d.moment_rownnz, moment_rowadr=d.moment_rowadr, moment_colind=d.moment_colind,
                         actuator_moment=t(d.actuator_moment), ten_J=t(d.ten_J), ctrl=t(d.ctrl), actuator_force=t(d.actuator_force),
                         qvel=t(d.qvel), ten_velocity=t(d.ten_velocity), efc=SimpleNamespace(Ma=t(d.efc.Ma)))  # fmt: skip
    scratch = Q.create_implicit_qh_scratch(m, dd, device)
    for fused in (True, False):
        scratch.implicit_qderiv.fill_(float("nan"))
        Q.deriv_smooth_vel(m, dd, scratch.implicit_qderiv, scratch, fused=fused)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(scratch.tables["dof_effective"].cpu().numpy(), dof_eff)
        np.testing.assert_array_equal(scratch.tendon_damping.cpu().numpy(), ten_eff)
        np.testing.assert_array_equal(scratch.implicit_qderiv.cpu().numpy(), want)
    # a fluid model is still refused
    m.has_fluid = True
    with pytest.raises(NotImplementedError):
        Q.create_implicit_qh_scratch(m, dd, device)
