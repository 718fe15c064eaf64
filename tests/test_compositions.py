"""The configured workloads end to end: the pieces each benchmark configuration names, chained on
the GPU as a caller would chain them and checked against the oracle chained the same way."""

from types import SimpleNamespace

import numpy as np
import pytest

from instantmimic_amd import synth
from oracle import planner as P
from oracle import ref as R

pytestmark = pytest.mark.gpu
Q = synth.QUADRATIC


def _t(a, device):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def _model(b):
    return type("m", (), dict(nv=b.shape.nv, M_rowadr=b.rowadr, M_rownnz=b.rownnz, M_colind=b.colind))


def test_g1_blocked_b8_against_tree_ldl_on_the_same_hessians(device):
    """Configuration 3: nv = 35, 8192 worlds, the blocked-dense factor with 8 x 8 blocks compared
    against the tree L'DL.  Both solve the same H = M + J'DJ (assembled once on the GPU); they
    agree with each other and with the fp64 solve to within what cond(H) allows in fp32."""
    import torch

    from instantmimic_amd.mjw_kernels import blocked_dense as BD
    from instantmimic_amd.mjw_kernels import tree_ldl as T

    b = synth.make_batch("g1")
    nworld, nv = b.nworld, b.shape.nv
    assert nworld == 8192 and nv == 35
    scratch = T.create_tree_factor_solve_scratch(_model(b), device)
    M, J, D, S, N, G = (_t(a, device) for a in (b.M, b.J, b.D, b.state[0], b.nefc, b.grad))
    x_fused, H = torch.zeros_like(G), torch.zeros_like(M)
    T.assemble_tree_factor_solve(scratch, M, J, D, S, N, G, x_fused, H_out=H)
    # tree L'DL alone on the assembled H
    x_tree = torch.zeros_like(G)
    T.tree_factor_solve(scratch, H, x_tree, G)
    # the same H as one dense tile per world through the blocked Cholesky, B = 8
    torch.cuda.synchronize()
    Hd64 = R.dense_from_csr(H.cpu().numpy().astype(np.float64), b.rowadr, b.rownnz, b.colind)
    Hd = _t(Hd64.reshape(nworld, -1).astype(np.float32), device)
    m = SimpleNamespace(nv=nv, M_tiles=[SimpleNamespace(size=nv, elemid=np.arange(nv * nv))])
    d = SimpleNamespace(nworld=nworld, M=Hd)
    blocked = BD.create_blocked_dense_factor_solve_scratch(m, d, device, block_size=8)
    assert blocked.pad == 40
    x_blk = torch.zeros_like(G)
    BD._blocked_dense_factor_solve(d, Hd, x_blk, G, blocked)
    torch.cuda.synchronize()
    xt, xb = x_tree.cpu().numpy(), x_blk.cpu().numpy()
    np.testing.assert_array_equal(xt, x_fused.cpu().numpy())  # the fused kernel is assembly + this solve
    x64 = np.linalg.solve(Hd64, b.grad.astype(np.float64)[:, :, None])[:, :, 0]
    cond = np.linalg.cond(Hd64)
    norm = np.linalg.norm(x64, axis=1)
    for name, x in (("tree", xt), ("blocked", xb)):
        err = np.linalg.norm(x - x64, axis=1) / norm
        assert (err / (cond * 6e-8)).max() < 1.0, name
    assert (np.linalg.norm(xt - xb, axis=1) / norm / (cond * 6e-8)).max() < 1.0
    # the factor of the blocked path reproduces H
    U = blocked.U.cpu().numpy().astype(np.float64)[:64]
    np.testing.assert_allclose(np.einsum("wki,wkj->wij", U, U)[:, :nv, :nv], Hd64[:64], rtol=2e-5, atol=2e-5 * np.abs(Hd64[:64]).max())


def test_snu_muscle_terms_into_the_fused_solve(device):
    """Configuration 4: nv = 56, 284 muscles, 4096 worlds, nefc = 128.  The implicit term
    h A' diag(s) A goes into M's CSR (im_muscle_implicit_gather), tau = A'f into the right-hand
    side (im_muscle_project), then the fused assemble + tree L'DL + solve: bit for bit the oracle's
    chain of the same three steps, every world."""
    import torch

    from instantmimic_amd.mjw_kernels import tree_ldl as T
    from instantmimic_amd.muscle import muscle_qfrc_projector as MQ

    b = synth.make_batch("snu")
    nworld, nv = b.nworld, b.shape.nv
    assert nworld == 4096 and nv == 56 and b.shape.nefc == 128
    mb = synth.make_muscles(nworld)
    st = (b.rowadr, b.rownnz, b.colind)
    ent = MQ.entries_from_muscle_dofs(mb.muscle_dofs, mb.nmuscle)
    offsets, order = MQ.torque_sorted_entries(ent.muscle_dof_torque_idx, nv - mb.root_dof_count)
    prepared = MQ.prepare_muscle_implicit_qderiv_pairs(
        pair_entry_i=ent.pair_entry_i, pair_entry_j=ent.pair_entry_j, pair_muscle_idx=ent.pair_muscle_idx,
        muscle_dof_torque_idx=ent.muscle_dof_torque_idx, matrix_elemid=synth.matrix_elemid(b.rowadr, b.rownnz, b.colind),
        root_dof_count=mb.root_dof_count,
    )  # fmt: skip
    assert prepared.dropped_pair_count == 0
    gather = MQ.build_muscle_implicit_qderiv_gather(prepared, ent.muscle_dof_muscle_idx, device)
    Mq = _t(b.M, device)  # receives h A'sA on top of M
    MQ.apply_muscle_implicit_qderiv_gather(gather, _t(mb.moment, device), _t(mb.slope, device), mb.timestep, Mq)
    tau = torch.zeros((nworld, nv), device=device)
    MQ.project_muscle_sparse_moment_qfrc(
        _t(mb.moment, device), _t(mb.force, device), _t(offsets.astype(np.int32), device), _t(order.astype(np.int32), device),
        _t(ent.muscle_dof_muscle_idx.astype(np.int32), device), mb.root_dof_count, tau,
    )  # fmt: skip
    rhs = _t(b.grad, device) - tau
    scratch = T.create_tree_factor_solve_scratch(_model(b), device)
    x = torch.zeros((nworld, nv), device=device)
    T.assemble_tree_factor_solve(scratch, Mq, _t(b.J, device), _t(b.D, device), _t(b.state[0], device), _t(b.nefc, device), rhs, x)
    torch.cuda.synchronize()
    # the oracle's chain
    tables = MQ.gather_tables(prepared, ent.muscle_dof_muscle_idx)
    Mq_ref = R.muscle_implicit_gather(mb.moment, mb.slope, ent.muscle_dof_muscle_idx, tables[0], tables[1], tables[2], tables[4], mb.timestep, b.M)
    tau_ref = R.muscle_project(mb.moment, mb.force, offsets, order, ent.muscle_dof_muscle_idx, mb.root_dof_count, nv)
    np.testing.assert_array_equal(Mq.cpu().numpy(), Mq_ref)
    np.testing.assert_array_equal(tau.cpu().numpy(), tau_ref)
    assert np.abs(Mq_ref - b.M).max() > 0 and np.abs(tau_ref).max() > 0
    x_ref = R.assemble_tree_ldl_solve(*st, P.best_tree_ldl_plan(*st), Mq_ref, b.J, b.D, b.state[0], b.nefc, b.grad - tau_ref)
    np.testing.assert_array_equal(x.cpu().numpy(), x_ref)


def test_stress_three_newton_iterations_at_the_full_batch(device):
    """Configuration 5: nv = 128, nefc = 256, 16384 worlds, three iterations with a fresh active
    mask each: J'DJ on the matrix cores, then twice the per-iteration stage (incremental update
    over the rows whose state flipped -- about half of them --, augmented blocked Cholesky with
    16 x 16 tiles, solve).  1024 source worlds are checked against the oracle; the full batch
    draws from them with repetition and every copy must equal its source bit for bit."""
    import dataclasses

    import torch

    from instantmimic_amd.mjw_kernels import blocked_dense as BD
    from instantmimic_amd.mjw_kernels import newton_fusion as NF
    from instantmimic_amd.mjw_kernels import newton_stages as NS

    nsrc, nworld = 1024, 16384
    shape = synth.SHAPES["stress"]
    b = synth.make_batch(dataclasses.replace(shape, iterations=3), nsrc)
    nv, njmax = shape.nv, shape.nefc
    pad = ((nv + 1 + 15) // 16) * 16
    Md = synth.dense_from_csr(b.M.astype(np.float64), b.rowadr, b.rownnz, b.colind).astype(np.float32)
    rng = np.random.default_rng(5)
    grads = rng.standard_normal((3, nsrc, nv)).astype(np.float32)
    perm_np = rng.integers(0, nsrc, nworld)
    perm_np[:nsrc] = np.arange(nsrc)  # every source world occurs, first
    perm = _t(perm_np, device)
    take = lambda a: _t(a, device).index_select(0, perm).contiguous()  # noqa: E731
    J, D, N = take(b.J), take(b.D), take(b.nefc)
    states = [take(b.state[it]) for it in range(3)]
    H = torch.zeros((nworld, pad, pad), device=device)
    BD.dense_hessian(take(Md), J, D, states[0], N, H)
    torch.cuda.synchronize()
    H0 = H[:nsrc].cpu().numpy()
    assert torch.equal(H, H[:nsrc].index_select(0, perm))
    assert R.rel_l2(H0, R.jtdj_dense(Md.reshape(nsrc, -1), b.J, b.D, b.state[0], b.nefc, pad)) <= 1e-5
    U = torch.zeros((nworld, pad, pad), device=device)
    uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=device)
    search = torch.zeros((nworld, pad, 1), device=device)
    sdot, decr = torch.zeros(nworld, device=device), torch.zeros(nworld, device=device)
    ids = torch.zeros((nworld, njmax), dtype=torch.int32, device=device)
    qcount = torch.zeros(nworld, dtype=torch.int32, device=device)
    scount = torch.zeros(nworld, dtype=torch.int32, device=device)
    done = torch.zeros(nworld, dtype=torch.uint8, device=device)
    stage = NS.factor_factory(nv, pad)
    H_ref, U_ref = H0, np.zeros_like(H0)
    for it in (1, 2):
        # the rows whose quadratic state flipped, listed on the GPU as the line search would
        NF.changed_rows(states[it - 1], states[it], ids, qcount, scount, nefc=N)
        g3 = torch.zeros((nworld, pad, 1), device=device)
        g3[:, :nv, 0] = take(grads[it])
        stage(J, D, states[it], ids, qcount, scount, done, g3, H, U, search, sdot, decr, uni)
        torch.cuda.synchronize()
        ids_h, qc_h, sc_h = ids[:nsrc].cpu().numpy(), qcount[:nsrc].cpu().numpy(), scount[:nsrc].cpu().numpy()
        assert 100 < qc_h.mean() < 156  # about half of the 256 rows change
        want = R.dense_update_factor(sc_h, qc_h, ids_h, b.J, b.D, b.state[it], grads[it], H_ref, U_ref, done=np.zeros(nsrc, np.uint8))
        np.testing.assert_array_equal(H[:nsrc].cpu().numpy(), want[0])
        np.testing.assert_array_equal(U[:nsrc].cpu().numpy(), want[1])
        np.testing.assert_array_equal(search[:nsrc, :nv, 0].cpu().numpy(), want[3])
        np.testing.assert_array_equal(decr[:nsrc].cpu().numpy(), want[5])
        for full, name in ((H, "H"), (U, "U"), (search, "search"), (sdot, "search_dot")):
            assert torch.equal(full, full[:nsrc].index_select(0, perm)), name
        H_ref, U_ref = want[0], want[1]
        # the updated Hessian is the fresh assembly with the new states (to fp32 rounding of the larger H)
        fresh = R.assemble_dense64(b.rowadr, b.rownnz, b.colind, b.M, b.J, b.D, b.state[it], b.nefc)[:32]
        got = np.triu(want[0][:32, :nv, :nv].astype(np.float64))
        assert np.abs(got - np.triu(fresh)).max() / np.abs(fresh).max() < 2e-5


def test_rows_outside_the_tree_pattern_are_counted(device):
    """A constraint row over two branches has products outside M's pattern, which the fused tree
    solve drops; im_tree_pattern_violations counts such rows per world and accumulates
    (reference: tests/test_mjw_sparse_hessian.py:426-452)."""
    import torch

    from instantmimic_amd.mjw_kernels import tree_ldl as T

    b = synth.make_batch("humanoid", 200, ragged_nefc=True)
    scratch = T.create_tree_factor_solve_scratch(_model(b), device)
    J, D, S, N = b.J.copy(), b.D.copy(), b.state[0].copy(), b.nefc.copy()
    N[[5, 7, 8, 9]] = np.maximum(N[[5, 7, 8, 9]], 8)
    N[11] = min(N[11], 60)
    # rows of the generator lie on one chain each: nothing to count
    count = torch.zeros(200, device=device)
    T.pattern_violations(scratch, _t(J, device), _t(D, device), _t(S, device), _t(N, device), count)
    torch.cuda.synchronize()
    assert float(count.abs().max()) == 0.0
    # humanoid: right leg 9..14 and left leg 15..20 hang off dof 8, the arms 21..23 and 24..26 off dof 5
    for w, r, dofs, state, d in (
        (5, 0, (9, 15), Q, 2.0e3), (5, 1, (14, 21), Q, 1.0e3), (5, 2, (20, 26), Q, 3.0e3),  # world 5: three rows over two limbs
        (7, 3, (9, 15), 0, 2.0),  # not quadratic: does not count
        (8, 4, (9, 15), Q, 0.0),  # zero weight: does not count
        (9, 1, (3, 9, 14), Q, 1.0),  # one chain: fine
        (11, int(N[11]), (9, 15), Q, 1.0),  # at nefc: ignored
    ):  # fmt: skip
        J[w, r, :] = 0.0
        J[w, r, list(dofs)] = 1.5
        S[w, r], D[w, r] = state, d
    want = np.zeros(200, np.float32)
    want[5] = 3.0
    for _ in range(2):  # the counter accumulates
        T.pattern_violations(scratch, _t(J, device), _t(D, device), _t(S, device), _t(N, device), count)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(count.cpu().numpy(), 2 * want)
    # what the count warns about: the fused solve drops the products outside M's pattern (as the oracle does),
    # so world 5 no longer solves its dense H while every other world does, to within cond(H) eps
    x = torch.zeros((200, 27), device=device)
    T.assemble_tree_factor_solve(scratch, _t(b.M, device), _t(J, device), _t(D, device), _t(S, device), _t(N, device), _t(b.grad, device), x)
    torch.cuda.synchronize()
    st = (b.rowadr, b.rownnz, b.colind)
    xh = x.cpu().numpy()
    np.testing.assert_array_equal(xh, R.assemble_tree_ldl_solve(*st, P.best_tree_ldl_plan(*st), b.M, J, D, S, N, b.grad))
    H64 = R.assemble_dense64(*st, b.M, J, D, S, N)
    x64 = np.linalg.solve(H64, b.grad.astype(np.float64)[:, :, None])[:, :, 0]
    err = np.linalg.norm(xh - x64, axis=1) / np.linalg.norm(x64, axis=1)
    assert err[5] > 0.5
    assert (np.delete(err, 5) / (np.delete(np.linalg.cond(H64), 5) * 6e-8)).max() < 1.0
