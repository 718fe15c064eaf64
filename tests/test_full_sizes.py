"""The configured shapes at their full batch sizes on the GPU.

g1 (8192 worlds) and snu (4096 worlds) through the fused assemble + tree L'DL + solve: every
world against the oracle bit for bit, plus the backward error of H x = g.  stress (nv 128,
nefc 256, 16384 worlds) through the dense J'DJ and the blocked Cholesky: worlds are independent,
so a world's result must not depend on where it sits in a batch -- the 16384 worlds are 1024
distinct ones drawn with repetition, every copy must equal its source bit for bit, and the 1024
sources are checked against the oracle."""

import dataclasses
from types import SimpleNamespace

import numpy as np
import pytest

from instantmimic_amd import synth
from oracle import planner as P
from oracle import ref as R

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,nworld", [("g1", 8192), ("snu", 4096)])
def test_fused_tree_full_batch(device, name, nworld):
    import torch

    from instantmimic_amd.mjw_kernels import tree_ldl as T

    b = synth.make_batch(name)
    assert b.nworld == nworld
    model = SimpleNamespace(nv=b.shape.nv, M_rowadr=b.rowadr, M_rownnz=b.rownnz, M_colind=b.colind)
    scratch = T.create_tree_factor_solve_scratch(model, device)
    st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    plan = P.best_tree_ldl_plan(*st)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    tM, tJ, tD, tN, tG = t(b.M), t(b.J), t(b.D), t(b.nefc), t(b.grad)
    for it in range(b.state.shape[0]):
        x, H = torch.full_like(tG, float("nan")), torch.full_like(tM, float("nan"))
        T.assemble_tree_factor_solve(scratch, tM, tJ, tD, t(b.state[it]), tN, tG, x, H_out=H)
        torch.cuda.synchronize()
        x, H = x.cpu().numpy(), H.cpu().numpy()
        np.testing.assert_array_equal(x, R.assemble_tree_ldl_solve(*st, plan, b.M, b.J, b.D, b.state[it], b.nefc, b.grad))
        Hd = R.dense_from_csr(H.astype(np.float64), *st)
        res = np.einsum("wij,wj->wi", Hd, x.astype(np.float64)) - b.grad
        scale = np.linalg.norm(Hd, axis=(1, 2)) * np.linalg.norm(x, axis=1) + np.linalg.norm(b.grad, axis=1)
        assert (np.linalg.norm(res, axis=1) / scale).max() < 2e-6


def test_stress_full_batch_by_world_independence(device):
    import torch

    from instantmimic_amd.mjw_kernels import blocked_dense as BD

    nsrc, nworld = 1024, 16384
    b = synth.make_batch("stress", nsrc)
    nv = b.shape.nv
    nv_pad = ((nv + 1 + 15) // 16) * 16
    Md = synth.dense_from_csr(b.M.astype(np.float64), b.rowadr, b.rownnz, b.colind).astype(np.float32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    src = [t(a) for a in (Md, b.J, b.D, b.state[0], b.nefc, b.grad)]
    perm = torch.from_numpy(np.random.default_rng(77).integers(0, nsrc, nworld)).to(device)
    full = [a.index_select(0, perm).contiguous() for a in src]

    def hessian(args, n):
        H = torch.zeros((n, nv_pad, nv_pad), device=device)
        BD.dense_hessian(*args[:5], H)
        return H

    Hs, Hf = hessian(src, nsrc), hessian(full, nworld)
    torch.cuda.synchronize()
    assert torch.equal(Hf, Hs.index_select(0, perm))
    assert torch.equal(Hs, Hs.transpose(1, 2))
    Hh = Hs.cpu().numpy()
    # the matrix cores sum in their own order: tolerance parity (1e-5 relative L2, fp32)
    assert R.rel_l2(Hh, R.jtdj_dense(Md.reshape(nsrc, -1), b.J, b.D, b.state[0], b.nefc, nv_pad)) <= 1e-5
    assert R.rel_l2(Hh[:, :nv, :nv], R.assemble_dense64(b.rowadr, b.rownnz, b.colind, b.M, b.J, b.D, b.state[0], b.nefc)) <= 1e-5

    # blocked Cholesky of those Hessians (B = 16), factor stored
    m = SimpleNamespace(nv=nv, M_tiles=[SimpleNamespace(size=nv, elemid=np.arange(nv * nv))])

    def solve(H, g, n):
        Hc = H[:, :nv, :nv].contiguous().reshape(n, -1)
        d = SimpleNamespace(nworld=n, M=Hc)
        scratch = BD.create_blocked_dense_factor_solve_scratch(m, d, device, block_size=16)
        x = torch.full((n, nv, 1), float("nan"), device=device)
        BD._blocked_dense_factor_solve(d, Hc, x, g.reshape(n, nv, 1), scratch)
        return x, scratch

    xs, ss = solve(Hs, src[5], nsrc)
    xf, sf = solve(Hf, full[5], nworld)
    torch.cuda.synchronize()
    assert torch.equal(xf, xs.index_select(0, perm))
    assert torch.equal(sf.U, ss.U.index_select(0, perm))
    H32 = np.ascontiguousarray(Hh[:, :nv, :nv].reshape(nsrc, -1))
    x_ref, U_ref = R.blocked_factor_solve(H32, ss.indices.cpu().numpy(), nv, ss.pad, 16, b.grad)
    np.testing.assert_array_equal(xs.cpu().numpy()[:, :, 0], x_ref)
    np.testing.assert_array_equal(ss.U.cpu().numpy(), U_ref)
    # U' U == H to the rounding of a 128-term sum, on the GPU in fp64 for every one of the 16384
    Uf = sf.U.double()
    back = torch.matmul(Uf.transpose(1, 2), Uf)[:, :nv, :nv]
    Hd = Hf[:, :nv, :nv].double()
    err = (back - Hd).flatten(1).norm(dim=1) / Hd.flatten(1).norm(dim=1)
    assert float(err.max()) < 2e-6


@pytest.mark.parametrize("name,nworld", [("g1", 8192), ("snu", 4096)])
def test_sparse_factor_full_batch(device, name, nworld):
    """Static-pattern sparse L'DL at the full batch: the initial assemble + factor + solve, then
    one per-iteration stage (changed rows, refactor or solve-only), every world bit for bit."""
    import torch

    from instantmimic_amd.mjw_kernels import newton_stages as NS
    from instantmimic_amd.mjw_kernels import sparse_hessian as S
    from test_newton_stages import _changes

    m = synth.model_from_parents(synth.SHAPES[name].parents)
    plan, reason = S.plan_for_model(m, None, [], S.block_width(m.nv_pad), device=device)
    assert plan is not None, reason
    oplan = R.sparse_plan(m, [], plan.block)
    b = synth.make_batch(dataclasses.replace(synth.SHAPES[name], iterations=2))  # a second state to move to
    assert b.nworld == nworld
    nv = m.nv
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    hf = torch.zeros((nworld, plan.nv_pad, plan.nv_pad), device=device)
    search = torch.full((nworld, nv, 1), float("nan"), device=device)
    sdot, decr = torch.zeros(nworld, device=device), torch.zeros(nworld, device=device)
    tJ, tD = t(b.J), t(b.D)
    S.init_factor_kernel(plan)(None, t(b.nefc), tJ, tD, t(b.state[0]), t(b.M), t(b.grad)[:, :, None].contiguous(), hf, search, sdot, decr)
    torch.cuda.synchronize()
    ref = R.sparse_init_factor(oplan, b.nefc, b.J, b.D, b.state[0], b.M, b.grad)
    n_used = 2 * plan.nfac + nv
    np.testing.assert_array_equal(hf.cpu().numpy().reshape(nworld, -1)[:, :n_used], ref[0].reshape(nworld, -1)[:, :n_used])
    np.testing.assert_array_equal(search.cpu().numpy()[:, :, 0], ref[1])
    np.testing.assert_array_equal(sdot.cpu().numpy(), ref[2])
    np.testing.assert_array_equal(decr.cpu().numpy(), ref[3])
    assert not hf[:, -1, -1].any()  # nothing fell outside the declared pattern
    # the per-iteration stage from there
    new, ids, changes, sc, done, grad = _changes(b, np.random.default_rng(5))
    want = R.sparse_update_factor(oplan, sc, changes, ids, b.J, b.D, new, grad, ref[0], done=done)
    uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=device)
    search2 = torch.zeros((nworld, nv), device=device)
    NS.factor_factory(nv, m.nv_pad, plan)(tJ, tD, t(new), t(ids), t(changes), t(sc), t(done), t(grad), None, hf, search2, sdot, decr, uni)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(hf.cpu().numpy().reshape(nworld, -1)[:, :n_used], want[0].reshape(nworld, -1)[:, :n_used])
    live = (sc != 0) & (done == 0)
    np.testing.assert_array_equal(uni.cpu().numpy()[live & (changes > 0)], want[1][live & (changes > 0)])
    np.testing.assert_array_equal(search2.cpu().numpy()[live], want[2][live])
    np.testing.assert_array_equal(sdot.cpu().numpy()[live], want[3][live])
    np.testing.assert_array_equal(decr.cpu().numpy()[live], want[4][live])
