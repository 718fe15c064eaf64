"""GPU parity of the fused assemble + tree L'DL + solve path, through the C ABI.

Bar: the HIP kernels perform the oracle's IEEE operations in the oracle's order, so
H and x are compared bit for bit; the 1e-5 relative-L2 bound of the contract follows
(asserted as well).  Elimination order and plan arrays are compared exactly."""

import os

import numpy as np
import pytest

from instantmimic_amd import synth
from oracle import planner as P
from oracle import ref as R

pytestmark = pytest.mark.gpu

TOL = 1e-5  # relative L2, fp32 (the contract's bound)
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _model(b):
    return type("m", (), dict(nv=b.shape.nv, M_rowadr=b.rowadr, M_rownnz=b.rownnz, M_colind=b.colind))


def _run_fused(T, scratch, b, it, device, nefc=True, negate=False, want_h=True):
    import torch

    tM, tJ, tD, tS, tN, tG = (torch.from_numpy(np.ascontiguousarray(a)).to(device) for a in (b.M, b.J, b.D, b.state[it], b.nefc, b.grad))
    x = torch.full_like(tG, float("nan"))
    H = torch.full_like(tM, float("nan")) if want_h else None
    T.assemble_tree_factor_solve(scratch, tM, tJ, tD, tS, tN if nefc else None, tG, x, H_out=H, negate=negate)
    torch.cuda.synchronize()
    return x.cpu().numpy(), (H.cpu().numpy() if want_h else None)


@pytest.mark.parametrize("kernel", ["auto", "generic"])
@pytest.mark.parametrize("ragged", [True, False])
@pytest.mark.parametrize("name,nworld", [("ant", 64), ("humanoid", 333), ("g1", 257), ("snu", 129)])
def test_fused_matches_oracle_bitwise(device, monkeypatch, name, nworld, ragged, kernel):
    """Both device kernels: the one generated for the tree ("auto" picks it for the
    benchmark trees) and the table-driven one that serves any tree."""
    from instantmimic_amd.mjw_kernels import tree_ldl as T

    monkeypatch.setenv("IMHIP_TREE_KERNEL", kernel)
    b = synth.make_batch(name, nworld, ragged_nefc=ragged)
    scratch = T.create_tree_factor_solve_scratch(_model(b), device)
    assert scratch is not None
    st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    plan = P.best_tree_ldl_plan(*st)
    # integer side: plan and elimination order
    assert scratch.plan.groups == plan.groups and scratch.plan.trunk == plan.trunk
    assert list(T.elimination_order(scratch.plan)) == P.elimination_order(plan)
    for it in range(b.state.shape[0]):
        x_ref, H_ref = R.assemble_tree_ldl_solve(*st, plan, b.M, b.J, b.D, b.state[it], b.nefc, b.grad, want_h=True)
        x, H = _run_fused(T, scratch, b, it, device)
        assert R.rel_l2(H, H_ref) <= TOL and R.rel_l2(x, x_ref) <= TOL
        np.testing.assert_array_equal(H, H_ref)
        np.testing.assert_array_equal(x, x_ref)
    # factor + solve alone on the assembled matrix
    import torch

    xs = torch.full((nworld, b.shape.nv), float("nan"), device=device)
    T.tree_factor_solve(scratch, torch.from_numpy(H_ref).to(device), xs, torch.from_numpy(b.grad).to(device))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(xs.cpu().numpy(), R.tree_ldl_solve(*st, plan, H_ref, b.grad))


def test_fused_full_humanoid_batch(device):
    """The benchmark shape at its full size: 4096 worlds, three Newton iterations."""
    from instantmimic_amd.mjw_kernels import tree_ldl as T

    b = synth.make_batch("humanoid")
    assert b.nworld == 4096 and b.state.shape[0] == 3
    scratch = T.create_tree_factor_solve_scratch(_model(b), device)
    st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    plan = P.best_tree_ldl_plan(*st)
    for it in range(3):
        x_ref = R.assemble_tree_ldl_solve(*st, plan, b.M, b.J, b.D, b.state[it], b.nefc, b.grad)
        x, H = _run_fused(T, scratch, b, it, device)
        np.testing.assert_array_equal(x, x_ref)
        # size-independent property: small backward error of H x = g
        Hd = R.dense_from_csr(H.astype(np.float64), *st)
        res = np.einsum("wij,wj->wi", Hd, x.astype(np.float64)) - b.grad
        scale = np.linalg.norm(Hd, axis=(1, 2)) * np.linalg.norm(x, axis=1) + np.linalg.norm(b.grad, axis=1)
        assert (np.linalg.norm(res, axis=1) / scale).max() < 2e-6


@pytest.mark.parametrize("name,nworld,ragged", [("humanoid", 4096, True), ("humanoid", 333, False), ("ant", 67, True), ("g1", 130, True)])
def test_fused_without_h_output_bitwise(device, name, nworld, ragged):
    """The fused entry without its optional H output (what the benchmark launches): x must be the
    oracle's bit for bit, with and without the per-world row counts and with the negated result."""
    from instantmimic_amd.mjw_kernels import tree_ldl as T

    b = synth.make_batch(name, nworld, ragged_nefc=ragged)
    scratch = T.create_tree_factor_solve_scratch(_model(b), device)
    st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    plan = P.best_tree_ldl_plan(*st)
    for it in range(b.state.shape[0]):
        x_ref = R.assemble_tree_ldl_solve(*st, plan, b.M, b.J, b.D, b.state[it], b.nefc, b.grad)
        x, _ = _run_fused(T, scratch, b, it, device, want_h=False)
        np.testing.assert_array_equal(x, x_ref)
    xn, _ = _run_fused(T, scratch, b, 0, device, want_h=False, negate=True)
    np.testing.assert_array_equal(xn, -R.assemble_tree_ldl_solve(*st, plan, b.M, b.J, b.D, b.state[0], b.nefc, b.grad))
    full = np.full_like(b.nefc, b.J.shape[1])
    x_all = R.assemble_tree_ldl_solve(*st, plan, b.M, b.J, b.D, b.state[0], full, b.grad)
    xa, _ = _run_fused(T, scratch, b, 0, device, nefc=False, want_h=False)
    np.testing.assert_array_equal(xa, x_all)


def test_stored_vectors(device):
    from instantmimic_amd.mjw_kernels import tree_ldl as T

    z = np.load(os.path.join(GOLDEN, "tree_small.npz"))
    b = synth.make_batch("ant", 4)
    b.M, b.J, b.D, b.grad, b.nefc = z["M"], z["J"], z["D"], z["grad"], z["nefc"]
    b.state = z["state"][None]
    scratch = T.create_tree_factor_solve_scratch(_model(b), device)
    x, H = _run_fused(T, scratch, b, 0, device)
    np.testing.assert_array_equal(H, z["H"])
    np.testing.assert_array_equal(x, z["x"])


@pytest.mark.parametrize("tree", ["branched", "limbs"])
@pytest.mark.parametrize("groups", [1, 2, 4])
def test_tree_factor_solve_matches_a_dense_solve(device, tree, groups):
    # reference: tests/test_tree_ldl.py:99-120 (37 worlds, groups 1/2/4, rtol 2e-4, atol 2e-5)
    import torch

    from instantmimic_amd.mjw_kernels import tree_ldl as T

    parent = synth.branched_parents() if tree == "branched" else synth.limbs_parents()
    rng = np.random.default_rng(0)
    nv, worlds = len(parent), 37
    mask = synth.chain_mask(parent)
    V = rng.standard_normal((worlds, nv, nv)) * mask[None]
    dense = np.einsum("wki,wkj->wij", V, V) + np.eye(nv) * (2.0 + rng.uniform(0, 0.2, (worlds, nv, 1)))
    rowadr, rownnz, colind = synth.csr_from_parents(parent)
    sparse = np.ascontiguousarray(dense[:, np.repeat(np.arange(nv), rownnz), colind], dtype=np.float32)
    st = T.tree_ldl_structure(rowadr, rownnz, colind)
    plan = T.plan_tree_ldl(*st, groups)
    scratch = T.scratch_for_plan(st, plan, device)
    y = np.random.default_rng(1).normal(size=(worlds, nv)).astype(np.float32)
    x = torch.zeros((worlds, nv), dtype=torch.float32, device=device)
    T.tree_factor_solve(scratch, torch.from_numpy(sparse).to(device), x, torch.from_numpy(y).to(device))
    torch.cuda.synchronize()
    expected = R.solve64(R.dense_from_csr(sparse.astype(np.float64), *st), y)
    np.testing.assert_allclose(x.cpu().numpy(), expected, rtol=2e-4, atol=2e-5)
    oplan = P.plan_tree_ldl(*st, groups)
    np.testing.assert_array_equal(x.cpu().numpy(), R.tree_ldl_solve(*st, oplan, sparse, y))


def test_edge_cases(device):
    import torch

    from instantmimic_amd.mjw_kernels import tree_ldl as T

    b = synth.make_batch("humanoid", 5)
    scratch = T.create_tree_factor_solve_scratch(_model(b), device)
    st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    plan = P.best_tree_ldl_plan(*st)
    # no constraint rows at all: H == M
    b0 = synth.make_batch("humanoid", 5)
    b0.nefc[:] = 0
    x, H = _run_fused(T, scratch, b0, 0, device)
    np.testing.assert_array_equal(H, b0.M)
    np.testing.assert_array_equal(x, R.tree_ldl_solve(*st, plan, b0.M, b0.grad))
    # every row inactive
    b1 = synth.make_batch("humanoid", 5)
    b1.state[:] = 0
    x, H = _run_fused(T, scratch, b1, 0, device)
    np.testing.assert_array_equal(H, b1.M)
    # nefc omitted = all rows; negated output; one world
    b2 = synth.make_batch("humanoid", 1)
    x, _ = _run_fused(T, scratch, b2, 0, device, nefc=False, negate=True)
    np.testing.assert_array_equal(-x, R.assemble_tree_ldl_solve(*st, plan, b2.M, b2.J, b2.D, b2.state[0], None, b2.grad))
    # strided world rows (leading dimension larger than the row)
    wideM = torch.zeros((5, 300), device=device)
    wideM[:, :243] = torch.from_numpy(b.M).to(device)
    widex = torch.zeros((5, 40), device=device)
    T.tree_factor_solve(scratch, wideM[:, :243], widex[:, :27], torch.from_numpy(b.grad).to(device))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(widex[:, :27].cpu().numpy(), R.tree_ldl_solve(*st, plan, b.M, b.grad))
    assert float(widex[:, 27:].abs().max()) == 0.0
    # rows that are not contiguous floats are refused like the reference does
    # (tests/test_tree_ldl.py:164-175)
    wide = torch.zeros((5, 54), device=device)
    with pytest.raises(ValueError, match="contiguous"):
        T.tree_factor_solve(scratch, torch.from_numpy(b.M).to(device), wide[:, ::2], wide[:, ::2])
    # empty batch
    e = torch.zeros((0, 27), device=device)
    T.tree_factor_solve(scratch, torch.zeros((0, 243), device=device), e, e)


def test_ineligible_models_return_none(device):
    from instantmimic_amd.mjw_kernels import tree_ldl as T

    rowadr, rownnz, colind = synth.csr_from_parents(synth.chain_parents(30))
    m = type("m", (), dict(nv=len(rowadr), M_rowadr=rowadr, M_rownnz=rownnz, M_colind=colind))
    assert T.create_tree_factor_solve_scratch(m, device) is None
    assert T.create_tree_factor_solve_scratch(type("m", (), dict(nv=0)), device) is None


@pytest.mark.parametrize("name,nworld,niter,ragged,per_iter_grad", [
    ("humanoid", 4096, 3, False, False), ("humanoid", 333, 5, True, True), ("ant", 65, 3, True, False),
    ("g1", 257, 3, True, True), ("snu", 130, 2, True, False), ("humanoid", 7, 1, True, False),
])  # fmt: skip
def test_iterations_in_one_call_match_the_oracle_bitwise(device, name, nworld, niter, ragged, per_iter_grad):
    """im_assemble_tree_ldl_solve_iters: the iterations of a step share M, J and D; every iteration
    assembles afresh, so each equals the single call (and the oracle) bit for bit -- on the
    straight-line kernel (humanoid, ant: up to 64 rows) and on the variant that loops over the
    listed constraint rows (g1: 96 rows, snu: 128 rows); both cover (worlds, iteration) with one grid."""
    import torch

    from instantmimic_amd.mjw_kernels import tree_ldl as T

    b = synth.make_batch(name, nworld, ragged_nefc=ragged)
    rng = np.random.default_rng(3)
    states = np.stack([np.where(rng.random(b.state[0].shape) < 0.6, synth.QUADRATIC, 0).astype(np.int32) for _ in range(niter)])
    grads = rng.normal(size=(niter, nworld, b.shape.nv)).astype(np.float32) if per_iter_grad else b.grad
    scratch = T.create_tree_factor_solve_scratch(_model(b), device)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    x = torch.full((niter, nworld, b.shape.nv), float("nan"), device=device)
    T.assemble_tree_factor_solve_iters(scratch, t(b.M), t(b.J), t(b.D), t(states), t(b.nefc), t(grads), x, negate=True)
    torch.cuda.synchronize()
    st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    plan = P.best_tree_ldl_plan(*st)
    for it in range(niter):
        g = grads[it] if per_iter_grad else grads
        x_ref = R.assemble_tree_ldl_solve(*st, plan, b.M, b.J, b.D, states[it], b.nefc, g)
        np.testing.assert_array_equal(x[it].cpu().numpy(), -x_ref, err_msg=f"iteration {it}")


def test_short_reciprocal_equals_the_division_for_every_float_in_its_range(device):
    """The pivot chain of the generated kernels replaces 1.0f / x by the hardware estimate and one
    exact-residual correction inside 2^-101 <= |x| < 2^102: all 3.4e9 such floats, both signs."""
    import torch

    from instantmimic_amd import _lib

    count = torch.zeros(1, dtype=torch.int64, device=device)
    stream = int(torch.cuda.current_stream(device).cuda_stream)
    assert _lib.lib().im_check_reciprocal(0, 0xFFFFFFFF, count.data_ptr(), stream) == _lib.IM_OK
    torch.cuda.synchronize()
    assert int(count.item()) == 0
