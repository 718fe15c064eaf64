"""Factor step of the upstream (non-fused) Newton iteration on the static pattern: the slots of
the factor gathered from the dense Hessian, refactor or solve with the stored factor per world
(reference: src/instantmimic/utils/mjw_kernels/sparse_hessian.py:639-679, 849-894)."""

import numpy as np
import pytest

from instantmimic_amd import synth
from instantmimic_amd.mjw_kernels import sparse_hessian as S
from oracle import ref as R

Q = synth.QUADRATIC
CASES = {"limbs84": (tuple(synth.limbs_parents(6, 13)), 64), "stress": (synth.SHAPES["stress"].parents, 128)}


def _case(name, nworld, seed=11):
    """A model the fused Newton does not take, its plan inputs, and dense Hessians M + J'DJ whose
    rows stay on one chain each (so H lies inside the tree pattern)."""
    parents, block = CASES[name]
    m = synth.model_from_parents(parents)
    shape = synth.Shape(name, tuple(parents), 48, nworld, (0.5, 8.0), 0.02, (-3.0, 3.0), 0.6, 2, seed)
    b = synth.make_batch(shape, nworld)
    Md = synth.dense_from_csr(b.M, b.rowadr, b.rownnz, b.colind).astype(np.float32)
    H = [R.jtdj_dense(Md.reshape(nworld, -1), b.J, b.D, b.state[it], b.nefc, m.nv_pad) for it in range(2)]
    return m, block, b, H


def _ctx(m, nworld):
    return type("c", (), dict(hfactor=np.zeros((nworld, m.nv_pad, m.nv_pad), np.float32)))()


@pytest.mark.parametrize("name", list(CASES))
def test_oracle_against_fp64(name):
    nworld = 12
    m, block, b, H = _case(name, nworld)
    plan, reason = S.plan_for_model(m, _ctx(m, nworld), [], 64, device=None)
    assert reason == "enabled" and plan.path == "nonfused" and plan.block == block
    oplan = R.sparse_plan(m, [], block, "nonfused")
    nv = m.nv
    assert S.pattern_misses(H[0], S.hessian_pattern(m, [])) == 0
    rng = np.random.default_rng(2)
    g0, g1 = (rng.standard_normal((nworld, nv)).astype(np.float32) for _ in range(2))
    hf0 = np.zeros((nworld, m.nv_pad, m.nv_pad), np.float32)
    hf1, search, sdot, decr = R.sparse_dense_factor(oplan, g0, H[0], hf0)
    H64 = H[0][:, :nv, :nv].astype(np.float64)
    cond = np.linalg.cond(H64)
    x64 = np.linalg.solve(H64, g0.astype(np.float64)[:, :, None])[:, :, 0]
    err = np.linalg.norm(-search - x64, axis=1) / np.linalg.norm(x64, axis=1)
    assert (err / (cond * 6e-8)).max() < 2.0
    np.testing.assert_allclose(sdot, (x64 * x64).sum(1), rtol=2e-3 * max(1.0, (cond * 6e-8).max() * 1e3))
    np.testing.assert_allclose(decr, (g0 * x64).sum(1), rtol=1e-4, atol=1e-4 * np.abs((g0 * x64).sum(1)).max() + (cond * 6e-8).max())
    # the stored factor: N = L D on the slots and 1 / D behind them reproduce H on the pattern
    nfac = oplan.nfac
    flat = hf1.reshape(nworld, -1)
    assert (flat[:, nfac : nfac + nv] > 0).all() and (flat[:, nfac + nv :] == 0).all()
    # solve-only (mode 5) for the worlds whose QUADRATIC rows did not change, refactor from the
    # second Hessian for the others; worlds without any state change are left alone with skip_noflip
    quad_changed = np.array([0, 3] * (nworld // 2), np.int32)
    state_changed = np.array([1, 1, 0, 5] * (nworld // 4), np.int32)
    hf2, search2, _, _ = R.sparse_dense_factor(oplan, g1, H[1], hf1, quad_changed, state_changed, skip_unchanged=True, skip_noflip=True)
    for w in range(nworld):
        Hw = H[1] if quad_changed[w] else H[0]
        x = np.linalg.solve(Hw[w, :nv, :nv].astype(np.float64), g1[w].astype(np.float64))
        if state_changed[w] == 0:
            assert (search2[w] == 0).all() and np.array_equal(hf2[w], hf1[w])
            continue
        cw = np.linalg.cond(Hw[w, :nv, :nv].astype(np.float64))
        assert np.linalg.norm(-search2[w] - x) / np.linalg.norm(x) < 2.0 * cw * 6e-8, w
        assert np.array_equal(hf2[w], hf1[w]) == (quad_changed[w] == 0)
    # without skip_unchanged every live world refactors
    hf3, *_ = R.sparse_dense_factor(oplan, g1, H[1], hf1, quad_changed, state_changed, skip_unchanged=False, skip_noflip=False)
    assert not any(np.array_equal(hf3[w], hf1[w]) for w in range(nworld))


def test_kernel_factories_check_the_path():
    m, _ = synth.contact_model()
    plan = S.build_plan(m, [], 32, device=None)
    with pytest.raises(RuntimeError, match="no device state"):
        S.nonfused_kernel(plan, True, True)


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld", [("limbs84", 70), ("stress", 40)])
def test_gpu_matches_oracle_bitwise(device, name, nworld):
    import torch

    m, block, b, H = _case(name, nworld)
    plan, reason = S.plan_for_model(m, _ctx(m, nworld), [], 64, device=device)
    assert reason == "enabled" and plan.path == "nonfused" and plan.block == block and plan.handle is not None
    oplan = R.sparse_plan(m, [], block, "nonfused")
    with pytest.raises(ValueError, match="fused path only"):
        S.init_factor_kernel(plan)
    nv = m.nv
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    rng = np.random.default_rng(4)
    g0, g1 = (rng.standard_normal((nworld, nv)).astype(np.float32) for _ in range(2))
    done = np.zeros(nworld, np.uint8)
    done[3] = 1
    quad_changed = (rng.random(nworld) < 0.5).astype(np.int32) * 4
    state_changed = np.maximum(quad_changed, (rng.random(nworld) < 0.8).astype(np.int32))
    hf = torch.zeros((nworld, m.nv_pad, m.nv_pad), device=device)
    search = torch.full((nworld, nv, 1), 7.0, device=device)
    sdot, decr = torch.zeros(nworld, device=device), torch.zeros(nworld, device=device)
    ctx = type("c", (), dict(done=t(done), grad=t(g0), h=t(H[0]), quad_changed_count=t(quad_changed), state_changed_count=t(state_changed),
                            hfactor=hf, search=search.reshape(nworld, nv), search_dot=sdot, newton_decrement=decr))()  # fmt: skip
    solve = S.nonfused_solver_functions(plan)
    d = type("d", (), dict(nworld=nworld))()
    solve(m, d, ctx)  # every live world refactors
    torch.cuda.synchronize()
    want = R.sparse_dense_factor(oplan, g0, H[0], np.zeros((nworld, m.nv_pad, m.nv_pad), np.float32), done=done)
    live = done == 0
    np.testing.assert_array_equal(hf.cpu().numpy(), want[0])
    np.testing.assert_array_equal(search.cpu().numpy()[live, :, 0], want[1][live])
    assert (search.cpu().numpy()[~live] == 7.0).all()
    np.testing.assert_array_equal(sdot.cpu().numpy(), want[2])
    np.testing.assert_array_equal(decr.cpu().numpy(), want[3])
    # second iteration: new gradient and Hessian, refactor only where QUADRATIC rows changed
    ctx.grad, ctx.h = t(g1), t(H[1])
    solve(m, d, ctx, skip_unchanged=True, skip_noflip=True)
    torch.cuda.synchronize()
    want2 = R.sparse_dense_factor(oplan, g1, H[1], want[0], quad_changed, state_changed, skip_unchanged=True, skip_noflip=True, done=done)
    np.testing.assert_array_equal(hf.cpu().numpy(), want2[0])
    ran = live & (state_changed != 0)
    np.testing.assert_array_equal(search.cpu().numpy()[ran, :, 0], want2[1][ran])
    np.testing.assert_array_equal(search.cpu().numpy()[live & ~ran, :, 0], want[1][live & ~ran])
    np.testing.assert_array_equal(decr.cpu().numpy()[ran], want2[3][ran])
    # a plan of the fused path is refused by this entry point, and this plan by the fused ones
    fused_model, _ = synth.contact_model()
    fused = S.build_plan(fused_model, [], 32, device=device)
    with pytest.raises(ValueError, match="nonfused path"):
        S.nonfused_kernel(fused, False, False)
