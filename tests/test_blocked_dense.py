"""Blocked dense Cholesky factor + solve and the dense J'DJ Hessian."""

from types import SimpleNamespace

import numpy as np
import pytest
import scipy.linalg

from instantmimic_amd import synth
from instantmimic_amd.mjw_kernels import blocked_dense as BD
from oracle import ref as R


def _dense_model(name, nworld, seed=0, well=False):
    """M of a benchmark tree stored as one dense tile: values (nworld, nv * nv), elemid = identity."""
    b = synth.make_batch(name, nworld)
    nv = b.shape.nv
    Md = synth.dense_from_csr(b.M.astype(np.float64), b.rowadr, b.rownnz, b.colind)
    if well:
        Md = Md + 5.0 * np.eye(nv)
    return b, nv, Md


def test_layout_matches_the_reference_scratch():
    # reference: tests/test_blocked_dense_factor_solve.py:66-91 (nv 56: 64 * 64 indices, 8 identity pads)
    nv = 56
    pad, layout, identity = BD.block_index_layout(np.arange(nv * nv), nv, nv * nv, 16)
    assert pad == 64 and layout.shape == (64 * 64,)
    assert identity.reshape(16, 16).diagonal().sum() == 8 and identity.sum() == 8
    assert (layout == nv * nv).sum() == 64 * 64 - nv * nv
    # block (kb, ib) element (r, c) is M[kb * 16 + r, ib * 16 + c]
    blk = layout.reshape(4, 4, 16, 16)
    assert blk[1, 2, 3, 4] == (16 + 3) * nv + 32 + 4
    # gating
    m = SimpleNamespace(nv=20, M_tiles=[SimpleNamespace(size=20, elemid=np.arange(400))])
    assert BD.create_blocked_dense_factor_solve_scratch(m, SimpleNamespace(nworld=1, M=None)) is None


@pytest.mark.parametrize("name,B", [("g1", 8), ("g1", 16), ("snu", 16), ("stress", 16)])
def test_oracle_against_scipy(name, B):
    b, nv, Md = _dense_model(name, 6, well=True)
    pad, layout, _ = BD.block_index_layout(np.arange(nv * nv), nv, nv * nv, B)
    M32 = Md.reshape(6, -1).astype(np.float32)
    x, U = R.blocked_factor_solve(M32, layout, nv, pad, B, b.grad)
    for w in range(6):
        A = M32[w].reshape(nv, nv).astype(np.float64)
        c = scipy.linalg.cho_factor(A)
        np.testing.assert_allclose(x[w], scipy.linalg.cho_solve(c, b.grad[w].astype(np.float64)), rtol=2e-4, atol=2e-5)
        Uw = U[w].astype(np.float64)
        assert np.abs(np.tril(Uw, -1)).max() == 0.0
        np.testing.assert_allclose((Uw.T @ Uw)[:nv, :nv], A, rtol=1e-5, atol=1e-5)
        # padded rows factor to the identity
        np.testing.assert_array_equal(Uw[nv:, nv:], np.eye(pad - nv))
        np.testing.assert_allclose(np.triu(Uw[:nv, :nv]), np.triu(scipy.linalg.cholesky(A)), rtol=2e-4, atol=2e-5)


def test_dense_hessian_oracle_against_fp64():
    b, nv, Md = _dense_model("g1", 5)
    H = R.jtdj_dense(Md.reshape(5, -1), b.J, b.D, b.state[0], b.nefc, 48)
    H64 = R.assemble_dense64(b.rowadr, b.rownnz, b.colind, b.M, b.J, b.D, b.state[0], b.nefc)
    assert R.rel_l2(H[:, :nv, :nv], H64) < 1e-6
    assert np.abs(H[:, nv:, :]).max() == 0 and np.abs(H[:, :, nv:]).max() == 0


@pytest.mark.gpu
@pytest.mark.parametrize("name,B,nworld", [("g1", 8, 70), ("g1", 8, 3), ("snu", 8, 33), ("g1", 16, 70), ("g1", 16, 5), ("snu", 16, 33), ("stress", 16, 9)])
def test_gpu_blocked_factor_solve_bitwise(device, name, B, nworld):
    import torch

    b, nv, Md = _dense_model(name, nworld)
    M32 = np.ascontiguousarray(Md.reshape(nworld, -1).astype(np.float32))
    m = SimpleNamespace(nv=nv, M_tiles=[SimpleNamespace(size=nv, elemid=np.arange(nv * nv))])
    M = torch.from_numpy(M32).to(device)
    d = SimpleNamespace(nworld=nworld, M=M)
    scratch = BD.create_blocked_dense_factor_solve_scratch(m, d, device, block_size=B)
    assert scratch is not None and scratch.pad == -(-nv // B) * B
    y = torch.from_numpy(b.grad).to(device)
    x = torch.full_like(y, float("nan"))
    BD._blocked_dense_factor_solve(d, M, x.reshape(nworld, nv, 1), y.reshape(nworld, nv, 1), scratch)
    torch.cuda.synchronize()
    x_ref, U_ref = R.blocked_factor_solve(M32, scratch.indices.cpu().numpy(), nv, scratch.pad, B, b.grad)
    np.testing.assert_array_equal(scratch.U.cpu().numpy(), U_ref)
    np.testing.assert_array_equal(x.cpu().numpy(), x_ref)
    assert R.rel_l2(x.cpu().numpy(), x_ref) <= 1e-5
    # residual of the fp32 solve against the matrix
    res = np.einsum("wij,wj->wi", Md, x.cpu().numpy().astype(np.float64)) - b.grad
    scale = np.linalg.norm(Md, axis=(1, 2)) * np.linalg.norm(x_ref, axis=1) + np.linalg.norm(b.grad, axis=1)
    assert (np.linalg.norm(res, axis=1) / scale).max() < 5e-6


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld", [("ant", 50), ("humanoid", 50), ("g1", 40), ("snu", 30), ("stress", 24)])
def test_gpu_dense_hessian_mfma(device, name, nworld):
    import torch

    b = synth.make_batch(name, nworld, ragged_nefc=True)
    nv = b.shape.nv
    nv_pad = ((nv + 1 + 15) // 16) * 16
    Md = synth.dense_from_csr(b.M.astype(np.float64), b.rowadr, b.rownnz, b.colind).astype(np.float32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    H = torch.zeros((nworld, nv_pad, nv_pad), device=device)
    BD.dense_hessian(t(Md), t(b.J), t(b.D), t(b.state[0]), t(b.nefc), H)
    torch.cuda.synchronize()
    Hh = H.cpu().numpy()
    H64 = R.assemble_dense64(b.rowadr, b.rownnz, b.colind, b.M, b.J, b.D, b.state[0], b.nefc)
    # the matrix cores sum in their own order: tolerance parity (1e-5 relative L2, fp32)
    assert R.rel_l2(Hh[:, :nv, :nv], H64) <= 1e-5
    assert R.rel_l2(Hh, R.jtdj_dense(Md.reshape(nworld, -1), b.J, b.D, b.state[0], b.nefc, nv_pad)) <= 1e-5
    np.testing.assert_array_equal(Hh, Hh.transpose(0, 2, 1))
    assert np.abs(Hh[:, nv:, :]).max() == 0


@pytest.mark.gpu
def test_gpu_dense_hessian_row_counts_and_masks(device):
    """The dense J'DJ kernel stages rows 0..31 as they lie and, behind them, only the rows that
    contribute (inside nefc, QUADRATIC).  Row counts on both sides of 32 and of a chunk of 32
    listed rows, no active row at all, every row active, njmax that is no multiple of 4, and
    non-finite values in rows that must not be read (inactive, or past nefc)."""
    import torch

    rng = np.random.default_rng(21)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    # widths: one code path per staged width class (32, 64, 96, 128 with seven and with eight blocks of 16 dofs)
    for nv, njmax in ((27, 70), (35, 33), (128, 131), (56, 300), (70, 50), (100, 40), (113, 66),
                      (1, 34), (16, 40), (17, 36), (48, 65), (64, 33), (65, 47), (96, 35), (97, 64), (112, 97), (127, 34),
                      (35, 9000)):  # the last one: a row list beyond the default 64 KB of LDS
        counts = [0, 1, 31, 32, 33, 63, 64, 65, njmax - 1, njmax]
        nworld = 3 * len(counts)
        nefc = np.array(counts * 3, np.int32)
        J = rng.normal(size=(nworld, njmax, nv)).astype(np.float32)
        D = rng.uniform(0.5, 4.0, (nworld, njmax)).astype(np.float32)
        state = np.where(rng.uniform(size=(nworld, njmax)) < 0.5, synth.QUADRATIC, 0).astype(np.int32)
        state[: len(counts)] = 0  # no active row
        state[len(counts) : 2 * len(counts)] = synth.QUADRATIC  # every row active
        A = rng.normal(size=(nworld, nv, nv))
        Md = (A @ A.transpose(0, 2, 1) / nv + np.eye(nv)).astype(np.float32)
        Jdirty = J.copy()
        for w in range(nworld):
            Jdirty[w, nefc[w] :] = np.nan
            idle = np.flatnonzero(state[w, 32:] != synth.QUADRATIC) + 32  # behind the first chunk
            Jdirty[w, idle] = np.inf
        nv_pad = ((nv + 1 + 15) // 16) * 16
        H = torch.full((nworld, nv_pad, nv_pad), 7.0, device=device)
        BD.dense_hessian(t(Md), t(Jdirty), t(D), t(state), t(nefc), H)
        torch.cuda.synchronize()
        Hh = H.cpu().numpy()[:, :nv, :nv]
        want = R.jtdj_dense(Md.reshape(nworld, -1), J, D, state, nefc, nv_pad)[:, :nv, :nv]
        assert np.isfinite(Hh).all(), (nv, njmax)
        assert R.rel_l2(Hh, want) <= 1e-5, (nv, njmax)
        np.testing.assert_array_equal(Hh[: len(counts)], Md[: len(counts)])  # M + nothing


@pytest.mark.gpu
def test_gpu_wavefront_per_world_kernel_for_small_tiles_agrees():
    """Matrices up to 64 x 64 run four worlds per wavefront; the kernel with a
    workgroup per world that serves every other shape is forced here in a child process and
    must pass the same oracle comparison."""
    import os
    import subprocess
    import sys

    env = dict(os.environ, IMHIP_BLOCKED_KERNEL="simple")
    code = (
        "import sys, torch; sys.path.insert(0, 'tests'); import test_blocked_dense as t;"
        "d = torch.device('cuda:0');"
        "t.test_gpu_blocked_factor_solve_bitwise(d, 'g1', 8, 70);"
        "t.test_gpu_blocked_factor_solve_bitwise(d, 'snu', 8, 33);"
        "t.test_gpu_blocked_factor_solve_bitwise(d, 'g1', 16, 70);"
        "t.test_gpu_blocked_factor_solve_bitwise(d, 'snu', 16, 33); print('simple kernel ok')"
    )
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "simple kernel ok" in out.stdout, out.stderr[-2000:]


def test_dense_hessian_staging_indices_stay_inside_a_row():
    """The staging step of the dense J'DJ kernel writes row r of a 32-row chunk at
    Js[r * nvr + (c ^ x)] for the columns c = lane and lane + 64 that lie below nvr = the dofs
    rounded up to 32, with x = 16 * (r & 3) where nvr is a multiple of 64 and 16 * (r & 1)
    otherwise (csrc/blocked_kernels.hip, stage()): replayed here for every supported width, every
    element of the chunk is written exactly once and nothing outside it, and the operand reads
    of the matrix-core loop (row 4 q + l / 16, column block b exchanged the same way) find
    column 16 b + l % 16 of that row."""
    for nv in (1, 14, 27, 32, 33, 35, 56, 64, 65, 96, 128):
        nvr = (nv + 31) // 32 * 32
        swz = 3 if nvr % 64 == 0 else 1
        hits = np.zeros(32 * nvr + 32, int)
        where = {}
        for wave in range(4):
            for lane in range(64):
                for i in range(8):
                    for c in (lane, lane + 64):
                        if c < nvr:
                            r = wave * 8 + i
                            at = r * nvr + (c ^ (16 * (r & swz)))
                            hits[at] += 1
                            where[r, c] = at
        assert (hits[: 32 * nvr] == 1).all() and (hits[32 * nvr :] == 0).all(), nv
        for lane in range(64):
            kq = lane >> 4
            for q in range(8):
                for b in range((nv + 15) // 16):
                    read = kq * nvr + ((b ^ (kq & swz)) * 16) + (lane & 15) + 4 * q * nvr
                    assert read == where[4 * q + kq, 16 * b + (lane & 15)], (nv, lane, q, b)


def test_multi_solve_oracle_against_the_single_solve_and_fp64():
    """The stored-factor solve, column by column, is the single-right-hand-side solve bit for bit
    (same substitution steps), and solves M x = y; inactive worlds keep their x."""
    b, nv, Md = _dense_model("snu", 5, well=True)
    pad, layout, _ = BD.block_index_layout(np.arange(nv * nv), nv, nv * nv, 16)
    M32 = Md.reshape(5, -1).astype(np.float32)
    rng = np.random.default_rng(2)
    y = rng.normal(size=(5, nv, 3)).astype(np.float32)
    _, U = R.blocked_factor_solve(M32, layout, nv, pad, 16, y[:, :, 0])
    active = np.array([1, 0, 1, 1, 0], np.int32)
    x = R.blocked_multi_solve(U, nv, 16, y, active)
    assert np.abs(x[active == 0]).max() == 0.0
    for c in range(3):
        single = R.blocked_factor_solve(M32, layout, nv, pad, 16, np.ascontiguousarray(y[:, :, c]), want_factor=False)
        np.testing.assert_array_equal(x[active == 1, :, c], single[active == 1])
    for w in np.flatnonzero(active):
        want = np.linalg.solve(M32[w].reshape(nv, nv).astype(np.float64), y[w].astype(np.float64))
        np.testing.assert_allclose(x[w], want, rtol=2e-4, atol=2e-5)


def test_factor_solve_dispatcher_precedence_and_errors():
    # reference: src/instantmimic/utils/mjw_step_optimized.py:1030-1070, 984-986
    with pytest.raises(RuntimeError, match="requires the blocked dense path"):
        BD._factor_solve_i_dense(None, None, None, None, None, None, factor_workspace=object())
    # keeping the factor without a blocked scratch, and a sparse tail behind the dense blocks, are
    # upstream's factor_solve_i: without the callback both say so
    with pytest.raises(NotImplementedError):
        BD._factor_solve_i_dense(None, None, None, None, None, None, retain_factor=True)
    tailed = SimpleNamespace(M_tiles=[], qLD_has_sparse=True)
    with pytest.raises(NotImplementedError):
        BD._factor_solve_i_dense(tailed, SimpleNamespace(nworld=1), None, None, None, None)
    seen = []
    BD._factor_solve_i_dense(tailed, SimpleNamespace(nworld=1), None, None, None, None, upstream=seen.append)
    assert seen == [False]
    seen = []
    BD._factor_solve_i_dense(None, None, None, None, None, None, retain_factor=True, upstream=seen.append)
    assert seen == [True]


@pytest.mark.gpu
@pytest.mark.parametrize("name,B,nworld,nrhs", [("snu", 16, 3, 5), ("g1", 8, 37, 3), ("g1", 16, 37, 1), ("stress", 16, 6, 9), ("snu", 8, 20, 17)])
def test_gpu_blocked_multi_solve(device, name, B, nworld, nrhs):
    """reference: tests/test_blocked_dense_factor_solve.py:528-626 -- several right-hand sides with
    an active mask; the reuse kernel on a factor stored by the single-solve path equals the
    fused kernel bit for bit; inactive worlds are untouched; everything equals the oracle."""
    import torch

    b, nv, Md = _dense_model(name, nworld, well=True)
    M32 = np.ascontiguousarray(Md.reshape(nworld, -1).astype(np.float32))
    m = SimpleNamespace(nv=nv, M_tiles=[SimpleNamespace(size=nv, elemid=np.arange(nv * nv))])
    M = torch.from_numpy(M32).to(device)
    d = SimpleNamespace(nworld=nworld, M=M)
    scratch = BD.create_blocked_dense_factor_solve_scratch(m, d, device, block_size=B)
    rng = np.random.default_rng(31)
    rhs = rng.normal(size=(nworld, nv, nrhs)).astype(np.float32)
    act = (rng.random(nworld) < 0.7).astype(np.int32)
    act[0], act[1] = 1, 0
    y, active = torch.from_numpy(rhs).to(device), torch.from_numpy(act).to(device)
    factor = torch.full((nworld, scratch.pad, scratch.pad), 7.0, device=device)
    solution = torch.zeros_like(y)
    BD.blocked_factor_multi_solve(M, scratch, y, active, factor, solution)
    # the single-solve path stores its factor in a second workspace; solve again from it
    reused_factor = torch.zeros_like(factor)
    single_x = torch.zeros((nworld, nv), device=device)
    BD._factor_solve_i_dense(m, d, M, single_x, y[:, :, 0].contiguous(), scratch, factor_workspace=reused_factor)
    reused = torch.zeros_like(y)
    BD.blocked_multi_solve(reused_factor, scratch, y, active, reused)
    torch.cuda.synchronize()
    got = solution.cpu().numpy()
    np.testing.assert_array_equal(reused.cpu().numpy(), got)
    np.testing.assert_array_equal(got[act == 0], 0.0)
    assert (factor.cpu().numpy()[act == 0] == 7.0).all()  # an inactive world's factor is not written either
    # the factor: the tiles on and right of the block diagonal; those below it keep the caller's values,
    # as in the reference, whose kernel stores U_kk and U_ki for i > k only (indexed_factor.py:322, 360)
    blk = np.arange(scratch.pad) // B
    upper = blk[:, None] <= blk[None, :]
    f, fr = factor.cpu().numpy()[act == 1], reused_factor.cpu().numpy()[act == 1]
    np.testing.assert_array_equal(f[:, upper], fr[:, upper])
    assert (f[:, ~upper] == 7.0).all() and (fr[:, ~upper] == 0.0).all()
    _, U_ref = R.blocked_factor_solve(M32, scratch.indices.cpu().numpy(), nv, scratch.pad, B, rhs[:, :, 0])
    np.testing.assert_array_equal(got, R.blocked_multi_solve(U_ref, nv, B, rhs, act))
    np.testing.assert_array_equal(single_x.cpu().numpy()[act == 1], got[act == 1, :, 0])
    for w in np.flatnonzero(act)[:4]:
        want = np.linalg.solve(M32[w].reshape(nv, nv).astype(np.float64), rhs[w].astype(np.float64))
        assert np.abs(got[w] - want).max() / max(np.abs(want).max(), 1e-6) < 2e-3


@pytest.mark.gpu
def test_gpu_retained_factor_goes_to_the_dense_block_layout(device):
    # reference: src/instantmimic/utils/mjw_step_optimized.py:875-886, 984-993
    import torch

    nworld = 11
    b, nv, Md = _dense_model("g1", nworld, well=True)
    M = torch.from_numpy(np.ascontiguousarray(Md.reshape(nworld, -1).astype(np.float32))).to(device)
    m = SimpleNamespace(nv=nv, M_tiles=[SimpleNamespace(size=nv, elemid=np.arange(nv * nv))],
                        qLD_block_adr=torch.tensor([13], dtype=torch.int32, device=device))  # fmt: skip
    d = SimpleNamespace(nworld=nworld, M=M, qLD=torch.full((nworld, 13 + nv * nv + 5), -3.0, device=device))
    scratch = BD.create_blocked_dense_factor_solve_scratch(m, d, device)
    y = torch.from_numpy(b.grad).to(device)
    x = torch.zeros_like(y)
    BD._factor_solve_i_dense(m, d, M, x, y, scratch, retain_factor=True)
    torch.cuda.synchronize()
    qLD, U = d.qLD.cpu().numpy(), scratch.U.cpu().numpy()
    np.testing.assert_array_equal(qLD[:, 13 : 13 + nv * nv].reshape(nworld, nv, nv), U[:, :nv, :nv])
    assert (qLD[:, :13] == -3.0).all() and (qLD[:, 13 + nv * nv :] == -3.0).all()
    with pytest.raises(RuntimeError, match="requires qLD block offsets"):
        BD._blocked_dense_factor_solve(d, M, x, y, scratch, factor_out=d.qLD)


@pytest.mark.gpu
def test_gpu_short_pivot_forms_equal_sqrtf_and_the_division(device):
    """The blocked Cholesky takes the square root of a pivot as the hardware's estimate plus a
    neighbour test and its reciprocal as the estimate plus one correction: both must be the IEEE
    results for every float in [2^-96, inf), all 1.9e9 of them."""
    import torch

    from instantmimic_amd import _lib

    count = torch.zeros(1, dtype=torch.int64, device=device)
    stream = int(torch.cuda.current_stream(device).cuda_stream)
    assert _lib.lib().im_check_pivot_sqrt(0, 0x7F800000, count.data_ptr(), stream) == _lib.IM_OK
    torch.cuda.synchronize()
    assert int(count.item()) == 0


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld", [("stress", 40), ("g1", 70), ("humanoid", 50), ("snu", 33), ("ant", 9)])
def test_gpu_hessian_factor_solve_in_one_launch(device, name, nworld):
    """im_jtdj_factor_solve against im_jtdj_mfma followed by im_blocked_factor_solve: H, the factor
    and x bit for bit; x against the fp64 solve within what cond(H) allows."""
    import torch

    b, nv, Md = _dense_model(name, nworld)
    pad16 = -(-nv // 16) * 16
    nv_pad = ((nv + 1 + 15) // 16) * 16
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    M32, J, D, S, N, g = t(Md.reshape(nworld, -1).astype(np.float32)), t(b.J), t(b.D), t(b.state[0]), t(b.nefc), t(b.grad)
    H1 = torch.zeros((nworld, nv_pad, nv_pad), device=device)
    BD.dense_hessian(M32, J, D, S, N, H1)
    Hc = H1[:, :nv, :nv].contiguous().reshape(nworld, -1)
    m = SimpleNamespace(nv=nv, M_tiles=[SimpleNamespace(size=nv, elemid=np.arange(nv * nv))])
    d = SimpleNamespace(nworld=nworld, M=Hc)
    scratch = BD.create_blocked_dense_factor_solve_scratch(m, d, device, block_size=16, minimum_nv=1)
    x1 = torch.zeros((nworld, nv), device=device)
    BD._blocked_dense_factor_solve(d, Hc, x1, g, scratch)
    H2 = torch.full_like(H1, 0.0)
    U2 = torch.full((nworld, pad16, pad16), float("nan"), device=device)
    x2 = torch.full((nworld, nv), float("nan"), device=device)
    BD.dense_hessian_factor_solve(M32, J, D, S, N, H2, g, x2, factor=U2)
    x3 = torch.full((nworld, nv), float("nan"), device=device)
    BD.dense_hessian_factor_solve(M32, J, D, S, N, None, g, x3)  # neither H nor the factor kept
    torch.cuda.synchronize()
    assert torch.equal(H1, H2)
    # the factor's tiles on and right of the block diagonal; the others are not written
    blk = torch.arange(pad16, device=device) // 16
    upper = blk[:, None] <= blk[None, :]
    assert torch.equal(scratch.U[:, upper], U2[:, upper]) and bool(torch.isnan(U2[:, ~upper]).all())
    assert torch.equal(x1, x2) and torch.equal(x1, x3)
    H64 = H1[:, :nv, :nv].double().cpu().numpy()
    x64 = np.linalg.solve(H64, b.grad.astype(np.float64)[:, :, None])[:, :, 0]
    err = np.linalg.norm(x2.cpu().numpy() - x64, axis=1) / np.linalg.norm(x64, axis=1)
    assert (err / (np.linalg.cond(H64) * 6e-8)).max() < 2.0
