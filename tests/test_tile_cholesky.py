"""Cholesky of matrices that fit one tile, with the solve and without a stored factor: the
reference's two tile kernels (src/instantmimic/utils/mjw_step_optimized.py:672-750), the dispatch
around them (:790-873, :1030-1070) and the Newton factor stage up to 32 dofs
(src/instantmimic/utils/mjw_kernels/newton_stages.py:723-733)."""

import dataclasses
from types import SimpleNamespace

import numpy as np
import pytest
import scipy.linalg as sl

import test_newton_stages as TS
from instantmimic_amd import synth
from instantmimic_amd.mjw_kernels import blocked_dense as BD
from instantmimic_amd.mjw_kernels import newton_stages as NS
from oracle import ref as R


def _spd(rng, nworld, n, scale=1.0):
    A = rng.normal(size=(nworld, n, n))
    return (A @ A.transpose(0, 2, 1) * scale + n * np.eye(n)).astype(np.float32)


def _block_diagonal(rng, nworld, sizes):
    n = sum(sizes)
    M = np.zeros((nworld, n, n), np.float32)
    at = 0
    for s in sizes:
        M[:, at : at + s, at : at + s] = _spd(rng, nworld, s)
        at += s
    return M


# ---------------------------------------------------------------- oracle pinning (CPU)


@pytest.mark.parametrize("n", [1, 2, 5, 14, 16, 27, 32, 33, 50, 64])
def test_oracle_tile_solve_against_scipy(n):
    rng = np.random.default_rng(n)
    A = _spd(rng, 9, n)
    y = rng.normal(size=(9, n)).astype(np.float32)
    x = R.tile_cholesky_solve(A, [0], n, y)
    for w in range(9):
        A64 = A[w].astype(np.float64)
        x64 = sl.cho_solve(sl.cho_factor(A64), y[w].astype(np.float64))
        assert np.linalg.norm(x[w] - x64) / np.linalg.norm(x64) < 4 * np.linalg.cond(A64) * 6e-8


def test_oracle_tile_solve_reads_one_triangle_and_leaves_other_dofs():
    rng = np.random.default_rng(3)
    sizes = [6, 6, 6]
    M = _block_diagonal(rng, 4, sizes)
    y = rng.normal(size=(4, 20)).astype(np.float32)  # two dofs behind the last tile
    Mp = np.zeros((4, 20, 20), np.float32)
    Mp[:, :18, :18] = M
    x = R.tile_cholesky_solve(Mp, [0, 6, 12], 6, y)
    assert not x[:, 18:].any()
    want = np.concatenate([R.tile_cholesky_solve(M[:, a : a + 6, a : a + 6].copy(), [0], 6, y[:, a : a + 6].copy()) for a in (0, 6, 12)], axis=1)
    np.testing.assert_array_equal(x[:, :18], want)
    # the dense form reads the lower triangle only
    junk = Mp + np.triu(rng.normal(size=Mp.shape).astype(np.float32), 1)
    np.testing.assert_array_equal(R.tile_cholesky_solve(junk, [0, 6, 12], 6, y), x)
    # the indexed form reads the upper triangle: element ids of a dense row-major tile, lower ids poisoned
    flat = Mp.reshape(4, -1)
    ids = np.zeros((3, 6, 6), np.int32)
    for t, a in enumerate((0, 6, 12)):
        r, c = np.meshgrid(np.arange(6), np.arange(6), indexing="ij")
        ids[t] = (a + r) * 20 + a + c
        ids[t][np.tril_indices(6, -1)] = 10**6  # past nM: would read as zero
    np.testing.assert_array_equal(R.tile_cholesky_solve(flat, [0, 6, 12], 6, y, elemid=ids), x)


@pytest.mark.parametrize("name", ["ant", "humanoid"])
def test_oracle_tile_solve_is_the_blocked_factor_up_to_one_block(name):
    """Up to 16 dofs the blocked factor has one diagonal tile and nothing else: the same operations.
    Beyond, the two agree to conditioning (different groupings of the same sums)."""
    shape = synth.SHAPES[name]
    b = synth.make_batch(shape, 12)
    nv, nM = shape.nv, b.M.shape[1]
    elemid = synth.matrix_elemid(b.rowadr, b.rownnz, b.colind)
    ids = np.where(elemid < 0, nM, elemid).astype(np.int32)
    x = R.tile_cholesky_solve(b.M, [0], nv, b.grad, elemid=ids)
    pad, layout, _ = BD.block_index_layout(ids, nv, nM, 16)
    xb = R.blocked_factor_solve(b.M, layout, nv, pad, 16, b.grad, want_factor=False)
    if nv <= 16:
        np.testing.assert_array_equal(x, xb)
    else:
        assert R.rel_l2(x, xb) < 1e-4  # conditioning of the synthetic M times fp32 rounding
    Md = synth.dense_from_csr(b.M.astype(np.float64), b.rowadr, b.rownnz, b.colind)
    assert R.rel_l2(x, R.solve64(Md, b.grad)) < 1e-4


@pytest.mark.parametrize("name", ["ant", "humanoid"])
def test_oracle_small_dense_stage_against_fp64(name):
    """Up to 32 dofs the stage factors the updated H as one tile at every call and keeps no factor."""
    shape = synth.SHAPES[name]
    b = synth.make_batch(dataclasses.replace(shape, iterations=2), 28, ragged_nefc=True)
    nv, pad = shape.nv, 32
    rng = np.random.default_rng(5)
    st, H0 = TS._dense_start(b, pad)
    new, ids, changes, sc, done, grad = TS._changes(b, rng)
    U0 = np.full_like(H0, 7.0)
    H1, U1, uni, search, sdot, decr = R.dense_update_factor(sc, changes, ids, b.J, b.D, new, grad, H0, U0, done=done)
    np.testing.assert_array_equal(U1, U0)
    live = TS._live(sc, done)
    assert not search[~live].any()
    np.testing.assert_array_equal(H1[~live], H0[~live])
    Hd = R.assemble_dense64(*st, b.M, b.J, b.D, new, b.nefc)
    iu = np.triu_indices(nv)
    Hold = R.assemble_dense64(*st, b.M, b.J, b.D, b.state[0], b.nefc)
    scale = np.maximum(np.abs(Hd).max(axis=(1, 2)), np.abs(Hold).max(axis=(1, 2)))[:, None]
    assert (np.abs(H1[:, :nv, :nv][:, iu[0], iu[1]] - Hd[:, iu[0], iu[1]]) / scale)[live].max() < 3e-6
    x64 = R.solve64(Hd, grad)
    cond = np.linalg.cond(Hd)
    err = np.linalg.norm(-search - x64, axis=1) / np.linalg.norm(x64, axis=1)
    assert (err / (cond * 6e-8))[live].max() < 4.0
    sd64 = (x64**2).sum(1)
    assert (np.abs(sdot - sd64) / sd64 / np.maximum(cond * 6e-8, 1e-6))[live].max() < 10.0
    np.testing.assert_allclose(decr[live], (grad * x64).sum(1)[live], rtol=2e-3, atol=2e-3 * np.abs(decr).max())
    # worlds without a changed row are factored again all the same (there is no stored factor)
    again = live & (changes == 0)
    assert again.any()
    direct = R.tile_cholesky_solve(np.triu(H1[:, :nv, :nv]).transpose(0, 2, 1).copy(), [0], nv, grad)
    np.testing.assert_array_equal(-search[again], direct[again])


# ---------------------------------------------------------------- GPU


def _t(a, device):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


@pytest.mark.gpu
@pytest.mark.parametrize("sizes", [[1], [5, 5, 5], [14], [16, 16], [27], [32], [33], [50, 50], [64], [8, 8, 8, 8, 8, 8, 8]])
def test_gpu_dense_tiles_bitwise(device, sizes):
    import torch

    rng = np.random.default_rng(sum(sizes))
    nworld, size = 133, sizes[0]
    M = _block_diagonal(rng, nworld, sizes)
    n = M.shape[1] + 3  # dofs behind the last tile stay as they are
    Mp = np.zeros((nworld, n, n), np.float32)
    Mp[:, : n - 3, : n - 3] = M
    adr = np.cumsum([0] + sizes[:-1]).astype(np.int32)
    y = rng.normal(size=(nworld, n)).astype(np.float32)
    want = R.tile_cholesky_solve(Mp, adr, size, y)
    tiles = [SimpleNamespace(size=size, adr=adr)]
    m, d = SimpleNamespace(qM_tiles=tiles, nv=n), SimpleNamespace(nworld=nworld)
    x = torch.full((nworld, n), 9.0, device=device)
    BD._factor_solve_i_dense(m, d, _t(Mp, device), x, _t(y, device))
    torch.cuda.synchronize()
    got = x.cpu().numpy()
    np.testing.assert_array_equal(got[:, : n - 3], want[:, : n - 3])
    assert (got[:, n - 3 :] == 9.0).all()


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld", [("ant", 257), ("humanoid", 4096)])
def test_gpu_structured_tiles_bitwise(device, name, nworld):
    """M stored by its structure with the tile's element ids, through ``factor_solve_i_no_l_store``
    and ``_factor_solve_i_dense`` without any scratch or upstream callback."""
    import torch

    shape = synth.SHAPES[name]
    b = synth.make_batch(shape, nworld)
    nv, nM = shape.nv, b.M.shape[1]
    elemid = synth.matrix_elemid(b.rowadr, b.rownnz, b.colind)
    ids = np.where(elemid < 0, nM, elemid).astype(np.int32)
    want = R.tile_cholesky_solve(b.M, [0], nv, b.grad, elemid=ids)
    tile = SimpleNamespace(size=nv, adr=np.zeros(1, np.int32), elemid=_t(ids.reshape(-1), device))
    m = SimpleNamespace(M_tiles=[tile], nv=nv, qLD_block_total=5)
    d = SimpleNamespace(nworld=nworld, qLD=torch.zeros((nworld, 5), device=device))
    M, y = _t(b.M, device), _t(b.grad, device)
    x = torch.zeros((nworld, nv), device=device)
    BD.factor_solve_i_no_l_store(m, d, M, None, None, x, y)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(x.cpu().numpy(), want)
    x2 = torch.zeros((nworld, nv), device=device)
    BD._factor_solve_i_dense(m, d, M, x2, y)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(x2.cpu().numpy(), want)
    # keeping the factor, or a sparse tail behind the blocks, is upstream's: it says so
    with pytest.raises(NotImplementedError):
        BD._factor_solve_i_dense(m, d, M, x2, y, retain_factor=True)
    d.qLD = torch.zeros((nworld, 9), device=device)
    called = []
    BD.factor_solve_i_no_l_store(m, d, M, None, None, x2, y, upstream=called.append)
    assert called == [True]


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld", [("ant", 131), ("humanoid", 4096)])
def test_gpu_small_dense_stage_bitwise(device, name, nworld):
    import torch

    shape = synth.SHAPES[name]
    b = synth.make_batch(dataclasses.replace(shape, iterations=2), nworld, ragged_nefc=True)
    nv, pad = shape.nv, 32
    rng = np.random.default_rng(9)
    _, H0 = TS._dense_start(b, pad)
    new, ids, changes, sc, done, grad = TS._changes(b, rng)
    U0 = np.full_like(H0, 3.0)
    want = R.dense_update_factor(sc, changes, ids, b.J, b.D, new, grad, H0, U0, done=done)
    H, U = _t(H0, device), _t(U0, device)
    uni = torch.zeros((nworld, nv + 1), dtype=torch.int32, device=device)
    search = torch.zeros((nworld, pad, 1), device=device)
    sdot, decr = torch.zeros(nworld, device=device), torch.zeros(nworld, device=device)
    stage = NS.factor_factory(nv, pad)
    g3 = torch.zeros((nworld, pad, 1), device=device)
    g3[:, :nv, 0] = _t(grad, device)
    stage(_t(b.J, device), _t(b.D, device), _t(new, device), _t(ids, device), _t(changes, device), _t(sc, device),
          _t(done, device), g3, H, U, search, sdot, decr, uni)  # fmt: skip
    torch.cuda.synchronize()
    live = TS._live(sc, done)
    np.testing.assert_array_equal(H.cpu().numpy(), want[0])
    np.testing.assert_array_equal(U.cpu().numpy(), U0)
    np.testing.assert_array_equal(uni.cpu().numpy()[live], want[2][live])
    np.testing.assert_array_equal(search.cpu().numpy()[:, :nv, 0], want[3])
    np.testing.assert_array_equal(sdot.cpu().numpy(), want[4])
    np.testing.assert_array_equal(decr.cpu().numpy(), want[5])
