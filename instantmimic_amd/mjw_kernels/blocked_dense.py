"""Blocked dense Cholesky factor + solve and the dense ``J'DJ`` Hessian on MI355X.

Drop-in for ``create_blocked_dense_factor_solve_scratch`` / ``_blocked_dense_factor_solve`` /
``_factor_solve_i_dense`` (src/instantmimic/utils/mjw_step_optimized.py:893-1070), for the
multi-right-hand-side kernels of src/instantmimic/utils/mjw_kernels/indexed_factor.py:217-493
and for the dense Hessian assembly the reference takes from mujoco_warp (call site
src/instantmimic/utils/mjw_kernels/newton_fusion.py:470).  Index tables and kernels live in
``libimhip`` (``csrc/blocked_kernels.hip``); this module checks shapes and passes pointers.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable

import numpy as np

from .. import _lib

_BLOCKED_DENSE_FACTOR_BLOCK_SIZE = 16
_BLOCKED_DENSE_FACTOR_BLOCK_DIM = 64
_BLOCKED_DENSE_FACTOR_MIN_NV = 32
QUADRATIC = 1


@dataclass(frozen=True)
class BlockedDenseFactorSolveScratch:
    nv: int
    pad: int
    block_size: int
    block_dim: int
    U: Any  # (nworld, pad, pad) factor workspace
    indices: Any  # (nblk * nblk * B * B,) int32 element ids into M[w, :]
    identity: Any  # (B * B,) 1 on the padded diagonal of the last block
    kernel: Any
    nM: int


def block_index_layout(elemid, nv: int, nM: int, block_size: int):
    """(pad, layout, identity) of a dense tile's element ids: ``im_blocked_index_layout``."""
    ids = np.ascontiguousarray(np.asarray(elemid).reshape(-1), np.int32)
    if ids.size != nv * nv:
        raise ValueError("elemid must hold nv * nv element ids")
    pad = -(-nv // block_size) * block_size
    layout, identity = np.zeros(pad * pad, np.int32), np.zeros(block_size * block_size, np.float32)
    status = _lib.lib().im_blocked_index_layout(ids.ctypes.data, nv, nM, block_size, layout.ctypes.data, identity.ctypes.data)
    _lib.check(status, "im_blocked_index_layout")
    return pad, layout, identity


def create_blocked_dense_factor_solve_scratch(
    m: Any, d: Any, device: Any = None, *, minimum_nv: int = _BLOCKED_DENSE_FACTOR_MIN_NV,
    block_size: int = _BLOCKED_DENSE_FACTOR_BLOCK_SIZE,
) -> BlockedDenseFactorSolveScratch | None:  # fmt: skip
    """Blocked factor + solve buffers when the model qualifies (:893-955): at least
    ``minimum_nv`` dofs and an inertia matrix stored as one dense tile spanning every dof
    (``m.M_tiles`` with one tile whose ``elemid`` is (nv * nv,)); else ``None``."""
    import torch

    nv = getattr(m, "nv", 0)
    if not isinstance(nv, int) or nv < minimum_nv:
        return None
    tiles = getattr(m, "M_tiles", None)
    if tiles is None or len(tiles) != 1:
        return None
    tile = tiles[0]
    elemid = getattr(tile, "elemid", None)
    if int(getattr(tile, "size", 0)) != nv or elemid is None:
        return None
    elemid = np.asarray(elemid.cpu().numpy() if hasattr(elemid, "cpu") else elemid)
    if elemid.shape != (nv * nv,):
        return None
    nworld = getattr(d, "nworld", 0)
    if not isinstance(nworld, int) or nworld <= 0 or getattr(d, "M", None) is None:
        return None
    dev = torch.device(device if device is not None else d.M.device)
    nM = int(d.M.shape[1])
    pad, layout, identity = block_index_layout(elemid, nv, nM, block_size)
    return BlockedDenseFactorSolveScratch(
        nv=nv, pad=pad, block_size=block_size, block_dim=256,
        U=torch.zeros((nworld, pad, pad), dtype=torch.float32, device=dev),
        indices=torch.from_numpy(layout).to(dev), identity=torch.from_numpy(identity).to(dev),
        kernel="im_blocked_factor_solve", nM=nM,
    )  # fmt: skip


def _stream(t) -> int:
    import torch

    return int(torch.cuda.current_stream(t.device).cuda_stream)


def _check_workspace(workspace, nworld: int, scratch) -> None:
    if tuple(workspace.shape) != (nworld, scratch.pad, scratch.pad) or not workspace.is_contiguous():
        raise ValueError("the factor workspace must be a contiguous (nworld, pad, pad) tensor")


def _blocked_dense_factor_solve(
    d: Any, M, x, y, scratch: BlockedDenseFactorSolveScratch, *, qLD_block_adr=None, factor_out=None,
    factor_workspace=None,
) -> None:  # fmt: skip
    """x = M^-1 y; the upper factor is left in ``scratch.U`` (or ``factor_workspace``) and, with
    ``factor_out``, copied into the caller's dense-block factor array at ``qLD_block_adr[0]``
    (:958-993)."""
    import torch

    nworld = int(d.nworld)
    workspace = scratch.U if factor_workspace is None else factor_workspace
    for t in (M, x, y, workspace):
        if t.dtype != torch.float32 or not t.is_cuda or t.stride(-1) != 1 or t.device != M.device:
            raise ValueError("blocked factor needs float32 CUDA tensors with contiguous rows on one device")
    _check_workspace(workspace, nworld, scratch)
    x2, y2 = x.reshape(nworld, -1), y.reshape(nworld, -1)
    if M.shape[0] != nworld or x2.shape[1] < scratch.nv or y2.shape[1] < scratch.nv or M.shape[1] < scratch.nM:
        raise ValueError("M, x and y do not match the scratch's sizes")
    if factor_out is not None and qLD_block_adr is None:
        raise RuntimeError("persisting a blocked factor requires qLD block offsets")
    with torch.cuda.device(M.device):
        status = _lib.lib().im_blocked_factor_solve(
            M.data_ptr(), M.stride(0), scratch.nM, scratch.indices.data_ptr(), scratch.block_size, scratch.nv,
            scratch.pad, y2.data_ptr(), y2.stride(0), workspace.data_ptr(), x2.data_ptr(), x2.stride(0), nworld,
            _stream(M),
        )  # fmt: skip
        _lib.check(status, "im_blocked_factor_solve")
        if factor_out is not None:
            if qLD_block_adr.dtype != torch.int32 or not qLD_block_adr.is_cuda or factor_out.dtype != torch.float32:
                raise TypeError("qLD_block_adr must be an int32 and factor_out a float32 CUDA tensor")
            if factor_out.dim() != 2 or factor_out.shape[0] != nworld or factor_out.stride(1) != 1:
                raise ValueError("factor_out must be (nworld, nC) with contiguous rows")
            status = _lib.lib().im_copy_dense_factor(
                workspace.data_ptr(), scratch.pad, qLD_block_adr.data_ptr(), scratch.nv, factor_out.data_ptr(),
                factor_out.stride(0), nworld, _stream(M),
            )  # fmt: skip
            _lib.check(status, "im_copy_dense_factor")


def _factor_solve_i_dense(
    m: Any, d: Any, M, x, y, dense_factor_solve: BlockedDenseFactorSolveScratch | None = None, *,
    retain_factor: bool = False, factor_workspace=None, tree_factor_solve=None,
    upstream: Callable[..., None] | None = None,
) -> None:  # fmt: skip
    """Dense factor + solve that prefers the tree L'DL when no factor is kept, then the blocked
    kernel when its scratch exists: the reference's precedence and errors (:1030-1070).  What is
    left after those two is upstream mujoco_warp code (``smooth.factor_solve_i`` and the
    single-tile solve), which is not part of this library: pass it as ``upstream(retain_factor)``."""
    from . import tree_ldl

    if factor_workspace is not None and dense_factor_solve is None:
        raise RuntimeError("a retained factor workspace requires the blocked dense path")
    if tree_factor_solve is not None and not retain_factor and factor_workspace is None:
        tree_ldl.tree_factor_solve(tree_factor_solve, M, x, y)
        return
    if dense_factor_solve is not None:
        _blocked_dense_factor_solve(
            d, M, x, y, dense_factor_solve, qLD_block_adr=m.qLD_block_adr if retain_factor else None,
            factor_out=d.qLD if retain_factor else None, factor_workspace=factor_workspace,
        )  # fmt: skip
        return
    if upstream is None:
        raise NotImplementedError("neither a tree nor a blocked scratch: the remaining solves are upstream's")
    upstream(retain_factor)


def _check_rhs(scratch, nworld: int, y, x, active) -> int:
    import torch

    if y.dim() != 3 or tuple(y.shape[:2]) != (nworld, scratch.nv) or tuple(x.shape) != tuple(y.shape):
        raise ValueError("y and x must be (nworld, nv, rhs_count)")
    for t in (y, x):
        if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
            raise ValueError("y and x must be contiguous float32 CUDA tensors")
    if active is not None and (active.dtype != torch.int32 or active.numel() != nworld or not active.is_contiguous()):
        raise TypeError("active must be a contiguous int32 tensor with one element per world")
    return int(y.shape[2])


def blocked_factor_multi_solve(M, scratch: BlockedDenseFactorSolveScratch, y, active, factor, x) -> None:
    """Factor every active world's M into ``factor`` (nworld, pad, pad) and solve for all
    ``rhs_count`` columns of ``y`` (nworld, nv, rhs_count): the launch of
    ``make_indexed_cholesky_factor_multi_solve_kernel`` (indexed_factor.py:217-391).  Inactive
    worlds keep their ``factor`` and ``x``."""
    import torch

    nworld = int(M.shape[0])
    nrhs = _check_rhs(scratch, nworld, y, x, active)
    _check_workspace(factor, nworld, scratch)
    with torch.cuda.device(M.device):
        status = _lib.lib().im_blocked_factor_multi_solve(
            M.data_ptr(), M.stride(0), scratch.nM, scratch.indices.data_ptr(), scratch.block_size, scratch.nv,
            scratch.pad, y.data_ptr(), nrhs, None if active is None else active.data_ptr(), factor.data_ptr(),
            x.data_ptr(), nworld, _stream(M),
        )  # fmt: skip
    _lib.check(status, "im_blocked_factor_multi_solve")


def blocked_multi_solve(factor, scratch: BlockedDenseFactorSolveScratch, y, active, x) -> None:
    """Solve with a stored factor: ``make_indexed_cholesky_multi_solve_kernel``
    (indexed_factor.py:394-493)."""
    import torch

    nworld = int(factor.shape[0])
    nrhs = _check_rhs(scratch, nworld, y, x, active)
    _check_workspace(factor, nworld, scratch)
    with torch.cuda.device(factor.device):
        status = _lib.lib().im_blocked_multi_solve(
            factor.data_ptr(), scratch.block_size, scratch.nv, scratch.pad, y.data_ptr(), nrhs,
            None if active is None else active.data_ptr(), x.data_ptr(), nworld, _stream(factor),
        )  # fmt: skip
    _lib.check(status, "im_blocked_multi_solve")


def dense_hessian(M_dense, J, D, state, nefc, H, *, quad: int = QUADRATIC) -> None:
    """``H[w, :nv, :nv] = M_dense[w] + J[w]' diag(D [state == quad, row < nefc]) J[w]`` on
    fp32 MFMA; ``H`` is (nworld, nv_pad, nv_pad)."""
    import torch

    nworld, njmax, nv = J.shape
    for t in (M_dense, J, D, state, H):
        if not t.is_cuda or not t.is_contiguous():
            raise ValueError("dense_hessian needs contiguous CUDA tensors")
    if njmax < 1 or tuple(D.shape) != (nworld, njmax) or tuple(state.shape) != (nworld, njmax):
        raise ValueError("D and state must be (nworld, njmax >= 1)")
    if H.dim() != 3 or H.shape[0] != nworld or H.shape[1] != H.shape[2] or H.shape[1] < nv or M_dense.numel() != nworld * nv * nv:
        raise ValueError("H must be (nworld, nv_pad, nv_pad) and M_dense (nworld, nv, nv)")
    with torch.cuda.device(J.device):
        status = _lib.lib().im_jtdj_mfma(
            M_dense.data_ptr(), J.data_ptr(), int(njmax), D.data_ptr(), state.data_ptr(),
            nefc.data_ptr() if nefc is not None else None, int(quad), H.data_ptr(), int(nv), int(H.shape[1]),
            int(nworld), int(torch.cuda.current_stream(J.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_jtdj_mfma")


def dense_hessian_factor_solve(M_dense, J, D, state, nefc, H, y, x, *, factor=None, quad: int = QUADRATIC) -> None:
    """:func:`dense_hessian` and the blocked Cholesky (16 x 16 tiles) with its solve in one launch:
    ``H`` (nworld, nv_pad, nv_pad) or None, ``x = H^-1 y`` (nworld, nv), ``factor`` (nworld, pad,
    pad) with ``pad`` = nv rounded up to 16, or None.  Bit for bit what :func:`dense_hessian`
    followed by :func:`_blocked_dense_factor_solve` on the whole H gives."""
    import torch

    nworld, njmax, nv = J.shape
    pad = -(-nv // 16) * 16
    for t in (M_dense, J, D, state, y, x):
        if not t.is_cuda or t.device != J.device:
            raise ValueError("dense_hessian_factor_solve needs CUDA tensors on one device")
    for t in (M_dense, J, D, state):
        if not t.is_contiguous():
            raise ValueError("M_dense, J, D and state must be contiguous")
    if njmax < 1 or tuple(D.shape) != (nworld, njmax) or tuple(state.shape) != (nworld, njmax) or M_dense.numel() != nworld * nv * nv:
        raise ValueError("D and state must be (nworld, njmax >= 1) and M_dense (nworld, nv, nv)")
    if H is not None and (not H.is_contiguous() or H.dim() != 3 or H.shape[0] != nworld or H.shape[1] != H.shape[2] or H.shape[1] < nv):
        raise ValueError("H must be a contiguous (nworld, nv_pad, nv_pad) tensor")
    y2, x2 = y.reshape(nworld, -1), x.reshape(nworld, -1)
    if y2.shape[1] < nv or x2.shape[1] < nv or y2.stride(1) != 1 or x2.stride(1) != 1 or y.dtype != torch.float32 or x.dtype != torch.float32:
        raise ValueError("y and x must be float32 (nworld, >= nv) tensors with contiguous rows")
    if factor is not None and (not factor.is_contiguous() or tuple(factor.shape) != (nworld, pad, pad) or factor.dtype != torch.float32):
        raise ValueError(f"factor must be a contiguous float32 (nworld, {pad}, {pad}) tensor")
    with torch.cuda.device(J.device):
        status = _lib.lib().im_jtdj_factor_solve(
            M_dense.data_ptr(), J.data_ptr(), int(njmax), D.data_ptr(), state.data_ptr(),
            nefc.data_ptr() if nefc is not None else None, int(quad), None if H is None else H.data_ptr(), int(nv),
            0 if H is None else int(H.shape[1]), y2.data_ptr(), y2.stride(0), None if factor is None else factor.data_ptr(),
            pad, x2.data_ptr(), x2.stride(0), int(nworld), _stream(J),
        )  # fmt: skip
    _lib.check(status, "im_jtdj_factor_solve")
