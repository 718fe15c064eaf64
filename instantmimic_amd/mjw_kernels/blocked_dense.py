"""Blocked dense Cholesky factor + solve and the dense ``J'DJ`` Hessian on MI355X.

Drop-in for ``create_blocked_dense_factor_solve_scratch`` / ``_blocked_dense_factor_solve``
(src/instantmimic/utils/mjw_step_optimized.py:893-993) and for the dense Hessian assembly
the reference takes from mujoco_warp (call site
src/instantmimic/utils/mjw_kernels/newton_fusion.py:470).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import numpy as np

from .. import _lib

_BLOCKED_DENSE_FACTOR_BLOCK_SIZE = 16
_BLOCKED_DENSE_FACTOR_BLOCK_DIM = 64
_BLOCKED_DENSE_FACTOR_MIN_NV = 32
QUADRATIC = 1


def _round_up(value: int, multiple: int) -> int:
    return ((value + multiple - 1) // multiple) * multiple


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


def block_index_layout(elemid: np.ndarray, nv: int, nM: int, block_size: int):
    """Element ids of M's dense tile in (nblk, nblk, B, B) order, ``nM`` (out of range,
    reads as zero) on the padding; and the identity pad of the last diagonal block."""
    pad = _round_up(nv, block_size)
    nblk = pad // block_size
    padded = np.full((pad, pad), nM, dtype=np.int32)
    padded[:nv, :nv] = np.asarray(elemid).reshape(nv, nv)
    layout = padded.reshape(nblk, block_size, nblk, block_size).transpose(0, 2, 1, 3).copy().reshape(-1)
    identity = np.zeros((block_size, block_size), np.float32)
    for index in range(block_size):
        if (nblk - 1) * block_size + index >= nv:
            identity[index, index] = 1.0
    return pad, layout, identity.reshape(-1)


def create_blocked_dense_factor_solve_scratch(
    m: Any, d: Any, device: Any = None, *, minimum_nv: int = _BLOCKED_DENSE_FACTOR_MIN_NV,
    block_size: int = _BLOCKED_DENSE_FACTOR_BLOCK_SIZE,
) -> BlockedDenseFactorSolveScratch | None:  # fmt: skip
    """Blocked factor + solve buffers when the model qualifies: at least ``minimum_nv``
    dofs and an inertia matrix stored as one dense tile spanning every dof
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


def _blocked_dense_factor_solve(d: Any, M, x, y, scratch: BlockedDenseFactorSolveScratch, *, factor_workspace=None) -> None:
    """x = M^-1 y; the upper factor is left in ``scratch.U`` (or ``factor_workspace``)."""
    import torch

    nworld = int(d.nworld)
    workspace = scratch.U if factor_workspace is None else factor_workspace
    for t in (M, x, y):
        if t.dtype != torch.float32 or not t.is_cuda or t.stride(-1) != 1:
            raise ValueError("blocked factor needs float32 CUDA tensors with contiguous rows")
    x2, y2 = x.reshape(nworld, -1), y.reshape(nworld, -1)
    with torch.cuda.device(M.device):
        status = _lib.lib().im_blocked_factor_solve(
            M.data_ptr(), M.stride(0), scratch.nM, scratch.indices.data_ptr(), scratch.block_size, scratch.nv,
            scratch.pad, y2.data_ptr(), y2.stride(0), workspace.data_ptr(), x2.data_ptr(), x2.stride(0), nworld,
            int(torch.cuda.current_stream(M.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_blocked_factor_solve")


def dense_hessian(M_dense, J, D, state, nefc, H, *, quad: int = QUADRATIC) -> None:
    """``H[w, :nv, :nv] = M_dense[w] + J[w]' diag(D [state == quad, row < nefc]) J[w]`` on
    fp32 MFMA; ``H`` is (nworld, nv_pad, nv_pad)."""
    import torch

    nworld, njmax, nv = J.shape
    for t in (M_dense, J, D, state, H):
        if not t.is_cuda or not t.is_contiguous():
            raise ValueError("dense_hessian needs contiguous CUDA tensors")
    with torch.cuda.device(J.device):
        status = _lib.lib().im_jtdj_mfma(
            M_dense.data_ptr(), J.data_ptr(), int(njmax), D.data_ptr(), state.data_ptr(),
            nefc.data_ptr() if nefc is not None else None, int(quad), H.data_ptr(), int(nv), int(H.shape[1]),
            int(nworld), int(torch.cuda.current_stream(J.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_jtdj_mfma")
