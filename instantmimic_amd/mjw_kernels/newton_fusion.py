"""The product ``M v`` of the fused Newton kernel on MI355X.

The reference evaluates it inside its Newton loop, one dof per lane
(src/instantmimic/utils/mjw_kernels/newton_fusion.py:171-176), from three tables of the
upstream model (``m.M_mulm_rowadr``, ``m.M_mulm_col``, ``m.M_mulm_madr``, :378-380): for every
dof the columns of its full symmetric row and where each element sits in M's tree CSR.
:func:`mul_m` takes those tables as they are; :func:`mul_m_tables` builds them from the CSR
for a model that does not carry them (ancestors root first, the diagonal, then descendants
ascending -- the upstream order is not visible from the reference's tree).

The rest of that kernel (line search, gradient, convergence) is upstream mujoco_warp code and
is not part of this module.
"""

from __future__ import annotations

from typing import Any

import numpy as np

from .. import _lib


def mul_m_tables(rowadr, rownnz, colind):
    """(mulm_rowadr[nv + 1], mulm_col, mulm_madr) int32 for M's CSR (row = ancestors root
    first, diagonal last)."""
    rowadr, rownnz, colind = (np.asarray(a, np.int64) for a in (rowadr, rownnz, colind))
    nv = rowadr.size
    rows: list[list[tuple[int, int]]] = [[] for _ in range(nv)]
    for i in range(nv):
        for k in range(rowadr[i], rowadr[i] + rownnz[i]):
            rows[i].append((int(colind[k]), int(k)))
    for i in range(nv):  # descendants ascending: row i's off-diagonal entries mirrored
        for k in range(rowadr[i], rowadr[i] + rownnz[i] - 1):
            rows[int(colind[k])].append((i, int(k)))
    out_adr = np.zeros(nv + 1, np.int32)
    out_adr[1:] = np.cumsum([len(r) for r in rows])
    col = np.array([c for r in rows for c, _ in r], np.int32)
    madr = np.array([a for r in rows for _, a in r], np.int32)
    return out_adr, col, madr


def mul_m(M, vec, out, mulm_rowadr, mulm_col, mulm_madr, *, skip_world: Any = None) -> None:
    """``out[w] = M[w] vec[w]`` over the tables; worlds whose ``skip_world`` byte is set keep
    their row.  M (nworld, nM), vec and out (nworld, nv) float32 with contiguous rows; the
    tables int32 tensors on the same GPU."""
    import torch

    for t in (M, vec, out):
        if t.dtype != torch.float32 or not t.is_cuda:
            raise TypeError("mul_m needs float32 CUDA tensors")
        if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
            raise ValueError("mul_m needs rows of contiguous floats")
    for t in (mulm_rowadr, mulm_col, mulm_madr):
        if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
            raise TypeError("the row tables must be contiguous int32 CUDA tensors")
    nworld, nv = vec.shape
    if out.shape != vec.shape or M.shape[0] != nworld or mulm_rowadr.numel() != nv + 1 or mulm_madr.numel() != mulm_col.numel():
        raise ValueError("shapes of M, vec, out and the row table disagree")
    if skip_world is not None:
        if skip_world.dtype not in (torch.bool, torch.uint8) or skip_world.numel() != nworld or not skip_world.is_contiguous():
            raise TypeError("skip_world must be a contiguous bool or uint8 tensor with one element per world")
    with torch.cuda.device(M.device):
        status = _lib.lib().im_mul_m_sparse(
            M.data_ptr(), M.stride(0), int(M.shape[1]), mulm_rowadr.data_ptr(), mulm_col.data_ptr(),
            mulm_madr.data_ptr(), int(mulm_col.numel()), vec.data_ptr(), vec.stride(0), None if skip_world is None else skip_world.data_ptr(),
            out.data_ptr(), out.stride(0), int(nv), int(nworld), int(torch.cuda.current_stream(M.device).cuda_stream),
        )  # fmt: skip
    _lib.check(status, "im_mul_m_sparse")
