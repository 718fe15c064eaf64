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


def _matrix_tiles(m: Any):
    return m.M_tiles if hasattr(m, "M_tiles") else m.qM_tiles


def _has_m_structure(m: Any, d: Any = None) -> bool:
    return hasattr(m, "M_tiles") or (d is not None and hasattr(d, "M"))


def _has_sparse_m_tail(m: Any, d: Any) -> bool:
    """Whether an L'DL sparse tail follows the dense blocks of M (:783-787)."""
    if not hasattr(m, "qLD_block_total"):
        return bool(getattr(m, "qLD_has_sparse", False))
    shape = tuple(getattr(d.qLD, "shape", ()))
    return (int(shape[1]) if len(shape) > 1 else 0) > int(m.qLD_block_total)


def _element_count(tile) -> int:
    elemid = getattr(tile, "elemid", None)
    if elemid is None:
        return 0
    return int(elemid.numel()) if hasattr(elemid, "numel") else int(np.asarray(elemid).size)


def _device_ints(a, like):
    """int32 on ``like``'s device; a host array is uploaded at every call, which a stream capture
    does not allow: hand over device arrays (the reference's tiles hold them) to be capturable."""
    import torch

    if isinstance(a, torch.Tensor):
        return a.to(device=like.device, dtype=torch.int32).contiguous().reshape(-1)
    return torch.as_tensor(np.ascontiguousarray(np.asarray(a).reshape(-1), np.int32), device=like.device)


def _factor_solve_i_dense_no_l_store(m: Any, d: Any, M, x, y, D=None, *, upstream: Callable[..., None] | None = None) -> None:
    """Dense factor + solve when the factor is not used again (:790-846): one Cholesky tile per
    dense block of M, gathered through the tile's ``elemid`` where M is stored by its structure
    (``im_tile_cholesky_solve_m``) or read from the dense (nworld, nv, nv) array
    (``im_tile_cholesky_solve``).  A sparse tail behind the dense blocks, and M-structure tiles
    without an ``elemid`` (upstream's small-block kernel, which also writes ``d.qLD``), are
    upstream mujoco_warp code: ``upstream(False)`` is called for them."""
    import torch

    nworld = int(d.nworld)
    structured = _has_m_structure(m, d)
    tiles = list(_matrix_tiles(m))
    needs_upstream = structured and (_has_sparse_m_tail(m, d) or any(_element_count(t) == 0 for t in tiles))
    if needs_upstream:
        if upstream is None:
            raise NotImplementedError("a sparse tail or a block without element ids is solved by upstream's factor_solve_i")
        upstream(False)
        return
    for t in (M, x, y):
        if t.dtype != torch.float32 or not t.is_cuda or t.stride(-1) != 1 or t.device != M.device:
            raise ValueError("tile solve needs float32 CUDA tensors with contiguous rows on one device")
    x2, y2 = x.reshape(nworld, -1), y.reshape(nworld, -1)
    lib = _lib.lib()
    with torch.cuda.device(M.device):
        for tile in tiles:
            adr = _device_ints(tile.adr, M)
            size = int(tile.size)
            if structured:
                if M.dim() != 2 or M.shape[0] != nworld:
                    raise ValueError("M must be (nworld, nM)")
                ids = _device_ints(tile.elemid, M)
                if ids.numel() != adr.numel() * size * size:
                    raise ValueError("tile.elemid must hold size * size ids per block")
                status = lib.im_tile_cholesky_solve_m(
                    M.data_ptr(), M.stride(0), M.shape[1], ids.data_ptr(), adr.data_ptr(), adr.numel(), size,
                    y2.data_ptr(), y2.stride(0), x2.data_ptr(), x2.stride(0), nworld, _stream(M),
                )  # fmt: skip
                _lib.check(status, "im_tile_cholesky_solve_m")
            else:
                if M.dim() != 3 or M.shape[0] != nworld or M.stride(2) != 1:
                    raise ValueError("M must be (nworld, nv, nv) with contiguous rows")
                status = lib.im_tile_cholesky_solve(
                    M.data_ptr(), M.stride(0), M.stride(1), adr.data_ptr(), adr.numel(), size, y2.data_ptr(),
                    y2.stride(0), x2.data_ptr(), x2.stride(0), nworld, _stream(M),
                )  # fmt: skip
                _lib.check(status, "im_tile_cholesky_solve")


def factor_solve_i_no_l_store(m: Any, d: Any, M, L, D, x, y, tree_factor_solve=None, *,
                              upstream: Callable[..., None] | None = None) -> None:  # fmt: skip
    """Factor and solve without the dense factor as an output (:849-873): the tree L'DL when its
    scratch is given, upstream's factor for a sparse tail (``upstream(True)``: its solve reads
    ``L`` and ``D``), else the tile solve that keeps the factor on chip."""
    from . import tree_ldl

    if tree_factor_solve is not None:
        tree_ldl.tree_factor_solve(tree_factor_solve, M, x, y)
        return
    if _has_sparse_m_tail(m, d):
        if upstream is None:
            raise NotImplementedError("a sparse tail is factored by upstream's factor_solve_i")
        upstream(True)
        return
    _factor_solve_i_dense_no_l_store(m, d, M, x, y, D, upstream=upstream)


def _factor_solve_i_dense(
    m: Any, d: Any, M, x, y, dense_factor_solve: BlockedDenseFactorSolveScratch | None = None, *,
    retain_factor: bool = False, factor_workspace=None, tree_factor_solve=None,
    upstream: Callable[..., None] | None = None,
) -> None:  # fmt: skip
    """Dense factor + solve that prefers the tree L'DL when no factor is kept, then the blocked
    kernel when its scratch exists, then the single-tile solve: the reference's precedence and
    errors (:1030-1070).  Keeping the factor without a blocked scratch is upstream mujoco_warp's
    ``smooth.factor_solve_i`` (its ``qLD`` layout is not part of the reference's tree): pass it
    as ``upstream(retain_factor)``."""
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
    if retain_factor:
        if upstream is None:
            raise NotImplementedError("keeping the factor without a blocked scratch is upstream's factor_solve_i")
        upstream(True)
        return
    _factor_solve_i_dense_no_l_store(m, d, M, x, y, upstream=upstream)


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


def dense_init_factor(M, elemid, J, D, state, nefc, done, grad, H, U, search, search_dot, decrement, dof_union,
                      *, quad: int = QUADRATIC) -> bool:  # fmt: skip
    """The first Hessian of a dense Newton solve and its factor in one launch
    (``im_dense_init_factor``): ``H = M + J' D_act J`` from the tree-sparse ``M`` (nworld, nM) and
    ``elemid`` (nv, nv), then for the worlds that are not ``done`` the dense stage without changed
    rows (factor into ``U`` above 32 dofs, solve for ``grad``, ``search``, ``search_dot``,
    ``decrement``, an empty ``dof_union``).  Returns False, with nothing launched, for a shape
    the launch does not take (64 dofs and more) or arrays it cannot address; the caller then issues
    ``dense_from_csr``, :func:`dense_hessian` and the stage."""
    import torch

    nworld, njmax, nv = J.shape
    pad = int(H.shape[1])
    if nv > 32 and pad not in (48, 64):
        return False
    tensors = dict(M=M, J=J, D=D, state=state, grad=grad, H=H, U=U, search=search, search_dot=search_dot, decrement=decrement)
    for name, t in tensors.items():
        if not t.is_cuda or t.device != J.device or t.dtype != (torch.int32 if name == "state" else torch.float32):
            return False
    for t in (J, D, state, H, U, search_dot, decrement, elemid, dof_union):
        if not t.is_contiguous():
            return False
    if M.dim() != 2 or M.shape[0] != nworld or (M.shape[1] > 1 and M.stride(1) != 1) or grad.stride(-1) != 1 or search.stride(-1) != 1:
        return False
    if tuple(H.shape) != (nworld, pad, pad) or tuple(U.shape) != (nworld, pad, pad) or pad % 4 or H.data_ptr() % 16:
        return False
    if elemid.dtype != torch.int32 or tuple(elemid.shape) != (nv, nv) or dof_union.dtype != torch.int32 or tuple(dof_union.shape) != (nworld, nv + 1):
        return False
    if njmax < 1 or tuple(D.shape) != (nworld, njmax) or tuple(state.shape) != (nworld, njmax):
        return False
    if nefc is not None and (nefc.dtype != torch.int32 or nefc.numel() != nworld or not nefc.is_contiguous()):
        return False
    if done is not None and (done.dtype not in (torch.bool, torch.uint8) or done.numel() != nworld or not done.is_contiguous()):
        return False
    if grad.shape[0] != nworld or search.shape[0] != nworld or grad[0].numel() < nv or search[0].numel() < nv:
        return False
    with torch.cuda.device(J.device):
        status = _lib.lib().im_dense_init_factor(
            None if done is None else done.data_ptr(), None if nefc is None else nefc.data_ptr(), J.data_ptr(), int(njmax),
            D.data_ptr(), state.data_ptr(), int(quad), M.data_ptr(), int(M.stride(0)), elemid.data_ptr(), grad.data_ptr(),
            int(grad.stride(0)), H.data_ptr(), U.data_ptr(), int(nv), pad, dof_union.data_ptr(), search.data_ptr(),
            int(search.stride(0)), search_dot.data_ptr(), decrement.data_ptr(), int(nworld), _stream(J),
        )  # fmt: skip
    if status == _lib.IM_ERR_UNSUPPORTED:
        return False
    _lib.check(status, "im_dense_init_factor")
    return True


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
