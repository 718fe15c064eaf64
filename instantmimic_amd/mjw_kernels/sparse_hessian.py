"""Static-pattern sparse L'DL of the Newton Hessian ``H = M + J'DJ`` on MI355X.

Drop-in for the reference module ``instantmimic.utils.mjw_kernels.sparse_hessian``
(src/instantmimic/utils/mjw_kernels/sparse_hessian.py).  This module only marshals: it reads
the model's arrays, names the sources of constraint rows to the library's pattern builder
(:62-171), asks the library for the plan (symbolic factor, levels, tables: :192-401) and
launches the numeric kernels (:804-894).  The planning itself is ``csrc/sparse_plan.cpp``, the
kernels ``csrc/sparse_kernels.hip``; the reference bakes its tables into generated CUDA
source, here they are device arrays owned by the plan handle.

Entries hold ``N = L D``; slots are row-major in elimination order (leaves first:
elimination index ``e = nv - 1 - dof``); the right-hand side rides as an augmented last row.
"""

from __future__ import annotations

import ctypes as C
from typing import Any, Iterable, Iterator, Sequence

import numpy as np

from .. import _lib

EQ_CONNECT, EQ_WELD, EQ_JOINT = 0, 1, 2
EQ_FLEX, EQ_FLEXVERT, EQ_FLEXSTRAIN = 4, 5, 6
OBJ_SITE = 6
MAX_DENSITY = 0.6  # sparse_hessian.py:183
MIN_NV = 33  # :184
NONFUSED_MIN_NV = 80  # :189
QUADRATIC = 1  # mjtConstraintState.mjCNSTRSTATE_QUADRATIC
PATHS = {"fused": 0, "nonfused": 1}
REFUSALS = {
    1: "sparse Hessian factor does not fit the packed layout",
    2: "sparse Hessian tables exceed 16-bit indices",
    3: "packed H and factor do not fit hfactor",
    4: "the factor does not fit the block's shared memory",
}


def _host(a, dtype=np.int32) -> np.ndarray:
    """A model array (NumPy, torch or anything with ``numpy()``) as a contiguous host array."""
    if a is None:
        return np.zeros(0, dtype)
    if hasattr(a, "detach"):
        a = a.detach().cpu()
    if hasattr(a, "numpy"):
        a = a.numpy()
    return np.ascontiguousarray(np.asarray(a), dtype)


class DofPattern:
    """Owns an ``im_dof_pattern``; reads like the reference's ``list[set[int]]`` adjacency
    (``len(p)``, ``p[dof]`` = set of coupled dofs)."""

    def __init__(self, m: Any):
        self.nv = int(m.nv)
        handle = C.c_void_p()
        arrays = [_host(getattr(m, k)) for k in ("dof_parentid", "body_parentid", "body_dofadr", "body_dofnum")]
        status = _lib.lib().im_dof_pattern_create(
            self.nv, arrays[0].ctypes.data, int(arrays[1].size), *[a.ctypes.data for a in arrays[1:]], C.byref(handle)
        )
        _lib.check(status, "im_dof_pattern_create")
        self.ptr = handle
        self._dense = None

    def __del__(self):
        ptr, self.ptr = getattr(self, "ptr", None), None
        if ptr:
            try:
                _lib.lib().im_dof_pattern_destroy(ptr)
            except Exception:
                pass

    def couple_bodies(self, bodies: Iterable[int]) -> None:
        ids = np.fromiter((int(b) for b in bodies), np.int32)
        self._dense = None
        _lib.check(_lib.lib().im_dof_pattern_couple_bodies(self.ptr, ids.ctypes.data, int(ids.size)), "im_dof_pattern_couple_bodies")

    def couple_dofs(self, dofs: Iterable[int]) -> None:
        ids = np.fromiter((int(d) for d in dofs), np.int32)
        self._dense = None
        _lib.check(_lib.lib().im_dof_pattern_couple_dofs(self.ptr, ids.ctypes.data, int(ids.size)), "im_dof_pattern_couple_dofs")

    def dense(self) -> np.ndarray:
        """(nv, nv) bool, True where two different dofs couple."""
        if self._dense is None:
            out = np.zeros((self.nv, self.nv), np.uint8)
            _lib.check(_lib.lib().im_dof_pattern_get(self.ptr, out.ctypes.data), "im_dof_pattern_get")
            self._dense = out.astype(bool)
        return self._dense

    def __len__(self) -> int:
        return self.nv

    def __getitem__(self, dof: int) -> set[int]:
        return set(np.flatnonzero(self.dense()[dof]).tolist())

    def __iter__(self) -> Iterator[set[int]]:
        return (self[d] for d in range(self.nv))


def _equality_sources(m: Any):
    """(kind, ids) per equality constraint: the two bodies a connect / weld ties together (a
    missing second object is the world), or the dofs a joint equality ties (:90-109)."""
    kinds = _host(m.eq_type)
    first, second, objtype = _host(m.eq_obj1id), _host(m.eq_obj2id), _host(m.eq_objtype)
    site_body, joint_dof = _host(getattr(m, "site_bodyid", None)), _host(getattr(m, "jnt_dofadr", None))
    if not (kinds.size == first.size == second.size == objtype.size):
        raise ValueError("equality arrays differ in length")
    for q in range(kinds.size):
        kind, a, b = int(kinds[q]), int(first[q]), int(second[q])
        if kind in (EQ_FLEX, EQ_FLEXVERT, EQ_FLEXSTRAIN):
            continue  # these rows stay inside the flex couplings
        if kind == EQ_JOINT:
            yield "dofs", [int(joint_dof[a])] + ([int(joint_dof[b])] if b >= 0 else [])
        elif kind in (EQ_CONNECT, EQ_WELD):
            if int(objtype[q]) == OBJ_SITE:
                a, b = int(site_body[a]), int(site_body[b])
            yield "bodies", (a, max(b, 0))
        else:
            raise ValueError(f"equality type {kind} is not supported")


def _flex_sources(m: Any):
    """Body sets one flex row can couple (:121-170): the vertex bodies of an element (or all
    nodes of an interpolated flex), an element together with the body of a geom it may touch,
    and two flexes that may collide (a flex with itself when it self-collides) as a whole."""
    nflex = int(m.nflex)
    vert_body, node_body = _host(m.flex_vertbodyid), _host(getattr(m, "flex_nodebodyid", None))
    vertadr, vertnum = _host(m.flex_vertadr), _host(m.flex_vertnum)
    elemnum, dataadr, dim = _host(m.flex_elemnum), _host(m.flex_elemdataadr), _host(m.flex_dim)
    elem, interp = _host(m.flex_elem), _host(m.flex_interp)
    nodeadr, nodenum = _host(getattr(m, "flex_nodeadr", None)), _host(getattr(m, "flex_nodenum", None))
    whole: list[tuple[int, ...]] = []  # every body of flex f
    pieces: list[list[tuple[int, ...]]] = []  # distinct element body sets of flex f
    for f in range(nflex):
        if interp[f]:
            nodes = tuple(int(b) for b in node_body[nodeadr[f] : nodeadr[f] + nodenum[f]])
            whole.append(nodes)
            pieces.append([nodes] if elemnum[f] else [])
            yield nodes
            continue
        mine = vert_body[vertadr[f] : vertadr[f] + vertnum[f]]
        whole.append(tuple(int(b) for b in mine))
        corners = elem[dataadr[f] : dataadr[f] + int(elemnum[f]) * (int(dim[f]) + 1)].reshape(int(elemnum[f]), int(dim[f]) + 1)
        distinct = list(dict.fromkeys(tuple(int(b) for b in mine[row]) for row in corners))
        pieces.append(distinct)
        yield from distinct
    contype, conaff = _host(m.flex_contype), _host(m.flex_conaffinity)
    gtype, gaff, geom_body = _host(m.geom_contype), _host(m.geom_conaffinity), _host(m.geom_bodyid)
    for f in range(nflex):
        touching = np.flatnonzero((contype[f] & gaff[: int(m.ngeom)]) | (gtype[: int(m.ngeom)] & conaff[f]))
        for body in dict.fromkeys(int(geom_body[g]) for g in touching):
            for piece in pieces[f]:
                yield (*piece, body)
    selfcollide = _host(m.flex_selfcollide)
    for f in range(nflex):
        for h in range(f, nflex):
            if ((contype[f] & conaff[h]) or (contype[h] & conaff[f])) and (f != h or selfcollide[f]):
                yield whole[f] + whole[h]


def hessian_pattern(m: Any, body_groups: Sequence[Sequence[int]]) -> DofPattern:
    """Upper bound of H's off-diagonal pattern (dof adjacency, MuJoCo dof order): tree
    ancestry, then one clique per declared body group, equality constraint, flex coupling and
    native collision candidate (:62-118)."""
    pattern = DofPattern(m)
    for group in body_groups:
        pattern.couple_bodies(group)
    if int(getattr(m, "neq", 0)):
        for kind, ids in _equality_sources(m):
            (pattern.couple_dofs if kind == "dofs" else pattern.couple_bodies)(ids)
    if int(getattr(m, "nflex", 0)):
        for bodies in _flex_sources(m):
            pattern.couple_bodies(bodies)
    pairs = _host(getattr(m, "nxn_geom_pair_filtered", None)).reshape(-1, 2)
    if pairs.size:
        geom_body = _host(m.geom_bodyid)
        for b1, b2 in dict.fromkeys(map(tuple, geom_body[pairs].tolist())):
            pattern.couple_bodies((b1, b2))
    return pattern


class SparseHessianPlan:
    """The reference's ``SparseHessianPlan`` (:38-50) over an ``im_sparse_plan`` handle; the
    generated-source fields are replaced by the handle, ``tables`` reads the SH_* arrays back."""

    def __init__(self, ptr, on_device: bool):
        self.ptr = ptr
        info = _lib.SparsePlanInfo()
        _lib.check(_lib.lib().im_sparse_plan_get_info(ptr, C.byref(info)), "im_sparse_plan_get_info")
        self.nv, self.nv_pad, self.block = int(info.nv), int(info.nv_pad), int(info.block)
        self.nslots, self.nterms, self.levels = int(info.nslots), int(info.nterms), int(info.nlevels)
        self.nfac = int(info.nfac)
        self.density = float(info.density)
        self.path = "fused" if info.path == PATHS["fused"] else "nonfused"
        self.device_ready = bool(info.device_ready)
        self.handle = self if (on_device and self.device_ready) else None
        self._tables = None

    def __del__(self):
        ptr, self.ptr = getattr(self, "ptr", None), None
        if ptr:
            try:
                _lib.lib().im_sparse_plan_destroy(ptr)
            except Exception:
                pass

    def __repr__(self) -> str:
        return (f"SparseHessianPlan(nv={self.nv}, nv_pad={self.nv_pad}, block={self.block}, nslots={self.nslots}, "
                f"nterms={self.nterms}, levels={self.levels}, density={self.density:.3f}, path={self.path!r})")  # fmt: skip

    @property
    def tables(self) -> dict[str, np.ndarray]:
        if self._tables is None:
            lib, out = _lib.lib(), {}
            for tid, name in enumerate(_lib.SPARSE_TABLES):
                arr = np.zeros(lib.im_sparse_plan_table_size(self.ptr, tid), np.int32)
                _lib.check(lib.im_sparse_plan_get_table(self.ptr, tid, arr.ctypes.data, int(arr.size)), "im_sparse_plan_get_table")
                out[name] = arr
            self._tables = out
        return self._tables

    def _structure(self):
        ptr, idx, lvl = np.zeros(self.nv + 1, np.int32), np.zeros(max(self.nfac - self.nv, 1), np.int32), np.zeros(self.nv, np.int32)
        _lib.check(_lib.lib().im_sparse_plan_get_structure(self.ptr, ptr.ctypes.data, idx.ctypes.data, lvl.ctypes.data), "im_sparse_plan_get_structure")
        return ptr, idx, lvl

    @property
    def colstruct(self) -> list[list[int]]:
        """Fill pattern: the later rows of every column of the factor, elimination indices."""
        ptr, idx, _ = self._structure()
        return [idx[ptr[k] : ptr[k + 1]].tolist() for k in range(self.nv)]

    @property
    def level_cols(self) -> list[list[int]]:
        _, _, lvl = self._structure()
        return [np.flatnonzero(lvl == q).tolist() for q in range(self.levels)]


def _rowi(m) -> np.ndarray:
    if getattr(m, "M_hinit_i", None) is not None:
        return _host(m.M_hinit_i)
    return np.repeat(np.arange(int(m.nv), dtype=np.int32), _host(m.M_rownnz))


def plan_from_pattern(pattern: DofPattern, nv_pad: int, M_rowi, M_colind, block: int, path: str = "fused", *, device=None) -> SparseHessianPlan:
    """The plan of a dof pattern; ``device=None`` plans on the host only (no GPU needed).
    Raises ``ValueError`` with the reference's messages when the factor exceeds its limits."""
    rowi, colind = _host(M_rowi), _host(M_colind)
    if rowi.size != colind.size:
        raise ValueError("M_rowi and M_colind differ in length")
    handle, refused = C.c_void_p(), C.c_int(0)

    def call():
        return _lib.lib().im_sparse_plan_build(
            pattern.ptr, int(nv_pad), int(block), PATHS[path], rowi.ctypes.data, colind.ctypes.data, int(rowi.size),
            int(device is None), C.byref(refused), C.byref(handle),
        )  # fmt: skip

    if device is None:
        status = call()
    else:
        import torch

        with torch.cuda.device(torch.device(device)):
            status = call()
    _lib.check(status, "im_sparse_plan_build")
    if not handle:
        raise ValueError(REFUSALS[refused.value])
    return SparseHessianPlan(handle, device is not None)


def build_plan(m: Any, body_groups: Sequence[Sequence[int]], block: int, path: str = "fused", *, device=None) -> SparseHessianPlan:
    """``build_plan`` of the reference (:229-702) for a model."""
    return plan_from_pattern(hessian_pattern(m, body_groups), int(m.nv_pad), _rowi(m), m.M_colind, block, path, device=device)


def block_width(nv_pad: int) -> int:
    """Block width of the fused Newton (newton_fusion.py:325-327)."""
    return 64 if nv_pad >= 64 else 32


def _on_gpu(m: Any, device) -> bool:
    arr = getattr(m, "body_parentid", None)
    dev = None if isinstance(arr, np.ndarray) else getattr(arr, "device", None)  # host-side NumPy copies say nothing
    if dev is not None:
        return bool(getattr(dev, "is_cuda", False) or getattr(dev, "type", "") == "cuda")
    return True if device is None else str(device).startswith("cuda")


def plan_for_model(m: Any, ctx: Any, body_groups, block: int, *, compact: bool = False, fused_runtime: bool = True, device="cuda"):
    """The plan when the model qualifies, else ``None`` and the reason: the reference's checks in
    the reference's order with its messages (:705-758).  ``device=None`` plans on the host and
    skips nothing but the upload; a model whose arrays say where they live is judged by that."""
    from . import newton_fusion

    nv = int(m.nv)
    if body_groups is None:
        return None, "a custom contact producer did not declare its body groups"
    if not _on_gpu(m, device):
        return None, "fused Newton not eligible (CPU)"
    if nv < MIN_NV:
        return None, f"nv {nv} < {MIN_NV}"
    if int(getattr(m, "ntendon", 0)) and (
        int(_host(getattr(m, "tendon_limited_adr", None)).shape[0]) or bool((_host(m.tendon_frictionloss, np.float32) > 0).any())
    ):
        return None, "tendon limit or frictionloss rows"
    if fused_runtime and newton_fusion.eligible(m, ctx, compact=compact, device=device):
        if int(getattr(m, "nflex", 0)):
            return None, "flex objects on the fused path"
        path, width = "fused", block
    elif newton_fusion.upstream_newton_structure(m, ctx, compact=compact):
        if nv < NONFUSED_MIN_NV:
            return None, f"upstream iteration with nv {nv} < {NONFUSED_MIN_NV}"
        path, width = "nonfused", 64 if nv <= 96 else 128
    else:
        return None, "Newton solver structure not supported"
    try:
        plan = build_plan(m, body_groups, width, path, device=device)
    except ValueError as exc:
        return None, str(exc)
    if plan.density > MAX_DENSITY:
        return None, f"pattern density {plan.density:.2f} > {MAX_DENSITY}"
    return plan, "enabled"


def violation_counter(hfactor, plan):
    """Per-world view of the pattern-violation counter, the last element of each world's
    ``hfactor``; accumulates until it is zeroed (:786-796)."""
    if plan.path != "fused":
        raise ValueError("the violation counter exists on the fused path only")
    last = plan.nv_pad - 1
    return hfactor[:, last, last]


def violations(hfactor, plan) -> np.ndarray:
    return violation_counter(hfactor, plan).cpu().numpy()


def _device_plan(plan: SparseHessianPlan):
    if plan.handle is None:
        raise RuntimeError("the plan has no device state (build it with device=...)")
    return plan.ptr


def init_factor_kernel(plan: SparseHessianPlan):
    """Launcher of the initial ``H = M + J'DJ`` on the pattern, factor and solve; fills
    ``hfactor``, ``search = -H^-1 grad``, ``search_dot`` and ``decrement``.  Called with
    the reference kernel's arguments
    ``(done, nefc, J, D, state, M, grad3, hfactor, search3, search_dot, decrement)`` (:804-846)."""
    ptr = _device_plan(plan)
    if plan.path != "fused":
        raise ValueError("the initial assemble + factor exists on the fused path only")

    def launch(done, nefc, J, D, state, M, grad, hfactor, search, search_dot, decrement, *, quad: int = QUADRATIC):
        import torch

        nworld, njmax, nv = J.shape
        if nv != plan.nv or tuple(hfactor.shape) != (nworld, plan.nv_pad, plan.nv_pad):
            raise ValueError("array shapes do not match the plan")
        if tuple(D.shape) != (nworld, njmax) or tuple(state.shape) != (nworld, njmax) or nefc.numel() != nworld:
            raise ValueError("D, state and nefc do not match J")
        if M.shape[0] != nworld or grad.shape[0] != nworld or grad[0].numel() < nv or search[0].numel() != nv:
            raise ValueError("M, grad and search do not match J")
        for t in (J, D, state, M, grad, hfactor, search, search_dot, decrement, nefc):
            if not t.is_cuda or not t.is_contiguous() or t.device != J.device:
                raise ValueError("arrays must be contiguous CUDA tensors on one device")
        done_ptr = None
        if done is not None:
            if done.dtype not in (torch.bool, torch.uint8) or done.numel() != nworld:
                raise TypeError("done must be a bool tensor with one element per world")
            done_ptr = done.data_ptr()
        with torch.cuda.device(J.device):
            status = _lib.lib().im_sparse_init_factor(
                ptr, done_ptr, nefc.data_ptr(), J.data_ptr(), int(njmax), D.data_ptr(), state.data_ptr(),
                int(quad), M.data_ptr(), int(M.shape[1]), grad.data_ptr(), int(grad[0].numel()), hfactor.data_ptr(),
                search.data_ptr(), search_dot.data_ptr(), decrement.data_ptr(), int(nworld),
                int(torch.cuda.current_stream(J.device).cuda_stream),
            )  # fmt: skip
        _lib.check(status, "im_sparse_init_factor")

    return launch


def nonfused_kernel(plan: SparseHessianPlan, skip_unchanged: bool, skip_noflip: bool):
    """Launcher of the upstream iteration's factor step with the sparse factor: refactor from the
    dense Hessian when rows changed QUADRATIC state (always without ``skip_unchanged``), else
    solve with the stored factor; ``skip_noflip`` leaves worlds without state changes alone.
    Called with the reference kernel's arguments
    ``(done, grad3, H, quad_changed, state_changed, hfactor, search3, search_dot, decrement)`` (:849-894)."""
    ptr = _device_plan(plan)
    if plan.path != "nonfused":
        raise ValueError("the upstream-iteration factor needs a plan of the nonfused path")
    skip_unchanged, skip_noflip = bool(skip_unchanged), bool(skip_noflip)

    def launch(done, grad, H, quad_changed, state_changed, hfactor, search, search_dot, decrement):
        import torch

        nworld = int(H.shape[0])
        if tuple(H.shape) != (nworld, plan.nv_pad, plan.nv_pad) or tuple(hfactor.shape) != tuple(H.shape):
            raise ValueError("H and hfactor must be (nworld, nv_pad, nv_pad)")
        if grad.shape[0] != nworld or grad[0].numel() < plan.nv or search.shape[0] != nworld or search[0].numel() < plan.nv:
            raise ValueError("grad and search do not match the plan")
        for t in (grad, H, hfactor, search, search_dot, decrement):
            if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous() or t.device != H.device:
                raise ValueError("arrays must be contiguous float32 CUDA tensors on one device")
        ptrs = []
        for t, name, dtypes, needed in ((done, "done", (torch.bool, torch.uint8), False),
                                        (quad_changed, "quad_changed", (torch.int32,), skip_unchanged),
                                        (state_changed, "state_changed", (torch.int32,), skip_noflip)):  # fmt: skip
            if t is None:
                if needed:
                    raise ValueError(f"{name} is needed with this kernel's skip flags")
                ptrs.append(None)
                continue
            if t.dtype not in dtypes or t.numel() != nworld or not t.is_cuda or not t.is_contiguous():
                raise TypeError(f"{name} must be a contiguous CUDA tensor with one element per world")
            ptrs.append(t.data_ptr())
        with torch.cuda.device(H.device):
            status = _lib.lib().im_sparse_dense_factor(
                ptr, ptrs[0], grad.data_ptr(), int(grad[0].numel()), H.data_ptr(), int(H.stride(0)), ptrs[1], ptrs[2],
                int(skip_unchanged), int(skip_noflip), hfactor.data_ptr(), search.data_ptr(), int(search[0].numel()),
                search_dot.data_ptr(), decrement.data_ptr(), nworld, int(torch.cuda.current_stream(H.device).cuda_stream),
            )  # fmt: skip
        _lib.check(status, "im_sparse_dense_factor")

    return launch


def nonfused_solver_functions(plan: SparseHessianPlan):
    """``cholesky_factorize_solve(m, d, ctx, skip_unchanged=False, skip_noflip=False)``: the
    function the reference substitutes for upstream's ``_cholesky_factorize_solve`` (:909-942),
    reading ``ctx.done, grad, h, quad_changed_count, state_changed_count, hfactor, search,
    search_dot, newton_decrement``.  Upstream's ``_update_gradient`` / ``_solver_iteration``,
    which the reference rebinds around it, are third-party code and stay the caller's."""
    kernels = {}

    def cholesky_factorize_solve(m, d, ctx, skip_unchanged=False, skip_noflip=False):
        key = (bool(skip_unchanged), bool(skip_noflip))
        if key not in kernels:
            kernels[key] = nonfused_kernel(plan, *key)
        state = ctx.state_changed_count if skip_noflip else ctx.quad_changed_count
        nworld = int(d.nworld)
        kernels[key](
            ctx.done, ctx.grad.reshape(nworld, ctx.grad.shape[1], 1), ctx.h, ctx.quad_changed_count, state, ctx.hfactor,
            ctx.search.reshape(nworld, int(m.nv), 1), ctx.search_dot, ctx.newton_decrement,
        )  # fmt: skip

    return cholesky_factorize_solve


def pattern_misses(h: np.ndarray, plan_adj, tol: float = 0.0) -> int:
    """Nonzero upper-triangle entries of dense Hessians ``h`` (nworld, nv_pad, nv_pad)
    outside a dof adjacency (:946-957)."""
    if isinstance(plan_adj, DofPattern):
        allowed = plan_adj.dense().copy()
    else:
        allowed = np.zeros((len(plan_adj), len(plan_adj)), bool)
        for a, neighbours in enumerate(plan_adj):
            allowed[a, list(neighbours)] = True
    nv = allowed.shape[0]
    np.fill_diagonal(allowed, True)
    outside = np.triu(~allowed)
    return int((np.abs(h[:, :nv, :nv][:, outside]) > tol).sum())
