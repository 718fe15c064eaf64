"""Static-pattern sparse L'DL of the Newton Hessian ``H = M + J'DJ`` on MI355X.

Drop-in for the reference module ``instantmimic.utils.mjw_kernels.sparse_hessian``
(src/instantmimic/utils/mjw_kernels/sparse_hessian.py): the coupling pattern of the
model (:62-118), its symbolic factor and elimination levels (:192-212), the level /
run / backward tables of the numeric factor (:229-401) and the launcher of the initial
assemble + factor + solve (:804-846).  Here the tables are NumPy arrays handed to
``libimhip`` (the reference bakes them into generated CUDA source); the numeric kernel
is ``csrc/sparse_kernels.hip``.

Entries hold ``N = L D``; slots are row-major in elimination order (leaves first:
elimination index ``e = nv - 1 - dof``) so an entry's terms are runs of contiguous
slots; the right-hand side rides as an augmented last row.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Any, Sequence

import numpy as np

from .. import _lib

EQ_CONNECT, EQ_WELD, EQ_JOINT = 0, 1, 2
EQ_FLEX, EQ_FLEXVERT, EQ_FLEXSTRAIN = 4, 5, 6
OBJ_SITE = 6
MAX_SHARED_BYTES = 46 * 1024
MAX_DENSITY = 0.6
MIN_NV = 33
NONFUSED_MIN_NV = 80
QUADRATIC = 1  # mjtConstraintState.mjCNSTRSTATE_QUADRATIC
ROWS_PER_TILE = 4  # constraint rows per staged tile of the initial assembly


def _arr(a) -> np.ndarray:
    if a is None:
        return np.zeros(0, np.int64)
    if hasattr(a, "detach"):
        a = a.detach().cpu()
    if hasattr(a, "numpy"):
        a = a.numpy()
    return np.asarray(a)


def _chain(body, body_parentid, body_dofadr, body_dofnum) -> list[int]:
    out, b = [], int(body)
    while b > 0:
        out += range(int(body_dofadr[b]), int(body_dofadr[b]) + int(body_dofnum[b]))
        b = int(body_parentid[b])
    return out


def hessian_pattern(m: Any, body_groups: Sequence[Sequence[int]]) -> list[set[int]]:
    """Upper bound of H's off-diagonal pattern as dof adjacency (MuJoCo dof order):
    tree ancestry, cliques over the dof chains of every declared body group, equality
    constraints and native collision candidates."""
    nv = int(m.nv)
    dof_parentid = _arr(m.dof_parentid)
    body_parentid, body_dofadr, body_dofnum = _arr(m.body_parentid), _arr(m.body_dofadr), _arr(m.body_dofnum)
    adj = [set() for _ in range(nv)]
    for d in range(nv):
        p = int(dof_parentid[d])
        while p >= 0:
            adj[d].add(p)
            adj[p].add(d)
            p = int(dof_parentid[p])

    def clique(bodies):
        dofs = sorted({d for b in bodies for d in _chain(b, body_parentid, body_dofadr, body_dofnum)})
        for a in dofs:
            adj[a].update(x for x in dofs if x != a)

    for group in body_groups:
        clique(group)
    if int(getattr(m, "neq", 0)):
        eq_type, obj1, obj2 = _arr(m.eq_type), _arr(m.eq_obj1id), _arr(m.eq_obj2id)
        objtype, site_bodyid, jnt_dofadr = _arr(m.eq_objtype), _arr(m.site_bodyid), _arr(m.jnt_dofadr)
        for t, a, b, ot in zip(eq_type, obj1, obj2, objtype, strict=True):
            if t in (EQ_CONNECT, EQ_WELD):
                if ot == OBJ_SITE:
                    a, b = site_bodyid[a], site_bodyid[b]
                clique((a, max(int(b), 0)))
            elif t in (EQ_FLEX, EQ_FLEXVERT, EQ_FLEXSTRAIN):
                continue
            elif t == EQ_JOINT:
                dofs = [int(jnt_dofadr[a])] + ([int(jnt_dofadr[b])] if b >= 0 else [])
                for x in dofs:
                    adj[x].update(y for y in dofs if y != x)
            else:
                raise ValueError(f"equality type {int(t)} is not supported")
    if int(getattr(m, "nflex", 0)):
        raise ValueError("flex objects are not supported by this build")
    pairs = _arr(getattr(m, "nxn_geom_pair_filtered", None))
    if pairs.size:
        geom_bodyid = _arr(m.geom_bodyid)
        for g1, g2 in pairs.reshape(-1, 2):
            clique((geom_bodyid[g1], geom_bodyid[g2]))
    return adj


def _symbolic(adj_e: list[set[int]]):
    """Fill pattern and elimination levels of an L'DL in index order.  Returns
    ``rowstruct`` (earlier columns of each row), ``colstruct`` (later rows of each
    column) and ``levels`` (columns grouped by longest path in the elimination tree)."""
    n = len(adj_e)
    upper = [set(a for a in adj_e[k] if a > k) for k in range(n)]
    for k in range(n):
        nb = sorted(upper[k])
        for i, a in enumerate(nb):
            upper[a].update(nb[i + 1 :])
    colstruct = [sorted(upper[k]) for k in range(n)]
    rowstruct = [[] for _ in range(n)]
    for k in range(n):
        for i in colstruct[k]:
            rowstruct[i].append(k)
    parent = [c[0] if c else -1 for c in colstruct]
    level = [0] * n
    for k in range(n):
        if parent[k] >= 0:
            level[parent[k]] = max(level[parent[k]], level[k] + 1)
    levels = [[] for _ in range(max(level) + 1)]
    for k in range(n):
        levels[level[k]].append(k)
    return rowstruct, colstruct, levels


def _team(nentries: int, maxterms: int, lanes: int) -> int:
    """Lanes per entry of a level: the width minimising sweeps x (terms per lane +
    reduction steps)."""
    best, cost = 1, None
    for T in (1, 2, 4, 8, 16, 32):
        c = -(-nentries // (lanes // T)) * (-(-maxterms // T) + 2 * int(np.log2(T)))
        if cost is None or c < cost:
            best, cost = T, c
    return best


@dataclass
class SparseHessianPlan:
    nv: int
    nv_pad: int
    block: int
    nslots: int
    nterms: int
    levels: int
    density: float
    path: str
    tables: dict = field(repr=False, default_factory=dict)
    colstruct: list = field(repr=False, default_factory=list)
    level_cols: list = field(repr=False, default_factory=list)
    handle: Any = field(repr=False, default=None)

    @property
    def nfac(self) -> int:
        return self.nslots - self.nv


def build_tables(nv: int, nv_pad: int, adj: list[set[int]], M_rowi, M_colind, block: int, path: str = "fused") -> SparseHessianPlan:
    """The plan (tables only, no device state) of a dof adjacency."""
    orig = [nv - 1 - e for e in range(nv)]
    adj_e = [set(nv - 1 - a for a in adj[orig[e]]) for e in range(nv)]
    rowstruct, colstruct, levels = _symbolic(adj_e)
    n = nv
    slot = {}
    for i in range(n):
        for k in rowstruct[i]:
            slot[i, k] = len(slot)
        slot[i, i] = len(slot)
    nfac = len(slot)
    for k in range(n):
        slot[n, k] = len(slot)
    nslots = len(slot)
    if nslots >= 65536 or nfac + n > nv_pad * nv_pad:
        raise ValueError("sparse Hessian factor does not fit the packed layout")
    rs = [set(r) for r in rowstruct]
    lvl_ptr, lvl_team, ent_slot, ent_col, run_ptr, run_ab, run_kl = [0], [], [], [], [0], [], []
    nterms = 0
    for cols in levels:
        entries = []
        for j in cols:
            for i in [j, *colstruct[j], n]:
                ks = sorted(rs[j]) if i in (j, n) else sorted(rs[j] & rs[i])
                runs = []
                for k in ks:
                    last = runs[-1] if runs else None
                    if last and k == last[2] + last[3] and slot[i, k] == last[0] + last[3] and slot[j, k] == last[1] + last[3]:
                        last[3] += 1
                    else:
                        runs.append([slot[i, k], slot[j, k], k, 1])
                entries.append((slot[i, j], j if i == j else -1, runs, len(ks)))
        entries.sort(key=lambda e: -e[3])  # stable: longest entries first
        for s, c, runs, nt in entries:
            ent_slot.append(s)
            ent_col.append(c)
            for a, b, k, ln in runs:
                run_ab.append(a | (b << 16))
                run_kl.append(k | (ln << 16))
            run_ptr.append(len(run_ab))
            nterms += nt
        lvl_ptr.append(len(ent_slot))
        lvl_team.append(_team(len(entries), max(e[3] for e in entries), block))
    by_slot = sorted(((s, ij) for ij, s in slot.items() if s < nfac))
    gat = [min(orig[i], orig[j]) * nv_pad + max(orig[i], orig[j]) for _, (i, j) in by_slot]
    f_lvl, f_row = [0], []
    for cols in levels:
        f_row += cols
        f_lvl.append(len(f_row))
    row_start = [slot[j, rowstruct[j][0]] if rowstruct[j] else slot[j, j] for j in range(n)]
    rk_ptr, rk = [0], []
    for j in range(n):
        rk += rowstruct[j]
        rk_ptr.append(len(rk))
    b_lvl, b_slot, b_src, b_dst = [0], [], [], []
    for cols in reversed(levels):
        for i in cols:
            for j in rowstruct[i]:
                b_slot.append(slot[i, j])
                b_src.append(i)
                b_dst.append(j)
        b_lvl.append(len(b_slot))
    for a in (lvl_ptr, ent_slot, run_ptr, f_lvl, f_row, row_start, rk_ptr, rk, b_lvl, b_slot, b_src, b_dst):
        if max(a, default=0) >= 65536:
            raise ValueError("sparse Hessian tables exceed 16-bit indices")
    pair = [-1] * (nv * nv)
    for a in range(nv):
        for b in range(a, nv):
            i, j = nv - 1 - a, nv - 1 - b
            if (i, j) in slot and slot[i, j] < nfac:
                pair[a * nv + b] = slot[i, j]
    csr = {}
    for e, (r, c) in enumerate(zip(_arr(M_rowi), _arr(M_colind), strict=True)):
        csr[min(int(r), int(c)), max(int(r), int(c))] = e
    s_a, s_b, s_m = [], [], []
    for _, (i, j) in by_slot:
        a, b = sorted((orig[i], orig[j]))
        s_a.append(a)
        s_b.append(b)
        s_m.append(csr.get((a, b), -1))
    words = (nv + 31) // 32
    pmask = []
    for a in range(nv):
        bits = [0] * words
        for b in range(nv):
            if b == a or pair[min(a, b) * nv + max(a, b)] >= 0:
                bits[b // 32] |= 1 << (b % 32)
        pmask += bits
    if 2 * nfac + n >= nv_pad * nv_pad - 1:
        raise ValueError("packed H and factor do not fit hfactor")
    nw = max(block // 32, 1)
    init_tile = ROWS_PER_TILE * nv + ROWS_PER_TILE if path == "fused" else 0
    if 4 * (nslots + n + 2 * nw + init_tile) > MAX_SHARED_BYTES:
        raise ValueError("the factor does not fit the block's shared memory")
    i32 = lambda v: np.asarray(v if len(v) else [0], np.int32)  # noqa: E731
    tables = {
        "SH_LP": i32(lvl_ptr), "SH_LT": i32(lvl_team), "SH_ES": i32(ent_slot), "SH_EC": i32(ent_col),
        "SH_RP": i32(run_ptr), "SH_RAB": np.asarray(run_ab if run_ab else [0], np.uint32).view(np.int32),
        "SH_RKL": np.asarray(run_kl if run_kl else [0], np.uint32).view(np.int32), "SH_ORIG": i32(orig),
        "SH_BL": i32(b_lvl), "SH_BS": i32(b_slot), "SH_BI": i32(b_src), "SH_BJ": i32(b_dst), "SH_PAIR": i32(pair),
        "SH_FL": i32(f_lvl), "SH_FR": i32(f_row), "SH_RS": i32(row_start), "SH_RKP": i32(rk_ptr), "SH_RK": i32(rk),
        "SH_PM": np.asarray(pmask, np.uint32).view(np.int32), "SH_SA": i32(s_a), "SH_SB": i32(s_b), "SH_SM": i32(s_m),
        "SH_GAT": i32(gat),
    }  # fmt: skip
    return SparseHessianPlan(
        nv, nv_pad, block, nslots, nterms, len(levels), nfac / (nv * (nv + 1) / 2), path, tables, colstruct, levels
    )


def _rowi(m) -> np.ndarray:
    if getattr(m, "M_hinit_i", None) is not None:
        return _arr(m.M_hinit_i)
    return np.repeat(np.arange(int(m.nv)), _arr(m.M_rownnz))


class _DevicePlan:
    """Owns the ``im_sparse_plan`` of a table set on the current device."""

    ORDER = ("SH_LP", "SH_LT", "SH_ES", "SH_EC", "SH_RP", "SH_RAB", "SH_RKL", "SH_ORIG", "SH_BL", "SH_BS", "SH_BI",
             "SH_BJ", "SH_PM", "SH_SA", "SH_SB", "SH_SM", "SH_PAIR", "SH_FL", "SH_FR", "SH_RS", "SH_RKP",
             "SH_RK")  # fmt: skip

    def __init__(self, plan: SparseHessianPlan):
        arrays = [np.ascontiguousarray(plan.tables[k], np.int32) for k in self.ORDER]
        ptrs = (C.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
        sizes = (C.c_int * len(arrays))(*[a.size for a in arrays])
        handle = C.c_void_p()
        status = _lib.lib().im_sparse_plan_create(
            plan.nv, plan.nv_pad, plan.block, plan.nslots, plan.levels, len(arrays), ptrs, sizes, C.byref(handle)
        )
        _lib.check(status, "im_sparse_plan_create")
        self.ptr = handle

    def __del__(self):
        ptr, self.ptr = getattr(self, "ptr", None), None
        if ptr:
            try:
                _lib.lib().im_sparse_plan_destroy(ptr)
            except Exception:
                pass


def build_plan(m: Any, body_groups: Sequence[Sequence[int]], block: int, path: str = "fused", *, device=None) -> SparseHessianPlan:
    """Tables of the model's pattern; with ``device`` also the device-side plan."""
    plan = build_tables(int(m.nv), int(m.nv_pad), hessian_pattern(m, body_groups), _rowi(m), m.M_colind, block, path)
    if device is not None:
        import torch

        with torch.cuda.device(torch.device(device)):
            plan.handle = _DevicePlan(plan)
    return plan


def block_width(nv_pad: int) -> int:
    """Block width of the fused Newton (newton_fusion.py:325-327)."""
    return 64 if nv_pad >= 64 else 32


def plan_for_model(m: Any, ctx: Any, body_groups, block: int, *, compact: bool = False, fused_runtime: bool = True, device="cuda"):
    """The plan when the model qualifies, else ``None`` and the reason (same order of
    checks and same messages as the reference, sparse_hessian.py:705-758).  Only the
    fused path exists in this build."""
    if body_groups is None:
        return None, "a custom contact producer did not declare its body groups"
    if int(m.nv) < MIN_NV:
        return None, f"nv {int(m.nv)} < {MIN_NV}"
    if int(getattr(m, "ntendon", 0)) and (
        int(_arr(getattr(m, "tendon_limited_adr", None)).shape[0]) or bool((_arr(m.tendon_frictionloss) > 0).any())
    ):
        return None, "tendon limit or frictionloss rows"
    if not fused_runtime or compact or int(m.nv) > 79:
        return None, "Newton solver structure not supported"
    if int(getattr(m, "nflex", 0)):
        return None, "flex objects on the fused path"
    try:
        plan = build_plan(m, body_groups, block, "fused", device=device)
    except ValueError as exc:
        return None, str(exc)
    if plan.density > MAX_DENSITY:
        return None, f"pattern density {plan.density:.2f} > {MAX_DENSITY}"
    return plan, "enabled"


def violation_counter(hfactor, plan: SparseHessianPlan):
    """Per-world view of the pattern-violation counter, the last element of each world's
    ``hfactor``; accumulates until it is zeroed."""
    if plan.path != "fused":
        raise ValueError("the violation counter exists on the fused path only")
    last = plan.nv_pad - 1
    return hfactor[:, last, last]


def violations(hfactor, plan: SparseHessianPlan) -> np.ndarray:
    return violation_counter(hfactor, plan).cpu().numpy()


def init_factor_kernel(plan: SparseHessianPlan):
    """Launcher of the initial ``H = M + J'DJ`` on the pattern, factor and solve; fills
    ``hfactor``, ``search = -H^-1 grad``, ``search_dot`` and ``decrement``.  Called with
    the reference kernel's arguments
    ``(done, nefc, J, D, state, M, grad3, hfactor, search3, search_dot, decrement)``."""
    if plan.handle is None:
        raise RuntimeError("the plan has no device state (build it with device=...)")

    def launch(done, nefc, J, D, state, M, grad, hfactor, search, search_dot, decrement, *, quad: int = QUADRATIC):
        import torch

        nworld, njmax, nv = J.shape
        if nv != plan.nv or tuple(hfactor.shape) != (nworld, plan.nv_pad, plan.nv_pad):
            raise ValueError("array shapes do not match the plan")
        for t in (J, D, state, M, grad, hfactor, search, search_dot, decrement, nefc):
            if not t.is_cuda or not t.is_contiguous():
                raise ValueError("arrays must be contiguous CUDA tensors")
        done_ptr = None
        if done is not None:
            if done.dtype not in (torch.bool, torch.uint8):
                raise TypeError("done must be a bool tensor")
            done_ptr = done.data_ptr()
        with torch.cuda.device(J.device):
            status = _lib.lib().im_sparse_init_factor(
                plan.handle.ptr, done_ptr, nefc.data_ptr(), J.data_ptr(), int(njmax), D.data_ptr(), state.data_ptr(),
                int(quad), M.data_ptr(), int(M.shape[1]), grad.data_ptr(), int(grad.shape[1]), hfactor.data_ptr(),
                search.data_ptr(), search_dot.data_ptr(), decrement.data_ptr(), int(nworld),
                int(torch.cuda.current_stream(J.device).cuda_stream),
            )  # fmt: skip
        _lib.check(status, "im_sparse_init_factor")

    return launch


def pattern_misses(h: np.ndarray, plan_adj: list[set[int]], tol: float = 0.0) -> int:
    """Nonzero upper-triangle entries of dense Hessians ``h`` (nworld, nv_pad, nv_pad)
    outside a dof adjacency."""
    nv = len(plan_adj)
    mask = np.eye(nv, dtype=bool)
    for a in range(nv):
        for b in plan_adj[a]:
            mask[a, b] = True
    off = np.triu(np.ones((nv, nv), bool)) & ~mask
    return int((np.abs(h[:, :nv, :nv][:, off]) > tol).sum())
