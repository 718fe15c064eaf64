"""Integer planning of the tree L'DL, restated from the reference (oracle only).

Follows src/instantmimic/utils/mjw_kernels/tree_ldl.py of the reference:

* ``tree_ldl_structure``    :66-91   nested-ancestor CSR validation
* ``shared_bytes``          :94-102  trunk exchange footprint of the CUDA kernel
* ``plan_tree_ldl``         :105-170 trunk / parts cut and LPT packing
* ``best_tree_ldl_plan``    :173-185 best over 1..4 groups under the 48 KB cap
* ``tree_ldl_beats_dense``  :188-193 eligibility rule
* ``elimination_order``     :256-257, 290  order in which dofs are eliminated

Pinned by: the invariants the reference's tests hold
(tests/test_tree_ldl.py:123-161), hand-derivable closed forms (one group means
an empty trunk and span = sum of costs) and the expected plans recorded for the
five benchmark trees (tests/golden/tree_plans.json).
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np

MAX_GROUPS = 4
MAX_SHARED_BYTES = 48 * 1024
MAX_SHORT_SPAN = 4096
MIN_DENSE_TO_SPAN_RATIO = 8.0


@dataclass(frozen=True)
class Plan:
    groups: tuple  # tuple of tuples, dofs descending
    trunk: tuple  # ascending
    span: int
    dense_cost: int


def tree_ldl_structure(rowadr, rownnz, colind):
    """CSR as three tuples if every row is ``ancestors root-first + diagonal``
    and each ancestor's row is a prefix of it; otherwise ``None``."""
    rowadr = np.asarray(rowadr, dtype=np.int64)
    rownnz = np.asarray(rownnz, dtype=np.int64)
    colind = np.asarray(colind, dtype=np.int64)
    nv = rowadr.size
    if nv == 0 or rownnz.size != nv or (rownnz < 1).any():
        return None
    if (rowadr + rownnz > colind.size).any():
        return None
    for k in range(nv):
        row = colind[rowadr[k] : rowadr[k] + rownnz[k]]
        if row[-1] != k:
            return None
        if (row[:-1] >= k).any():
            return None
        for p in range(len(row) - 1):
            i = row[p]
            if rownnz[i] != p + 1:
                return None
            if not np.array_equal(colind[rowadr[i] : rowadr[i] + rownnz[i]], row[: p + 1]):
                return None
    return (
        tuple(int(v) for v in rowadr),
        tuple(int(v) for v in rownnz),
        tuple(int(v) for v in colind),
    )


def shared_bytes(rowadr, rownnz, groups, trunk):
    if not trunk:
        return 0
    entries = sum(rownnz[i] for i in trunk)
    return 4 * 32 * (groups * (entries + len(trunk)) + len(trunk))


def parents_of(rowadr, rownnz, colind):
    return [colind[rowadr[k] + rownnz[k] - 2] if rownnz[k] > 1 else -1 for k in range(len(rowadr))]


def plan_tree_ldl(rowadr, rownnz, colind, groups):
    nv = len(rowadr)
    parent = parents_of(rowadr, rownnz, colind)
    children = [[] for _ in range(nv)]
    for k in range(nv):
        if parent[k] >= 0:
            children[parent[k]].append(k)
    cost = [n * (n - 1) // 2 + 2 * n for n in rownnz]
    subtree = list(cost)
    size = [1] * nv
    for k in reversed(range(nv)):
        if parent[k] >= 0:
            subtree[parent[k]] += subtree[k]
            size[parent[k]] += size[k]
    roots = [k for k in range(nv) if parent[k] < 0]
    dense_cost = sum(size[r] ** 3 // 3 for r in roots)

    def lpt(parts):
        loads = [0] * groups
        members = [[] for _ in range(groups)]
        order = sorted(parts, key=lambda r: (-subtree[r], r))
        for r in order:
            g = loads.index(min(loads))
            loads[g] += subtree[r]
            members[g].append(r)
        return max(loads), members

    parts = list(roots)
    trunk = []
    best = None
    while True:
        heaviest, members = lpt(parts)
        span = heaviest + sum(cost[k] + 2 * rownnz[k] for k in trunk)
        if best is None or span < best[0]:
            best = (span, sorted(trunk), members)
        splittable = [r for r in parts if children[r]]
        if not splittable:
            break
        r = max(splittable, key=lambda r: (subtree[r], -r))
        parts.remove(r)
        trunk.append(r)
        parts += children[r]
    span, trunk, members = best
    out_groups = []
    for part_roots in members:
        nodes = []
        stack = list(part_roots)
        while stack:
            k = stack.pop()
            nodes.append(k)
            stack += children[k]
        out_groups.append(tuple(sorted(nodes, reverse=True)))
    return Plan(tuple(out_groups), tuple(trunk), int(span), int(dense_cost))


def best_tree_ldl_plan(rowadr, rownnz, colind):
    best = None
    for g in range(1, MAX_GROUPS + 1):
        plan = plan_tree_ldl(rowadr, rownnz, colind, g)
        if shared_bytes(rowadr, rownnz, g, plan.trunk) > MAX_SHARED_BYTES:
            continue
        if best is None or plan.span < best.span:
            best = plan
    assert best is not None
    return best


def tree_ldl_beats_dense(plan):
    return plan.span <= MAX_SHORT_SPAN or plan.dense_cost >= MIN_DENSE_TO_SPAN_RATIO * plan.span


def elimination_order(plan):
    """Dofs in the order the generated code eliminates them: each group's dofs
    (descending), groups in index order, then the trunk descending."""
    out = []
    for g in plan.groups:
        out += list(g)
    out += list(reversed(plan.trunk))
    return out


def csr_from_parents(parent):
    """MuJoCo's M CSR for a dof tree: row k = ancestors root-first, then k."""
    nv = len(parent)
    rowadr, rownnz, colind = [], [], []
    for k in range(nv):
        chain = []
        p = k
        while p >= 0:
            chain.append(p)
            p = parent[p]
        chain.reverse()
        rowadr.append(len(colind))
        rownnz.append(len(chain))
        colind += chain
    return tuple(rowadr), tuple(rownnz), tuple(colind)


# ------------------------------------------------------------- static-pattern sparse L'DL
# Restated from src/instantmimic/utils/mjw_kernels/sparse_hessian.py of the reference, in the
# reference's own form (sets and dictionaries), as the second derivation the product's
# bit-row planner (instantmimic_amd/csrc/sparse_plan.cpp) is compared with table for table:
#
# * ``sparse_pattern``   :62-118  dof adjacency: tree ancestry, cliques over body chains
# * ``sparse_symbolic``  :192-212 fill pattern and elimination levels
# * ``sparse_team``      :215-221 lanes per entry of a level
# * ``sparse_tables``    :229-401, 680-684 slots, level / run / solve / pair / assembly tables
#
# Pinned by: the reference-held invariants (symbolic pattern contains numpy's Cholesky
# pattern, strict level order: tests/test_mjw_sparse_hessian.py:73-98), the fp64 executor of
# the tables solving H x = g to 1e-10 (:199-291), closed forms on tree-only patterns (no fill,
# nfac = nM, levels = longest chain) and the expected counts of the five benchmark trees.

SPARSE_MAX_SHARED_BYTES = 46 * 1024
EQ_CONNECT, EQ_WELD, EQ_JOINT = 0, 1, 2
EQ_FLEX, EQ_FLEXVERT, EQ_FLEXSTRAIN = 4, 5, 6
OBJ_SITE = 6


def _np(a):
    return np.zeros(0, np.int64) if a is None else np.asarray(a)


def body_chain(body, body_parentid, body_dofadr, body_dofnum):
    out, b = [], int(body)
    while b > 0:
        out += range(int(body_dofadr[b]), int(body_dofadr[b]) + int(body_dofnum[b]))
        b = int(body_parentid[b])
    return out


def sparse_pattern(m, body_groups):
    """Dof adjacency (list of sets) of a model namespace: sparse_hessian.py:62-118 without the
    flex couplings."""
    nv = int(m.nv)
    dof_parentid = _np(m.dof_parentid)
    bp, ba, bn = _np(m.body_parentid), _np(m.body_dofadr), _np(m.body_dofnum)
    adj = [set() for _ in range(nv)]
    for d in range(nv):
        p = int(dof_parentid[d])
        while p >= 0:
            adj[d].add(p)
            adj[p].add(d)
            p = int(dof_parentid[p])

    def clique(bodies):
        dofs = sorted({d for b in bodies for d in body_chain(b, bp, ba, bn)})
        for a in dofs:
            adj[a].update(x for x in dofs if x != a)

    for group in body_groups:
        clique(group)
    if int(getattr(m, "neq", 0)):
        site_bodyid, jnt_dofadr = _np(m.site_bodyid), _np(m.jnt_dofadr)
        for t, a, b, ot in zip(_np(m.eq_type), _np(m.eq_obj1id), _np(m.eq_obj2id), _np(m.eq_objtype), strict=True):
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
    pairs = _np(getattr(m, "nxn_geom_pair_filtered", None))
    if pairs.size:
        geom_bodyid = _np(m.geom_bodyid)
        for g1, g2 in pairs.reshape(-1, 2):
            clique((geom_bodyid[g1], geom_bodyid[g2]))
    return adj


def sparse_symbolic(adj_e):
    """``rowstruct`` (earlier columns of each row), ``colstruct`` (later rows of each column)
    and ``levels`` (columns by longest path in the elimination tree): sparse_hessian.py:192-212."""
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


def sparse_team(nentries, maxterms, lanes):
    best, cost = 1, None
    for T in (1, 2, 4, 8, 16, 32):
        c = -(-nentries // (lanes // T)) * (-(-maxterms // T) + 2 * int(np.log2(T)))
        if cost is None or c < cost:
            best, cost = T, c
    return best


@dataclass
class SparsePlan:
    nv: int
    nv_pad: int
    block: int
    nslots: int
    nterms: int
    levels: int
    density: float
    path: str
    tables: dict
    colstruct: list
    level_cols: list

    @property
    def nfac(self):
        return self.nslots - self.nv


def sparse_tables(nv, nv_pad, adj, M_rowi, M_colind, block, path="fused"):
    """The plan of a dof adjacency: sparse_hessian.py:229-401 and the limits of :249, 337, 680-684
    (ValueError with the reference's messages)."""
    orig = [nv - 1 - e for e in range(nv)]
    adj_e = [set(nv - 1 - a for a in adj[orig[e]]) for e in range(nv)]
    rowstruct, colstruct, levels = sparse_symbolic(adj_e)
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
        entries.sort(key=lambda e: -e[3])
        for s, c, runs, nt in entries:
            ent_slot.append(s)
            ent_col.append(c)
            for a, b, k, ln in runs:
                run_ab.append(a | (b << 16))
                run_kl.append(k | (ln << 16))
            run_ptr.append(len(run_ab))
            nterms += nt
        lvl_ptr.append(len(ent_slot))
        lvl_team.append(sparse_team(len(entries), max(e[3] for e in entries), block))
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
    for e, (r, c) in enumerate(zip(_np(M_rowi), _np(M_colind), strict=True)):
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
    nw = block // 32
    init_tile = 4 * nv + 4 if path == "fused" else 0
    if 4 * (nslots + n + 2 * nw + init_tile) > SPARSE_MAX_SHARED_BYTES:
        raise ValueError("the factor does not fit the block's shared memory")
    i32 = lambda v: np.asarray(v if len(v) else [0], np.int32)  # noqa: E731
    u32 = lambda v: np.asarray(v if len(v) else [0], np.uint32).view(np.int32)  # noqa: E731
    tables = {
        "SH_LP": i32(lvl_ptr), "SH_LT": i32(lvl_team), "SH_ES": i32(ent_slot), "SH_EC": i32(ent_col),
        "SH_RP": i32(run_ptr), "SH_RAB": u32(run_ab), "SH_RKL": u32(run_kl), "SH_ORIG": i32(orig),
        "SH_BL": i32(b_lvl), "SH_BS": i32(b_slot), "SH_BI": i32(b_src), "SH_BJ": i32(b_dst), "SH_PAIR": i32(pair),
        "SH_FL": i32(f_lvl), "SH_FR": i32(f_row), "SH_RS": i32(row_start), "SH_RKP": i32(rk_ptr), "SH_RK": i32(rk),
        "SH_PM": u32(pmask), "SH_SA": i32(s_a), "SH_SB": i32(s_b), "SH_SM": i32(s_m), "SH_GAT": i32(gat),
    }  # fmt: skip
    return SparsePlan(nv, nv_pad, block, nslots, nterms, len(levels), nfac / (nv * (nv + 1) / 2), path, tables, colstruct, levels)
