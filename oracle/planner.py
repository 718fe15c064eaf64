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
