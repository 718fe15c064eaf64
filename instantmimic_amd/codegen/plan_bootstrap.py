"""Build-time planning for the kernel generator.

The generator needs each known tree's plan (groups, trunk) before ``libimhip.so``
exists, so the cut/pack rule of the library's host planner
(``csrc/tree_plan.cpp``; reference tree_ldl.py:105-193) is evaluated here once more in
a compact form.  A kernel generated for a plan that differs from the library's is
never selected: kernels are looked up by a key over structure *and* plan, and
``tests/test_capi.py`` checks that the two planners agree.
"""

from __future__ import annotations


def _csr(parent):
    rowadr, rownnz, colind = [], [], []
    for k in range(len(parent)):
        chain, p = [], k
        while p >= 0:
            chain.append(p)
            p = parent[p]
        rowadr.append(len(colind))
        rownnz.append(len(chain))
        colind += chain[::-1]
    return tuple(rowadr), tuple(rownnz), tuple(colind)


def _plan(rowadr, rownnz, colind, parent, groups):
    nv = len(parent)
    kids = [[] for _ in range(nv)]
    for k, p in enumerate(parent):
        if p >= 0:
            kids[p].append(k)
    cost = [n * (n - 1) // 2 + 2 * n for n in rownnz]
    sub, size = list(cost), [1] * nv
    for k in range(nv - 1, -1, -1):
        if parent[k] >= 0:
            sub[parent[k]] += sub[k]
            size[parent[k]] += size[k]
    roots = [k for k in range(nv) if parent[k] < 0]
    parts, trunk, best = list(roots), [], None
    while True:
        loads, bins = [0] * groups, [[] for _ in range(groups)]
        for r in sorted(parts, key=lambda r: (-sub[r], r)):
            g = loads.index(min(loads))
            loads[g] += sub[r]
            bins[g].append(r)
        span = max(loads) + sum(cost[k] + 2 * rownnz[k] for k in trunk)
        if best is None or span < best[0]:
            best = (span, sorted(trunk), bins)
        cand = [r for r in parts if kids[r]]
        if not cand:
            break
        r = max(cand, key=lambda r: (sub[r], -r))
        parts.remove(r)
        trunk.append(r)
        parts += kids[r]
    span, trunk, bins = best
    out = []
    for b in bins:
        nodes, stack = [], list(b)
        while stack:
            k = stack.pop()
            nodes.append(k)
            stack += kids[k]
        out.append(tuple(sorted(nodes, reverse=True)))
    dense = sum(size[r] ** 3 // 3 for r in roots)
    return tuple(out), tuple(trunk), span, dense


def best_plan(parent):
    st = _csr(parent)
    best = None
    for g in range(1, 5):
        groups, trunk, span, dense = _plan(*st, parent, g)
        smem = 4 * 32 * (g * (sum(st[1][i] for i in trunk) + len(trunk)) + len(trunk)) if trunk else 0
        if smem > 48 * 1024:
            continue
        if best is None or span < best[2]:
            best = (groups, trunk, span, dense)
    groups, trunk, span, dense = best
    return st, groups, trunk, (span <= 4096 or dense >= 8.0 * span)
