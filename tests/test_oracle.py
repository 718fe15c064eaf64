"""Pins the CPU oracle: planner invariants the reference's tests hold, the recorded
plans of the benchmark trees, and the numeric restatement against fp64 algebra."""

import json
import os

import numpy as np
import pytest

from instantmimic_amd import synth
from oracle import planner as P
from oracle import ref as R

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _structure(parent):
    return P.csr_from_parents(list(parent))


# ---------------------------------------------------------------- integer planning


def test_limbs_plans_cover_every_dof_once_and_split_off_a_trunk():
    # reference: tests/test_tree_ldl.py:123-136
    st = _structure(synth.limbs_parents(4, 6))
    nv = len(st[0])
    for g in (1, 2, 4):
        plan = P.plan_tree_ldl(*st, g)
        dofs = sorted([*plan.trunk, *(k for nodes in plan.groups for k in nodes)])
        assert dofs == list(range(nv))
    single = P.plan_tree_ldl(*st, 1)
    split = P.plan_tree_ldl(*st, 4)
    assert not single.trunk
    assert split.trunk == tuple(range(6))
    assert sorted(len(n) for n in split.groups) == [6, 6, 6, 6]
    assert split.span < single.span


def test_one_group_span_is_the_sum_of_costs():
    for name, shape in synth.SHAPES.items():
        st = _structure(shape.parents)
        plan = P.plan_tree_ldl(*st, 1)
        assert plan.trunk == ()
        assert plan.span == sum(n * (n - 1) // 2 + 2 * n for n in st[1]), name


def test_eligibility_matches_the_reference_cases():
    # reference: tests/test_tree_ldl.py:139-145
    assert P.tree_ldl_beats_dense(P.best_tree_ldl_plan(*_structure(synth.limbs_parents())))
    assert not P.tree_ldl_beats_dense(P.best_tree_ldl_plan(*_structure(synth.chain_parents(30))))


def test_structure_requires_nested_ancestor_rows():
    # reference: tests/test_tree_ldl.py:148-161
    rowadr, rownnz, colind = (np.array(a) for a in _structure(synth.branched_parents()))
    assert P.tree_ldl_structure(rowadr, rownnz, colind) is not None
    k = int(np.flatnonzero(rownnz > 2)[-1])
    broken = colind.copy()
    s = rowadr[k]
    broken[s], broken[s + 1] = broken[s + 1], broken[s]
    assert P.tree_ldl_structure(rowadr, rownnz, broken) is None
    shifted = colind.copy()
    shifted[rowadr[k] + rownnz[k] - 1] = 0
    assert P.tree_ldl_structure(rowadr, rownnz, shifted) is None
    assert P.tree_ldl_structure(rowadr[:0], rownnz[:0], colind) is None
    assert P.tree_ldl_structure(rowadr, rownnz, colind[:-1]) is None


def test_recorded_plans():
    with open(os.path.join(GOLDEN, "tree_plans.json")) as f:
        golden = json.load(f)
    # the table of expected plans (cross-check values derived independently of this code)
    expected = {
        "ant": ([393, 277, 277, 198], 4, 198, 14592, 914, True),
        "humanoid": ([1656, 1023, 890, 890], 3, 890, 21888, 6561, True),
        "g1": ([2424, 1407, 1042, 1042], 3, 1042, 21888, 14291, True),
        "snu": ([6372, 3818, 2858, 2433], 4, 2433, 47616, 58538, True),
        "stress": ([115136, 77228, 70644, 70644], 1, 115136, 0, 699050, False),
    }
    for name, (spans, ng, span, smem, dense, ok) in expected.items():
        st = _structure(synth.SHAPES[name].parents)
        assert [P.plan_tree_ldl(*st, g).span for g in (1, 2, 3, 4)] == spans
        best = P.best_tree_ldl_plan(*st)
        assert (len(best.groups), best.span, best.dense_cost) == (ng, span, dense)
        assert P.shared_bytes(st[0], st[1], ng, best.trunk) == smem
        assert P.tree_ldl_beats_dense(best) == ok
        g = golden[name]
        assert [list(x) for x in best.groups] == g["groups"] and list(best.trunk) == g["trunk"]
        assert P.elimination_order(best) == g["elimination_order"]
    assert golden["humanoid"]["elimination_order"] == [*range(14, 8, -1), *range(20, 14, -1), *range(26, 20, -1), *range(8, -1, -1)]
    assert golden["humanoid"]["trunk"] == list(range(9))
    assert golden["g1"]["trunk"] == [0, 1, 2, 3, 4, 5, 18, 19, 20]
    assert golden["snu"]["trunk"] == [0, 1, 2, 3, 4, 5, 26, 27, 28, 29, 30, 31]
    assert golden["snu"]["nM"] == 716 and golden["humanoid"]["nM"] == 243 and golden["g1"]["nM"] == 341


# ---------------------------------------------------------------- numeric statements


def _well_conditioned(parent, worlds, seed):
    """M like the reference's test matrices: SPD with tree sparsity plus a damping
    diagonal (tests/test_tree_ldl.py:63-80), kept well conditioned."""
    rng = np.random.default_rng(seed)
    nv = len(parent)
    mask = synth.chain_mask(parent)
    V = rng.standard_normal((worlds, nv, nv)) * mask[None]
    dense = np.einsum("wki,wkj->wij", V, V) + np.eye(nv) * (2.0 + rng.uniform(0, 0.2, (worlds, nv, 1)))
    dense = 0.5 * (dense + dense.transpose(0, 2, 1))
    rowadr, rownnz, colind = synth.csr_from_parents(parent)
    rowi = np.repeat(np.arange(nv), rownnz)
    return dense, dense[:, rowi, colind].astype(np.float32), (rowadr, rownnz, colind)


@pytest.mark.parametrize("tree", ["branched", "limbs"])
@pytest.mark.parametrize("groups", [1, 2, 4])
def test_tree_solve_matches_a_dense_solve(tree, groups):
    # reference: tests/test_tree_ldl.py:99-120 (37 worlds, rtol 2e-4, atol 2e-5)
    parent = synth.branched_parents() if tree == "branched" else synth.limbs_parents()
    dense, sparse, st = _well_conditioned(parent, 37, 0)
    st = P.tree_ldl_structure(*st)
    plan = P.plan_tree_ldl(*st, groups)
    y = np.random.default_rng(1).normal(size=(37, len(parent))).astype(np.float32)
    x = R.tree_ldl_solve(*st, plan, sparse, y)
    full = R.dense_from_csr(sparse.astype(np.float64), *st)
    expected = R.solve64(full, y)
    np.testing.assert_allclose(x, expected, rtol=2e-4, atol=2e-5)


def test_factor_reconstructs_the_matrix():
    """L' D L == H with L unit lower triangular in (ancestor, descendant) order."""
    parent = synth.humanoid_parents()
    dense, sparse, st = _well_conditioned(parent, 5, 3)
    st = P.tree_ldl_structure(*st)
    plan = P.best_tree_ldl_plan(*st)
    y = np.ones((5, len(parent)), np.float32)
    _, ld = R.tree_ldl_solve(*st, plan, sparse, y, want_factor=True)
    nv = len(parent)
    rowi = R.rows_of(st[1])
    col = np.array(st[2])
    for w in range(5):
        L = np.eye(nv)
        Dg = np.zeros(nv)
        for e in range(len(col)):
            if rowi[e] == col[e]:
                Dg[rowi[e]] = ld[w, e]
            else:
                L[rowi[e], col[e]] = ld[w, e]
        rebuilt = L.T @ np.diag(Dg) @ L
        np.testing.assert_allclose(rebuilt, R.dense_from_csr(sparse[w : w + 1].astype(np.float64), *st)[0], rtol=2e-5, atol=2e-5)


def test_tiny_trees_brute_force():
    """Every tree with up to 5 dofs against exact fp64 elimination."""
    import itertools

    for nv in range(1, 6):
        for parent in itertools.product(*[range(-1, k) for k in range(nv)]):
            parent = list(parent)
            dense, sparse, st = _well_conditioned(parent, 2, nv)
            st = P.tree_ldl_structure(*st)
            assert st is not None
            y = np.random.default_rng(7).normal(size=(2, nv)).astype(np.float32)
            for g in (1, 2, 3):
                x = R.tree_ldl_solve(*st, P.plan_tree_ldl(*st, g), sparse, y)
                full = R.dense_from_csr(sparse.astype(np.float64), *st)
                np.testing.assert_allclose(x, R.solve64(full, y), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("name", ["ant", "humanoid", "g1", "snu"])
def test_assembly_matches_fp64(name):
    b = synth.make_batch(name, 16, ragged_nefc=True)
    st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    H = R.assemble_csr(*st, b.M, b.J, b.D, b.state[0], b.nefc)
    Hd = R.assemble_dense64(*st, b.M, b.J, b.D, b.state[0], b.nefc)
    nv = b.shape.nv
    on = np.zeros((nv, nv), bool)
    on[R.rows_of(st[1]), np.array(st[2])] = True
    on |= on.T
    # chain-supported rows: J'DJ has exactly M's pattern
    assert np.abs(Hd[:, ~on]).max() == 0.0
    H64 = Hd[:, R.rows_of(st[1]), np.array(st[2])]
    assert R.rel_l2(H, H64) < 1e-6
    # inactive rows and rows past nefc contribute nothing
    H2 = R.assemble_csr(*st, b.M, b.J, b.D, np.zeros_like(b.state[0]), b.nefc)
    np.testing.assert_array_equal(H2, b.M)
    H3 = R.assemble_csr(*st, b.M, b.J, b.D, b.state[0], np.zeros_like(b.nefc))
    np.testing.assert_array_equal(H3, b.M)


@pytest.mark.parametrize("name", ["ant", "humanoid", "g1", "snu"])
def test_fused_solve_residual_and_plan_independence(name):
    b = synth.make_batch(name, 32)
    st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    plan = P.best_tree_ldl_plan(*st)
    x, H = R.assemble_tree_ldl_solve(*st, plan, b.M, b.J, b.D, b.state[0], b.nefc, b.grad, want_h=True)
    Hd = R.dense_from_csr(H.astype(np.float64), *st)
    # backward error of an fp32 factorisation
    res = np.einsum("wij,wj->wi", Hd, x.astype(np.float64)) - b.grad
    scale = np.linalg.norm(Hd, axis=(1, 2)) * np.linalg.norm(x, axis=1) + np.linalg.norm(b.grad, axis=1)
    assert (np.linalg.norm(res, axis=1) / scale).max() < 2e-6
    # forward error bounded by conditioning
    x64 = R.solve64(Hd, b.grad)
    cond = np.linalg.cond(Hd)
    err = np.linalg.norm(x - x64, axis=1) / np.linalg.norm(x64, axis=1)
    assert (err / (cond * 6e-8)).max() < 4.0
    # other group counts change only the rounding
    x1 = R.tree_ldl_solve(*st, P.plan_tree_ldl(*st, 1), H, b.grad)
    assert R.rel_l2(x1, x) < 1e-3


def test_stored_vectors_reproduce():
    z = np.load(os.path.join(GOLDEN, "tree_small.npz"))
    b = synth.make_batch("ant", 4)
    np.testing.assert_array_equal(z["M"], b.M)
    np.testing.assert_array_equal(z["J"], b.J)
    st = P.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    plan = P.best_tree_ldl_plan(*st)
    x, H = R.assemble_tree_ldl_solve(*st, plan, z["M"], z["J"], z["D"], z["state"], z["nefc"], z["grad"], want_h=True)
    np.testing.assert_array_equal(x, z["x"])
    np.testing.assert_array_equal(H, z["H"])
