"""The C ABI without a GPU: the library loads, exports what the header declares,
and its host planner equals the oracle's restatement of the reference planner."""

import ctypes as C
import os
import re

import numpy as np
import pytest

from instantmimic_amd import _lib, synth
from instantmimic_amd.mjw_kernels import tree_ldl as T
from oracle import planner as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    names = set()
    inc = os.path.join(ROOT, "include")
    for fn in os.listdir(inc):
        if fn.endswith(".h"):
            text = open(os.path.join(inc, fn)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            names |= set(re.findall(r"\b(im_[a-z0-9_]+)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol():
    lib = _lib.lib()
    declared = _declared_symbols()
    assert declared, "no declarations found"
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    assert lib.im_version() >= 100
    assert lib.im_status_string(_lib.IM_ERR_STRUCTURE)


def _same(a, b):
    return (a.groups, a.trunk, a.span, a.dense_cost) == (b.groups, b.trunk, b.span, b.dense_cost)


def test_host_planner_equals_the_oracle_on_the_benchmark_trees():
    for name, shape in synth.SHAPES.items():
        st = T.tree_ldl_structure(*synth.csr_from_parents(shape.parents))
        assert st == P.tree_ldl_structure(*st)
        for g in (1, 2, 3, 4):
            assert _same(T.plan_tree_ldl(*st, g), P.plan_tree_ldl(*st, g)), (name, g)
        best = T.best_tree_ldl_plan(*st)
        assert _same(best, P.best_tree_ldl_plan(*st)), name
        assert T.tree_ldl_beats_dense(best) == P.tree_ldl_beats_dense(P.best_tree_ldl_plan(*st))
        assert list(T.elimination_order(best)) == P.elimination_order(P.best_tree_ldl_plan(*st))


def test_host_planner_equals_the_oracle_on_random_forests():
    rng = np.random.default_rng(5)
    for _ in range(200):
        nv = int(rng.integers(1, 64))
        parent = [-1] + [int(rng.integers(-1 if rng.random() < 0.1 else 0, k)) for k in range(1, nv)]
        st = T.tree_ldl_structure(*synth.csr_from_parents(parent))
        assert st is not None
        for g in (0, 1, 2, 3, 4):
            a = T.plan_tree_ldl(*st, g) if g else T.best_tree_ldl_plan(*st)
            b = P.plan_tree_ldl(*st, g) if g else P.best_tree_ldl_plan(*st)
            assert _same(a, b), (parent, g)


def test_limbs_plan_invariants_through_the_c_abi():
    # reference: tests/test_tree_ldl.py:123-145
    st = T.tree_ldl_structure(*synth.csr_from_parents(synth.limbs_parents()))
    single, split = T.plan_tree_ldl(*st, 1), T.plan_tree_ldl(*st, 4)
    assert not single.trunk and split.trunk == tuple(range(6))
    assert sorted(len(g) for g in split.groups) == [6, 6, 6, 6] and split.span < single.span
    chain = T.tree_ldl_structure(*synth.csr_from_parents(synth.chain_parents(30)))
    assert T.tree_ldl_beats_dense(T.best_tree_ldl_plan(*st))
    assert not T.tree_ldl_beats_dense(T.best_tree_ldl_plan(*chain))


def test_structure_check_rejects_what_the_reference_rejects():
    # reference: tests/test_tree_ldl.py:148-161
    rowadr, rownnz, colind = synth.csr_from_parents(synth.branched_parents())
    assert T.tree_ldl_structure(rowadr, rownnz, colind) is not None
    k = int(np.flatnonzero(rownnz > 2)[-1])
    broken = colind.copy()
    s = rowadr[k]
    broken[s], broken[s + 1] = broken[s + 1], broken[s]
    assert T.tree_ldl_structure(rowadr, rownnz, broken) is None
    shifted = colind.copy()
    shifted[rowadr[k] + rownnz[k] - 1] = 0
    assert T.tree_ldl_structure(rowadr, rownnz, shifted) is None
    assert T.tree_ldl_structure(rowadr, rownnz, colind[:-1]) is None
    assert T.tree_ldl_structure([], [], []) is None
    zero = rownnz.copy()
    zero[3] = 0
    assert T.tree_ldl_structure(rowadr, zero, colind) is None


def test_status_codes():
    lib = _lib.lib()
    rowadr, rownnz, colind = synth.csr_from_parents(synth.ant_parents())
    handle = C.c_void_p()
    args = (rowadr.ctypes.data, rownnz.ctypes.data, colind.ctypes.data, int(colind.size))
    assert lib.im_tree_plan_create(14, *args, 5, 1, C.byref(handle)) == _lib.IM_ERR_ARG
    assert lib.im_tree_plan_create(14, None, None, None, 0, 0, 1, C.byref(handle)) == _lib.IM_ERR_ARG
    bad = colind.copy()
    bad[-1] = 0
    assert lib.im_tree_plan_create(14, rowadr.ctypes.data, rownnz.ctypes.data, bad.ctypes.data, int(bad.size), 0, 1, C.byref(handle)) == _lib.IM_ERR_STRUCTURE
    assert lib.im_tree_plan_create(14, *args, 0, 1, C.byref(handle)) == _lib.IM_OK
    info = _lib.TreePlanInfo()
    assert lib.im_tree_plan_get_info(handle, C.byref(info)) == _lib.IM_OK
    assert (info.nv, info.nM, info.ngroups, info.span, info.device_ready) == (14, 81, 4, 198, 0)
    # a host-only plan cannot launch
    assert lib.im_tree_factor_solve(handle, 1, 81, 1, 14, 1, 14, 1, None) == _lib.IM_ERR_UNSUPPORTED
    lib.im_tree_plan_destroy(handle)
    with pytest.raises(_lib.ImhipError):
        _lib.check(_lib.IM_ERR_STRIDE, "x")


def test_tree_walk_entry_points_check_their_arguments_before_any_launch():
    """Every refusal below happens on the host, before a HIP call: negative sizes, null
    pointers, rows shorter than their contents, worlds too large for LDS; empty batches
    succeed."""
    lib = _lib.lib()
    one = 16  # any non-null address: nothing is dereferenced on these paths
    # M v
    assert lib.im_mul_m_sparse(one, 81, 81, one, one, one, 148, one, 14, None, one, 14, 14, -1, None) == _lib.IM_ERR_ARG
    assert lib.im_mul_m_sparse(None, 81, 81, one, one, one, 148, one, 14, None, one, 14, 14, 3, None) == _lib.IM_ERR_ARG
    assert lib.im_mul_m_sparse(one, 80, 81, one, one, one, 148, one, 14, None, one, 14, 14, 3, None) == _lib.IM_ERR_STRIDE
    assert lib.im_mul_m_sparse(one, 81, 81, one, one, one, 148, one, 14, None, one, 13, 14, 3, None) == _lib.IM_ERR_STRIDE
    assert lib.im_mul_m_sparse(one, 70000, 70000, one, one, one, 139000, one, 1000, None, one, 1000, 1000, 3, None) == _lib.IM_ERR_UNSUPPORTED
    assert lib.im_mul_m_sparse(one, 20000, 20000, one, one, one, 39000, one, 1000, None, one, 1000, 1000, 3, None) == _lib.IM_ERR_UNSUPPORTED
    assert lib.im_mul_m_sparse(None, 0, 0, None, None, None, 0, None, 0, None, None, 0, 0, 0, None) == _lib.IM_OK
    # accumulation
    assert lib.im_tree_accumulate(one, one, one, 3, 3, 0, one, 30, 10, -1, None) == _lib.IM_ERR_ARG
    assert lib.im_tree_accumulate(one, one, one, 3, 3, 0, None, 30, 10, 4, None) == _lib.IM_ERR_ARG
    assert lib.im_tree_accumulate(one, one, one, 3, 3, 0, one, 29, 10, 4, None) == _lib.IM_ERR_STRIDE
    assert lib.im_tree_accumulate(one, one, one, 3, 10, 0, one, 20000, 2000, 4, None) == _lib.IM_ERR_UNSUPPORTED
    assert lib.im_tree_accumulate(None, None, None, 1, 3, 0, None, 30, 10, 4, None) == _lib.IM_OK  # a single level: nothing to add
    assert lib.im_tree_accumulate(None, None, None, 3, 3, 0, None, 30, 10, 0, None) == _lib.IM_OK
    # wrench projection
    w, t = _lib.BodyWrenches(), _lib.WrenchTopology()
    assert lib.im_project_body_wrenches(C.byref(w), None, 6, 50, 0, one, 50, 4, None) == _lib.IM_ERR_ARG
    t.body_count, t.levels = 26, 8
    assert lib.im_project_body_wrenches(C.byref(w), C.byref(t), 6, 50, 0, one, 50, 4, None) == _lib.IM_ERR_ARG  # null arrays
    assert lib.im_project_body_wrenches(C.byref(w), C.byref(t), 6, 0, 0, None, 0, 4, None) == _lib.IM_OK
    for name in ("body_force", "body_torque", "xipos", "subtree_com", "cdof", "body_rootid"):
        setattr(w, name, one)
    for name in ("dof_bodyid", "body_parentid", "level_bodies", "level_offsets"):
        setattr(t, name, one)
    assert lib.im_project_body_wrenches(C.byref(w), C.byref(t), 6, 50, 2, one, 51, 4, None) == _lib.IM_ERR_STRIDE
    t.body_count = 3000
    assert lib.im_project_body_wrenches(C.byref(w), C.byref(t), 6, 50, 0, one, 50, 4, None) == _lib.IM_ERR_UNSUPPORTED


def test_newton_entry_points_check_their_arguments_before_any_launch():
    lib = _lib.lib()
    one = 16  # any non-null address: nothing is dereferenced on these paths
    g = lambda **k: lib.im_newton_gradient(  # noqa: E731
        k.get("nefc"), k.get("J", one), 64, one, k.get("ldf", 64), one, 27, one, 27, one, one, None, one, 27, one,
        k.get("ldg", 27), one, one, one, one, 27, k.get("block", 64), k.get("nworld", 4), None)  # fmt: skip
    assert g(nworld=-1) == _lib.IM_ERR_ARG and g(J=None) == _lib.IM_ERR_ARG
    assert g(block=48) == _lib.IM_ERR_UNSUPPORTED
    assert g(ldf=63) == _lib.IM_ERR_STRIDE and g(ldg=26) == _lib.IM_ERR_STRIDE
    assert g(nworld=0) == _lib.IM_OK
    assert lib.im_newton_jv(one, 64, None, one, 26, None, one, 64, 27, 4, None) == _lib.IM_ERR_STRIDE
    assert lib.im_newton_jv(one, 64, None, one, 27, None, one, 63, 27, 4, None) == _lib.IM_ERR_STRIDE
    assert lib.im_newton_jv(None, 64, None, one, 27, None, one, 64, 27, 4, None) == _lib.IM_ERR_ARG
    assert lib.im_newton_jv(one, 64, None, one, 400, None, one, 64, 400, 4, None) == _lib.IM_ERR_UNSUPPORTED  # 64 rows of 400 dofs exceed LDS
    assert lib.im_newton_jv(one, 0, None, one, 27, None, one, 0, 27, 4, None) == _lib.IM_OK
    assert lib.im_newton_advance(one, one, 27, one, 27, one, 64, None, None, one, 26, one, 27, one, 64, 27, 64, 4, None) == _lib.IM_ERR_STRIDE
    assert lib.im_newton_advance(None, one, 27, one, 27, one, 64, None, None, one, 27, one, 27, one, 64, 27, 64, 4, None) == _lib.IM_ERR_ARG
    assert lib.im_newton_changed_rows(one, None, 64, None, 1, None, one, 64, one, one, 4, None) == _lib.IM_ERR_ARG
    assert lib.im_newton_changed_rows(one, one, 64, None, 1, None, one, 64, one, one, 0, None) == _lib.IM_OK
    assert lib.im_newton_converged(one, one, one, one, one, 0, one, 1, 27, 5, 0, one, None, one, None, 4, None) == _lib.IM_ERR_ARG
    assert lib.im_newton_converged(one, one, one, one, one, 1, one, 1, 27, 5, 0, one, None, None, None, 4, None) == _lib.IM_ERR_ARG
    assert lib.im_newton_init_empty_worlds(one, one, 26, one, one, one, one, 27, 27, 4, None) == _lib.IM_ERR_STRIDE
    assert lib.im_qfrc_constraint_from_grad(one, one, 27, one, 27, one, 27, None, one, 27, 27, 4, None) == _lib.IM_ERR_ARG


def _newton_args(**over):
    """An ``im_newton_args`` block with every pointer non-null (nothing is dereferenced before the checks)."""
    import ctypes as C

    a = _lib.NewtonArgs()
    for name, kind in a._fields_:
        setattr(a, name, 16 if kind is C.c_void_p else 0)
    a.ntolerance = a.nls_tolerance = a.nmeaninertia = 1
    a.ls_iterations, a.iterations, a.block, a.quad = 50, 10, 32, 1
    a.nterm, a.ldM, a.njmax, a.ld_grad, a.ld_ids, a.nworld = 243, 243, 64, 32, 64, 4
    for k, v in over.items():
        setattr(a, k, v)
    return a


def test_init_context_entry_point_checks_its_arguments_before_any_launch():
    import ctypes as C

    lib = _lib.lib()
    one = 16
    call = lambda a, smooth=one, lds=27, aref=one, lda=64, nv=27, nM=243: lib.im_newton_init_context(  # noqa: E731
        C.byref(a), smooth, lds, aref, lda, nv, nM, None)
    assert call(_newton_args(nworld=0)) == _lib.IM_OK
    assert call(_newton_args(nworld=-1)) == _lib.IM_ERR_ARG
    assert call(_newton_args(), smooth=None) == _lib.IM_ERR_ARG and call(_newton_args(), aref=None) == _lib.IM_ERR_ARG
    assert call(_newton_args(efc_J=None)) == _lib.IM_ERR_ARG and call(_newton_args(block=48)) == _lib.IM_ERR_ARG
    assert call(_newton_args(), lds=26) == _lib.IM_ERR_STRIDE and call(_newton_args(), lda=63) == _lib.IM_ERR_STRIDE
    assert call(_newton_args(ldM=242)) == _lib.IM_ERR_STRIDE and call(_newton_args(ld_grad=26)) == _lib.IM_ERR_STRIDE
    # four worlds' vectors and a tile of J per workgroup: 4 (3 nv + 3 njmax + 1088) words must fit a CU's LDS
    assert call(_newton_args(njmax=4000, ld_ids=4000), lda=4000) == _lib.IM_ERR_UNSUPPORTED
    # the resident solves: no plan, no argument block
    assert lib.im_newton_solve_tree(None, C.byref(_newton_args()), None) == _lib.IM_ERR_ARG
    assert lib.im_newton_solve_sparse(None, C.byref(_newton_args()), one, one, None) == _lib.IM_ERR_ARG


def test_dense_init_entry_point_checks_its_arguments_before_any_launch():
    lib = _lib.lib()
    one = 16
    call = lambda **k: lib.im_dense_init_factor(  # noqa: E731
        None, None, k.get("J", one), k.get("njmax", 96), one, one, 1, k.get("M", one), 341, k.get("elemid", one), one,
        k.get("ldg", 48), k.get("H", one), k.get("U", one), k.get("nv", 35), k.get("pad", 48), one, one, k.get("lds", 35), one,
        one, k.get("nworld", 4), None)  # fmt: skip
    assert call(nworld=0) == _lib.IM_OK and call(nworld=-1) == _lib.IM_ERR_ARG and call(njmax=0) == _lib.IM_ERR_ARG
    assert call(J=None) == _lib.IM_ERR_ARG and call(M=None) == _lib.IM_ERR_ARG and call(elemid=None) == _lib.IM_ERR_ARG
    assert call(U=None) == _lib.IM_ERR_ARG and call(H=None) == _lib.IM_ERR_ARG and call(pad=32) == _lib.IM_ERR_ARG
    assert call(ldg=34) == _lib.IM_ERR_STRIDE and call(lds=34) == _lib.IM_ERR_STRIDE and call(H=20) == _lib.IM_ERR_STRIDE
    # 64 dofs and more (a padded size of 80 and up) have no launch of this kind
    assert call(nv=64, pad=80, ldg=80, lds=64) == _lib.IM_ERR_UNSUPPORTED and call(nv=35, pad=52) == _lib.IM_ERR_UNSUPPORTED
    # the single tile: at most 32 dofs
    tile = lambda nv, pad: lib.im_dense_init_tile(None, None, one, 64, one, one, 1, one, 243, one, one, 32, one, nv, pad, one,  # noqa: E731
                                                  one, 32, one, one, 4, None)  # fmt: skip
    assert tile(33, 48) == _lib.IM_ERR_ARG and tile(27, 16) == _lib.IM_ERR_ARG


def test_implicit_matrix_entry_points_check_their_arguments_before_any_launch():
    lib = _lib.lib()
    one = 16
    q = lambda **k: lib.im_implicit_qh(  # noqa: E731
        k.get("M", one), k.get("ldM", 737), 737, one, one, 0, 0.004, one, one, one, one, k.get("ldprm", 10), None, None, one,
        k.get("ld_input", 40), None, 0, one, 40, k.get("nu", 40), k.get("ta"), k.get("tt"), one, k.get("ldq", 737),
        k.get("nworld", 4), None)  # fmt: skip
    assert q(nworld=-1) == _lib.IM_ERR_ARG and q(M=None) == _lib.IM_ERR_ARG and q(ldprm=2) == _lib.IM_ERR_ARG
    assert q(ldM=700) == _lib.IM_ERR_STRIDE and q(ldq=700) == _lib.IM_ERR_STRIDE and q(ld_input=39) == _lib.IM_ERR_ARG
    assert q(nworld=0) == _lib.IM_OK
    term = _lib.RowPairTerm()
    term.nentry, term.nelem, term.chunk_count = 80, 60, 30  # tables missing
    assert q(ta=C.byref(term)) == _lib.IM_ERR_ARG
    for name in ("values", "entry_row", "elem_ids", "chunk_offsets", "chunk_pairs"):
        setattr(term, name, one)
    assert q(tt=C.byref(term)) == _lib.IM_ERR_ARG  # the tendon term needs its weights
    assert q(ta=C.byref(term), nu=0) == _lib.IM_ERR_ARG  # the actuator term's weights are the gains
    term.nentry = 40000
    assert q(ta=C.byref(term)) == _lib.IM_ERR_UNSUPPORTED  # entry indices travel as 15 bits
    term.nentry, term.chunk_count = 9000, 9000
    assert q(ta=C.byref(term)) == _lib.IM_ERR_UNSUPPORTED  # a world's rows exceed 64 KB of LDS
    assert lib.im_implicit_qh_base(one, 700, 737, one, one, 0, 0.004, one, 737, 4, None) == _lib.IM_ERR_STRIDE
    assert lib.im_actuator_velocity_gain(one, one, one, one, 2, None, None, one, 40, None, 0, one, 40, 40, 4, None) == _lib.IM_ERR_ARG


def test_entry_points_that_clamp_rows_refuse_an_empty_row_range():
    """The assembly kernels clamp a row index to njmax - 1 (every load is issued, the value
    selected afterwards), so njmax = 0 is refused on the host instead of reading before the
    arrays; likewise an empty entry list of the torque projection."""
    lib = _lib.lib()
    one = 16
    assert lib.im_jtdj_mfma(one, one, 0, one, one, None, 1, one, 27, 32, 4, None) == _lib.IM_ERR_ARG
    assert lib.im_muscle_project(one, 0, one, 4, one, one, one, 0, 4, 3, 0, one, 3, 2, None) == _lib.IM_ERR_ARG
    assert lib.im_muscle_project(one, 0, one, 4, one, one, one, 0, 4, 0, 0, one, 3, 2, None) == _lib.IM_OK
    assert lib.im_dense_update_factor(None, one, one, one, 8, one, 0, one, one, 1, one, 27, 32, 32, 27, 32, one, one, 27, one, one, 4, None) == _lib.IM_ERR_ARG


def test_ctypes_structs_match_the_header(tmp_path):
    """Every structure of include/imhip.h that the Python side fills through ctypes: the same size
    and the same offset for every field, read from a probe that gcc compiles against the header."""
    import ctypes as C
    import os
    import subprocess

    pairs = {
        "im_tree_plan_info": _lib.TreePlanInfo, "im_sparse_plan_info": _lib.SparsePlanInfo,
        "im_muscle_force_model": _lib.MuscleForceModel, "im_muscle_force_velocity_model": _lib.MuscleForceVelocityModel,
        "im_newton_args": _lib.NewtonArgs, "im_row_pair_term": _lib.RowPairTerm, "im_muscle_geometry": _lib.MuscleGeometry,
        "im_muscle_segments": _lib.MuscleSegments, "im_muscle_entries": _lib.MuscleEntries,
        "im_body_wrenches": _lib.BodyWrenches, "im_wrench_topology": _lib.WrenchTopology,
    }  # fmt: skip
    lines = ["#include <stddef.h>", "#include <stdio.h>", '#include "imhip.h"', "int main(void) {"]
    for cname, ctype in pairs.items():
        lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
        for field, _ in ctype._fields_:
            lines.append(f'  printf("{cname}.{field} %zu\\n", offsetof({cname}, {field}));')
    lines += ["  return 0;", "}"]
    src, exe = tmp_path / "probe.c", tmp_path / "probe"
    src.write_text("\n".join(lines))
    include = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    subprocess.run(["gcc", "-std=c11", "-I", include, str(src), "-o", str(exe)], check=True)
    seen = dict(line.split() for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for cname, ctype in pairs.items():
        assert int(seen[cname]) == C.sizeof(ctype), cname
        for field, _ in ctype._fields_:
            assert int(seen[f"{cname}.{field}"]) == getattr(ctype, field).offset, f"{cname}.{field}"
