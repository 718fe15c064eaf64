"""Kernels generated for a model at plan creation (the reference emits straight-line code for any
model: src/instantmimic/utils/mjw_kernels/tree_ldl.py:196-359, 393-416; its test models:
tests/test_tree_ldl.py:22-60, 99-236): source from the generator, a gfx950 code object, loaded
into the plan through the C ABI."""

import ctypes as C

import numpy as np
import pytest

from instantmimic_amd import _lib, build, synth
from instantmimic_amd.codegen import jit, tree_row16
from oracle import planner as P
from oracle import ref as R

TREES = synth.extra_trees()


def test_code_objects_and_keys():
    for name in ("limbs", "branched"):
        st, groups, trunk, _ = build._plan_of_tree(TREES[name])
        blob = jit.code_object(st, groups, trunk)
        assert blob is not None and len(blob) > 10000 and blob == jit.code_object(st, groups, trunk)
        for symbol in (b"im_row16_fused", b"im_row16_fused_long", b"im_row16_solve", b"im_row16_key", b"im_row16_info"):
            assert symbol in blob
        # the library's key of the same plan (host-only plan: no GPU needed)
        rowadr, rownnz, colind = (np.asarray(a, np.int32) for a in st)
        handle = C.c_void_p()
        assert _lib.lib().im_tree_plan_create(len(rowadr), rowadr.ctypes.data, rownnz.ctypes.data, colind.ctypes.data, len(colind), 0, 1, C.byref(handle)) == 0
        key, has = C.c_ulonglong(0), C.c_int(7)
        assert _lib.lib().im_tree_plan_kernel_key(handle, C.byref(key), C.byref(has)) == 0
        assert key.value == tree_row16.structure_key(*st, groups, trunk) and has.value == 0
        # a host-only plan takes no kernels
        buf = C.create_string_buffer(blob, len(blob))
        assert _lib.lib().im_tree_plan_attach_kernels(handle, buf) == _lib.IM_ERR_UNSUPPORTED
        assert _lib.lib().im_tree_plan_attach_kernels(handle, None) == _lib.IM_ERR_ARG
        _lib.lib().im_tree_plan_destroy(handle)
    # the module form differs from the library form in its kernel heads and tail only
    st, groups, trunk, _ = build._plan_of_tree(TREES["limbs"])
    a, b = tree_row16.generate("t", *st, groups, trunk), tree_row16.generate("t", *st, groups, trunk, module=True)
    la, lb = a.splitlines(), b.splitlines()
    assert sum(x != y for x, y in zip(la, lb)) <= 24 and abs(len(la) - len(lb)) < 20 and len(la) > 500


def _random_forest(rng, nv, nroots):
    parents = []
    for k in range(nv):
        parents.append(-1 if k < nroots and (k == 0 or rng.random() < 0.7) else int(rng.integers(max(0, k - 6), k)))
    return parents


def test_generator_takes_or_declines_random_forests(tmp_path, monkeypatch):
    """Every eligible plan either gets source or an explicit refusal (a trunk with two roots or a
    fork does not fit the generator's lane layout): nothing else may escape to the caller that
    creates a model's scratch, whose table-driven kernel serves the refused ones."""
    rng = np.random.default_rng(5)
    taken, declined, reasons = 0, [], set()
    for case in range(150):
        nv = int(rng.integers(2, 65))
        parents = _random_forest(rng, nv, 1 if case % 3 else int(rng.integers(2, 4)))
        st, groups, trunk, _ = build._plan_of_tree(parents, int(rng.integers(0, 5)))
        try:
            src = tree_row16.generate("t", *st, groups, trunk, module=True)
            assert "im_row16_fused" in src
            taken += 1
        except tree_row16.Declined as why:
            declined.append((st, groups, trunk))
            reasons.add(str(why))
    assert taken >= 100 and len(declined) >= 5, (taken, len(declined))
    assert reasons <= {"the plan's trunk is not a single chain from one root", "a plan with an empty group"}, reasons
    # the run-time path answers None for a refused plan and does not leave a file behind
    monkeypatch.setenv("IMHIP_KERNEL_CACHE", str(tmp_path))
    assert jit.code_object(*declined[0]) is None
    assert list(tmp_path.iterdir()) == []
    # an occupancy beyond four workgroups per CU is an error, not a silent clamp
    monkeypatch.setenv("IMHIP_OCC", "6")
    st, groups, trunk, _ = build._plan_of_tree(TREES["limbs"])
    with pytest.raises(ValueError, match="IMHIP_OCC"):
        tree_row16.generate("t", *st, groups, trunk)


def test_cache_is_keyed_by_everything_that_changes_the_source(monkeypatch):
    base = jit._source_tag()
    for knob, value in (("IMHIP_EXP", "timing"), ("IMHIP_SP", "3"), ("IMHIP_OCC", "2")):
        monkeypatch.setenv(knob, value)
        assert jit._source_tag() != base
        monkeypatch.delenv(knob)
    assert jit._source_tag() == base
    monkeypatch.setattr(jit, "FLAGS", jit.FLAGS + ["-DX"])
    assert jit._source_tag() != base


def test_kernel_descriptors_of_a_code_object():
    st, groups, trunk, _ = build._plan_of_tree(TREES["limbs"])
    res = jit.kernel_resources(jit.code_object(st, groups, trunk))
    assert set(res) == {"im_row16_fused", "im_row16_fused_long", "im_row16_solve", "im_row16_newton", "im_row16_newton_long"}
    assert all(res[k][1] == 0 for k in ("im_row16_fused", "im_row16_fused_long", "im_row16_solve"))  # the best plan's kernels keep to registers
    # one group for the whole tree holds every row in one wavefront's registers and spills
    st, groups, trunk, _ = build._plan_of_tree(TREES["limbs62"], 1)
    assert jit.code_object(st, groups, trunk) is None


def test_both_compilers_give_the_same_kernels(monkeypatch):
    """The run-time compiler inside the process and the compiler subprocess: the same five kernels
    with the same LDS and private-segment sizes; ``IMHIP_JIT_COMPILER`` allows one of them only."""
    st, groups, trunk, _ = build._plan_of_tree(TREES["branched"])
    src = tree_row16.generate("t", *st, groups, trunk, module=True)
    inside, outside = jit.compile_hiprtc(src, "t"), jit.compile_hipcc(src, "t")
    assert inside is not None and outside is not None
    assert jit.kernel_resources(inside) == jit.kernel_resources(outside)
    assert b"im_row16_key" in inside and b"im_row16_info" in inside
    calls = []
    monkeypatch.setattr(jit, "compile_hiprtc", lambda *a: calls.append("hiprtc"))
    monkeypatch.setattr(jit, "compile_hipcc", lambda *a: calls.append("hipcc"))
    jit.compile_source(src, "t")
    monkeypatch.setenv("IMHIP_JIT_COMPILER", "hipcc")
    jit.compile_source(src, "t")
    monkeypatch.setenv("IMHIP_JIT_COMPILER", "hiprtc")
    jit.compile_source(src, "t")
    assert calls == ["hiprtc", "hipcc", "hipcc", "hiprtc"]
    monkeypatch.setenv("IMHIP_JIT_COMPILER", "nvcc")
    with pytest.raises(ValueError):
        jit.compile_source(src, "t")


def _has_kernel(scratch) -> bool:
    key, has = C.c_ulonglong(0), C.c_int(0)
    assert _lib.lib().im_tree_plan_kernel_key(scratch.kernel.ptr, C.byref(key), C.byref(has)) == 0
    return bool(has.value)


def _batch(name, nworld, nefc=48):
    parents = TREES[name]
    shape = synth.Shape(name, tuple(parents), nefc, nworld, (0.5, 8.0), 0.02, (-4.0, 4.0), 0.6, 3, 31)
    return synth.make_batch(shape, nworld, ragged_nefc=True)


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld", [("limbs", 203), ("branched", 64), ("limbs62", 130), ("contact", 99), ("snu_free", 77)])
def test_gpu_generated_kernels_match_the_oracle_bitwise(device, monkeypatch, name, nworld):
    _generated_against_oracle(device, monkeypatch, name, nworld, table_driven_too=True)


@pytest.mark.gpu
@pytest.mark.parametrize("name,nworld", [("limbs70", 101), ("limbs78", 67)])
def test_gpu_more_than_64_dofs_run_on_generated_kernels(device, monkeypatch, name, nworld):
    """The reference's fused Newton takes up to 79 dofs (its test models have 68, 70 and 78:
    tests/test_tree_ldl.py:178-236); beyond 64 the table-driven kernel does not apply."""
    from instantmimic_amd.mjw_kernels import tree_ldl as T

    _generated_against_oracle(device, monkeypatch, name, nworld, table_driven_too=False)
    b = _batch(name, 4)
    m = type("m", (), dict(nv=b.shape.nv, M_rowadr=b.rowadr, M_rownnz=b.rownnz, M_colind=b.colind))
    monkeypatch.setenv("IMHIP_TREE_JIT", "0")
    assert T.create_tree_factor_solve_scratch(m, device) is None  # nothing to run it on without generated kernels


@pytest.mark.gpu
def test_gpu_cold_compile_inside_the_process(device, monkeypatch, tmp_path):
    """An empty cache directory and a tree that nothing was built for beforehand: the kernels are
    generated and compiled here, in this process (no compiler subprocess), loaded, and right."""
    rng = np.random.default_rng(20261)
    parents = [-1, 0, 1, 2, 3, 4]  # a floating base, then five limbs of random lengths off dof 5
    for _ in range(5):
        at = 5
        for _ in range(int(rng.integers(4, 9))):
            parents.append(at)
            at = len(parents) - 1
    assert tuple(parents) not in {tuple(v) for v in TREES.values()}
    TREES["cold"] = parents
    monkeypatch.setenv("IMHIP_KERNEL_CACHE", str(tmp_path))
    monkeypatch.setenv("IMHIP_JIT_COMPILER", "hiprtc")
    try:
        _generated_against_oracle(device, monkeypatch, "cold", 150, table_driven_too=True)
    finally:
        del TREES["cold"]
    made = [p.name for p in tmp_path.iterdir()]
    assert len(made) == 1 and made[0].startswith("tree_row16_") and made[0].endswith(".co")


@pytest.mark.gpu
def test_gpu_declined_forest_runs_on_the_table_driven_kernel(device, monkeypatch, tmp_path):
    """Two roots: the generator declines the plan (its trunk is no single chain); creating the
    model's scratch must not raise, and the scratch solves on the table-driven kernel."""
    import torch

    from instantmimic_amd.mjw_kernels import tree_ldl as T

    parents = [-1, 0, 0, 2, -1, 4, 4, 6, 1, 1, 3, 3, 5, 5, 7, 7]
    st, groups, trunk, _ = build._plan_of_tree(parents)
    with pytest.raises(tree_row16.Declined):
        tree_row16.generate("t", *st, groups, trunk, module=True)
    monkeypatch.setenv("IMHIP_KERNEL_CACHE", str(tmp_path))
    TREES["forest"] = parents
    try:
        b = _batch("forest", 77, nefc=24)
    finally:
        del TREES["forest"]
    m = type("m", (), dict(nv=b.shape.nv, M_rowadr=b.rowadr, M_rownnz=b.rownnz, M_colind=b.colind))
    scratch = T.create_tree_factor_solve_scratch(m, device)
    assert scratch is not None and not _has_kernel(scratch) and list(tmp_path.iterdir()) == []
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    G = t(b.grad)
    x = torch.full_like(G, float("nan"))
    T.assemble_tree_factor_solve(scratch, t(b.M), t(b.J), t(b.D), t(b.state[0]), t(b.nefc), G, x)
    torch.cuda.synchronize()
    stc = (b.rowadr, b.rownnz, b.colind)
    want = R.assemble_tree_ldl_solve(*stc, P.best_tree_ldl_plan(*stc), b.M, b.J, b.D, b.state[0], b.nefc, b.grad)
    np.testing.assert_array_equal(x.cpu().numpy(), want)


def _generated_against_oracle(device, monkeypatch, name, nworld, table_driven_too):
    import torch

    from instantmimic_amd.mjw_kernels import tree_ldl as T

    b = _batch(name, nworld)
    m = type("m", (), dict(nv=b.shape.nv, M_rowadr=b.rowadr, M_rownnz=b.rownnz, M_colind=b.colind))
    scratch = T.create_tree_factor_solve_scratch(m, device)
    assert scratch is not None and _has_kernel(scratch)
    kernels = [scratch]
    if table_driven_too:
        monkeypatch.setenv("IMHIP_TREE_KERNEL", "generic")
        kernels.append(T.create_tree_factor_solve_scratch(m, device))
        monkeypatch.delenv("IMHIP_TREE_KERNEL")
        assert not _has_kernel(kernels[1])
    st = (b.rowadr, b.rownnz, b.colind)
    oplan = P.best_tree_ldl_plan(*st)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    M, J, D, N, G = t(b.M), t(b.J), t(b.D), t(b.nefc), t(b.grad)
    for sc in kernels:
        x, H = torch.full_like(G, float("nan")), torch.full_like(M, float("nan"))
        T.assemble_tree_factor_solve(sc, M, J, D, t(b.state[0]), N, G, x, H_out=H)
        torch.cuda.synchronize()
        x_ref, H_ref = R.assemble_tree_ldl_solve(*st, oplan, b.M, b.J, b.D, b.state[0], b.nefc, b.grad, want_h=True)
        np.testing.assert_array_equal(H.cpu().numpy(), H_ref)
        np.testing.assert_array_equal(x.cpu().numpy(), x_ref)
        assert R.rel_l2(x.cpu().numpy(), x_ref) <= 1e-5
    # factor + solve alone and a step's three iterations in one launch, on the generated kernels
    x = torch.full_like(G, float("nan"))
    T.tree_factor_solve(scratch, M, x, G)
    x3 = torch.full((3,) + tuple(G.shape), float("nan"), device=device)
    T.assemble_tree_factor_solve_iters(scratch, M, J, D, t(b.state), N, G, x3)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(x.cpu().numpy(), R.tree_ldl_solve(*st, oplan, b.M, b.grad))
    for it in range(3):
        np.testing.assert_array_equal(x3[it].cpu().numpy(), R.assemble_tree_ldl_solve(*st, oplan, b.M, b.J, b.D, b.state[it], b.nefc, b.grad))


@pytest.mark.gpu
def test_gpu_attach_checks_the_structure(device):
    import torch

    from instantmimic_amd.mjw_kernels import tree_ldl as T

    st, groups, trunk, _ = build._plan_of_tree(TREES["limbs"])
    other = jit.code_object(st, groups, trunk)
    b = _batch("branched", 8)
    st_b = T.tree_ldl_structure(b.rowadr, b.rownnz, b.colind)
    with torch.cuda.device(device):
        handle = T._PlanHandle(st_b, 0, host_only=False)
        buf = C.create_string_buffer(other, len(other))
        assert _lib.lib().im_tree_plan_attach_kernels(handle.ptr, buf) == _lib.IM_ERR_STRUCTURE  # generated for another tree
        assert jit.attach(handle.ptr, handle.structure, handle.plan().groups, handle.plan().trunk)
        mine = jit.code_object(handle.structure, handle.plan().groups, handle.plan().trunk)
        assert _lib.lib().im_tree_plan_attach_kernels(handle.ptr, C.create_string_buffer(mine, len(mine))) == _lib.IM_ERR_ARG  # once per plan
    # a benchmark tree has its kernels in the library: nothing to attach
    h = synth.make_batch("humanoid", 4)
    scratch = T.create_tree_factor_solve_scratch(type("m", (), dict(nv=27, M_rowadr=h.rowadr, M_rownnz=h.rownnz, M_colind=h.colind)), device)
    assert _has_kernel(scratch)
