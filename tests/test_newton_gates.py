"""Capability boundaries of the fused Newton loop: which models it takes, the block width, the
modes that keep the stock path (reference: src/instantmimic/utils/mjw_kernels/newton_fusion.py
:307-327; the cases are the reference's own, tests/test_mjw_newton_fusion.py:31-98) and the
iteration bound of ``run``."""

from types import SimpleNamespace

import pytest

from instantmimic_amd.mjw_kernels import newton_fusion as fusion
from instantmimic_amd.mjw_kernels import sparse_hessian

# mujoco_warp's enums are not importable here: members with a name, as the model would carry them
NEWTON, CG = SimpleNamespace(name="NEWTON", value=2), SimpleNamespace(name="CG", value=1)
PYRAMIDAL, ELLIPTIC = SimpleNamespace(name="PYRAMIDAL", value=0), SimpleNamespace(name="ELLIPTIC", value=1)
IMPLICITFAST, DISCRETE = SimpleNamespace(name="IMPLICITFAST", value=3), SimpleNamespace(name="DISCRETE", value=4)


def _model(**updates):
    model = SimpleNamespace(
        nv=34, nv_pad=48, is_sparse=False,
        opt=SimpleNamespace(solver=NEWTON, cone=PYRAMIDAL, iterations=4, integrator=IMPLICITFAST),
        block_dim=SimpleNamespace(linesearch_iterative=32),
        body_parentid=SimpleNamespace(device=SimpleNamespace(is_cuda=True)),
    )  # fmt: skip
    for key, value in updates.items():
        setattr(model, key, value)
    return model


@pytest.mark.parametrize("nv,pad,expected", [
    (0, 0, False), (12, 12, False), (13, 16, True), (16, 16, True), (17, 32, True), (31, 32, True), (32, 32, True),
    (32, 48, True), (33, 48, True), (35, 48, True), (56, 64, True), (60, 64, True), (61, 64, True), (64, 80, True),
    (70, 80, True), (79, 80, True), (80, 96, False), (34, 40, False),
])  # fmt: skip
def test_eligibility_uses_dof_layout_not_model_name(nv, pad, expected):
    assert fusion.eligible(_model(nv=nv, nv_pad=pad), object()) is expected


@pytest.mark.parametrize("pad,expected", [(32, 32), (48, 32), (64, 64), (80, 64)])
def test_newton_block_width_uses_padded_dof_layout(pad, expected):
    assert fusion.newton_block_dim(_model(nv_pad=pad)) == expected
    assert sparse_hessian.block_width(pad) == expected


@pytest.mark.parametrize("reason", ["compact", "sparse", "sparse_compact", "cg", "discrete", "elliptic", "zero_iterations",
                                    "reduction_layout", "cpu_device"])  # fmt: skip
def test_unsupported_solver_modes_keep_original_path(reason):
    model, ctx = _model(), SimpleNamespace(sparse_compact=reason == "sparse_compact")
    if reason == "sparse":
        model.is_sparse = True
    if reason == "discrete":
        model.opt.integrator = DISCRETE
    if reason == "cg":
        model.opt.solver = CG
    if reason == "elliptic":
        model.opt.cone = ELLIPTIC
    if reason == "zero_iterations":
        model.opt.iterations = 0
    if reason == "reduction_layout":
        model.block_dim.linesearch_iterative = 64
    if reason == "cpu_device":
        model.body_parentid.device.is_cuda = False
    assert fusion.eligible(_model(), SimpleNamespace(sparse_compact=False))
    assert not fusion.eligible(model, ctx, compact=reason == "compact")


def test_enum_members_match_by_name_or_by_mujocos_numbers():
    plain = _model()
    plain.opt = SimpleNamespace(solver=2, cone=0, iterations=4, integrator=3)  # mjSOL_NEWTON, mjCONE_PYRAMIDAL
    assert fusion.eligible(plain, None)
    plain.opt.solver = 1
    assert not fusion.eligible(plain, None)
    # a model that says nothing of a field the reference reads does not qualify
    silent = _model()
    del silent.is_sparse
    assert not fusion.eligible(silent, None)
    # an explicit use_incremental overrides the solver reading (upstream's _use_incremental)
    assert not fusion.eligible(_model(use_incremental=False), None)


def test_upstream_iteration_gate():
    ctx = SimpleNamespace(hfactor=SimpleNamespace(shape=(8, 48, 48)), sparse_compact=False)
    assert fusion.upstream_newton_structure(_model(), ctx)
    assert not fusion.upstream_newton_structure(_model(), ctx, compact=True)
    assert not fusion.upstream_newton_structure(_model(nv_pad=64), ctx)
    assert not fusion.upstream_newton_structure(_model(), SimpleNamespace(hfactor=None))
    cg = _model()
    cg.opt.solver = CG
    assert not fusion.upstream_newton_structure(cg, ctx)
