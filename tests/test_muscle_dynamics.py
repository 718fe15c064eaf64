"""Muscle path geometry, activation -> torque operator and its gradient.

CPU tests pin the oracle against fp64 formulations that share no code with it (rotation
matrices, dense subtree masks instead of entry lists, the closed form of the reference's
own two-body fixture); GPU tests compare libimhip with the oracle bit for bit wherever only
IEEE-exact operations are involved and to 2e-6 where expf/cosf enter.
"""

import gc

import numpy as np
import pytest
import torch

from instantmimic_amd import synth
from instantmimic_amd.muscle import warp_custom_ops as ops
from instantmimic_amd.muscle.muscle_dynamics import (
    MuscleDynamicsLayer,
    MuscleMechanics,
    MuscleTopology,
    build_dof_subtree_mask,
    build_muscle_sparse_torque_entries,
    build_torque_sparse_segment_entries,
)
from oracle import ref

FORCE_RTOL = 2e-6  # expf / cosf differ by a few ulp between libm and the GPU


# ---------------------------------------------------------------- fixtures


def fixture_layer(device="cpu", muscle_count=3, torque_dim=2, root_dof_count=6, mechanics=None):
    """The layer of the reference's tests/muscle_warp_fixtures.py:17-131: two bodies, one
    segment per muscle from (0,1,0) on the root body to (1,1,0) on the child."""
    nv = torque_dim + root_dof_count
    idx = np.arange(muscle_count)
    topo = MuscleTopology(
        muscle_params=np.tile(np.float32([[1.0, 1.0, 0.0, 0.0, 1.0]]), (muscle_count, 1)),
        muscle_rest_length=np.ones(muscle_count, np.float32),
        muscle_waypoints_local=np.tile(np.float32([[0, 1, 0], [1, 1, 0]]), (muscle_count, 1)),
        muscle_waypoint_body=np.tile([0, 1], muscle_count),
        all_segment_muscle_idx=idx, all_segment_start_idx=idx * 2, apply_segment_muscle_idx=idx,
        apply_segment_start_idx=idx * 2, apply_segment_end_idx=idx * 2 + 1,
        apply_segment_body_start_idx=np.zeros_like(idx), apply_segment_body_end_idx=np.ones_like(idx),
        body_parentid=np.array([0, 0]), body_rootid=np.array([0, 0]), dof_bodyid=np.array([0] * (nv - 1) + [1]),
    )  # fmt: skip
    mech = mechanics or MuscleMechanics(length_norm_min=0.2, length_norm_max=1.4)
    return MuscleDynamicsLayer(topo, body_count=2, full_torque_dim=nv, torque_dim=torque_dim,
                               muscle_count=muscle_count, mechanics=mech, device=device)  # fmt: skip


def fixture_context(layer, batch=4):
    """tests/muscle_warp_fixtures.py:151-180: child body at x = 1, identity orientations,
    the last torque dof rotates about z."""
    body = np.zeros((batch, layer.body_count, 3), np.float32)
    body[:, 1, 0] = 1.0
    quat = np.zeros((batch, layer.body_count, 4), np.float32)
    quat[..., 0] = 1.0
    cdof = np.zeros((batch, layer.full_torque_dim, 6), np.float32)
    cdof[:, layer.root_dof_count + layer.torque_dim - 1, 2] = 1.0
    flat = [a.reshape(batch, int(np.prod(a.shape[1:]))) for a in (body, quat, body, body, cdof)]
    return np.concatenate(flat, axis=1)


def split_context(layer, ctx):
    nb, nv = layer.body_count, layer.full_torque_dim
    B = ctx.shape[0]
    xpos = ctx[:, : 3 * nb].reshape(B, nb, 3)
    xquat = ctx[:, 3 * nb : 7 * nb].reshape(B, nb, 4)
    com = ctx[:, 10 * nb : 13 * nb].reshape(B, nb, 3)
    cdof = ctx[:, 13 * nb : 13 * nb + 6 * nv].reshape(B, nv, 6)
    return xpos, xquat, com, cdof


def model9(mech: MuscleMechanics):
    return np.float32([mech.force_scale, mech.length_norm_min, mech.length_norm_max, *mech.active_params(),
                       *mech.passive_params()])  # fmt: skip


def oracle_forward(layer, ctx, act, include_passive, unit=None, passive=None, waypoints=None):
    xpos, xquat, com, cdof = split_context(layer, ctx)
    wp = ref.muscle_waypoints(xpos, xquat, layer.waypoint_body, layer.waypoints_local) if waypoints is None else waypoints
    if unit is None:
        unit, passive = ref.muscle_force_magnitudes(
            wp, layer.all_segment_start_idx, layer.all_muscle_segment_offsets, layer.muscle_params,
            layer.muscle_rest_length, model9(layer.mechanics), include_passive,
        )  # fmt: skip
    tq = layer.torque_entries_host
    out = ref.muscle_torque_forward(
        wp, com, cdof, layer.segments_host, (tq[0], tq[2], tq[3], tq[4], tq[5]), unit,
        passive if include_passive else None, act, layer.root_dof_count,
    )  # fmt: skip
    return out, wp, unit, passive


def oracle_backward(layer, ctx, gout, wp, unit):
    _, _, com, cdof = split_context(layer, ctx)
    return ref.muscle_activation_grad(wp, com, cdof, layer.segments_host, layer.muscle_entries_host, unit, gout,
                                      layer.root_dof_count)  # fmt: skip


# ---------------------------------------------------------------- fp64 references (independent)


def rotmat64(q):
    q = q.astype(np.float64)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-8)
    w, x, y, z = np.moveaxis(q, -1, 0)
    return np.stack(
        [1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y),
         2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x),
         2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)], axis=-1,
    ).reshape(q.shape[:-1] + (3, 3))  # fmt: skip


def waypoints64(layer, xpos, xquat):
    R = rotmat64(xquat)[:, layer.waypoint_body]
    return xpos.astype(np.float64)[:, layer.waypoint_body] + np.einsum("bwij,wj->bwi", R, layer.waypoints_local.astype(np.float64))


def curves64(mech, ln):
    if mech.active_force_type == "gaussian":
        fa = np.exp(-((ln - 1) ** 2) / mech.active_force_gamma)
    else:
        lmin, lmax = mech.active_force_lmin, mech.active_force_lmax
        lo, hi = 0.5 * (lmin + 1), 0.5 * (1 + lmax)
        fa = np.select(
            [(ln < lmin) | (ln > lmax), ln <= lo, ln <= 1.0, ln <= hi],
            [0.0, 0.5 * ((ln - lmin) / (lo - lmin)) ** 2, 1 - 0.5 * ((1 - ln) / (1 - lo)) ** 2,
             1 - 0.5 * ((ln - 1) / (hi - 1)) ** 2],
            0.5 * ((lmax - ln) / (lmax - hi)) ** 2,
        )  # fmt: skip
    if mech.passive_force_type == "exponential":
        k, e = mech.passive_force_k_pe, mech.passive_force_e_mo
        fp = np.where(ln < 1, 0.0, (np.exp(np.clip(k * (ln - 1) / e, -80, 80)) - 1) / (np.exp(k) - 1))
    else:
        lmax, fpmax = mech.passive_force_lmax, mech.passive_force_fpmax
        mid = 0.5 * (1 + lmax)
        w = mid - 1
        fp = np.select([ln <= 1, ln <= mid], [0.0, 0.5 * fpmax * ((ln - 1) / w) ** 2], fpmax * (0.5 + (ln - mid) / w))
    return fa, fp


def forces64(layer, wp):
    mech = layer.mechanics
    seg_len = np.linalg.norm(wp[:, layer.all_segment_start_idx + 1] - wp[:, layer.all_segment_start_idx], axis=-1)
    length = np.zeros((wp.shape[0], layer.muscle_count))
    muscle_of = np.repeat(np.arange(layer.muscle_count), np.diff(layer.all_muscle_segment_offsets))
    np.add.at(length, (slice(None), muscle_of), seg_len)
    p = layer.muscle_params.astype(np.float64)
    ln = np.clip((length / np.maximum(layer.muscle_rest_length, 1e-6) - p[:, 2]) / np.maximum(p[:, 1], 1e-6),
                 np.float32(mech.length_norm_min), np.float32(mech.length_norm_max))  # fmt: skip
    fa, fp = curves64(mech, ln)
    gain = p[:, 0] * np.cos(p[:, 3]) * mech.force_scale
    return gain * fa, gain * fp, ln


def moment_matrix64(layer, wp, com, cdof):
    """T[b, j, m] = d torque_j / d force_m from the dense subtree masks."""
    p0i, p1i, b0, b1 = layer.segments_host
    com = com.astype(np.float64)
    cd = cdof.astype(np.float64)[:, layer.root_dof_count :]
    ang, lin = cd[..., :3], cd[..., 3:]
    p0, p1 = wp[:, p0i], wp[:, p1i]
    seg = p1 - p0
    length = np.linalg.norm(seg, axis=-1, keepdims=True)
    u = np.where(length < 1e-8, 0.0, seg / np.maximum(length, 1e-300))
    r0, r1 = p0 - com[:, b0], p1 - com[:, b1]
    # (lin + ang x r) . u = lin . u + ang . (r x u)
    t0 = np.einsum("bjc,bsc->bjs", lin, u) + np.einsum("bjc,bsc->bjs", ang, np.cross(r0, u))
    t1 = np.einsum("bjc,bsc->bjs", lin, u) + np.einsum("bjc,bsc->bjs", ang, np.cross(r1, u))
    per_seg = layer.segment_start_dof_mask[None] * t0 - layer.segment_end_dof_mask[None] * t1
    onehot = np.zeros((len(p0i), layer.muscle_count))
    onehot[np.arange(len(p0i)), layer.apply_segment_muscle_idx] = 1.0
    return per_seg @ onehot


@pytest.fixture(scope="module")
def rig_layer():
    rig = synth.make_muscle_rig(nmuscle=60, seed=5)
    mech = MuscleMechanics(length_norm_min=0.2, length_norm_max=1.8)
    return rig, MuscleDynamicsLayer(rig.topology, **rig.dims(), mechanics=mech, device="cpu")


# ---------------------------------------------------------------- host tables


def test_subtree_mask_and_entry_tables():
    parent = [0, 0, 1, 2, 1]
    dof_body = [0, 0, 1, 2, 2, 3, 4]
    mask = build_dof_subtree_mask(parent, dof_body, 5, 7)
    # brute force: dof on body d moves body b when d is b or an ancestor of b; world dofs move all
    for d, db in enumerate(dof_body):
        for b in range(5):
            chain, p = [], b
            while p != 0:
                chain.append(p)
                p = parent[p]
            assert mask[d, b] == (1.0 if db == 0 or db in chain else 0.0)
    rng = np.random.default_rng(3)
    start = (rng.random((5, 9)) < 0.4).astype(np.float32)
    end = (rng.random((5, 9)) < 0.4).astype(np.float32)
    muscle = rng.integers(0, 4, 9)
    off, tq, seg, mus, a, b = build_torque_sparse_segment_entries(start, end, muscle)
    want = [(j, s) for j in range(5) for s in range(9) if start[j, s] or end[j, s]]
    assert list(zip(tq.tolist(), seg.tolist())) == want
    assert off.tolist() == [sum(1 for j, _ in want if j < k) for k in range(6)]
    assert np.array_equal(mus, muscle[seg]) and np.array_equal(a, start[tq, seg]) and np.array_equal(b, end[tq, seg])
    moff, mseg, mtq, ma, mb = build_muscle_sparse_torque_entries(off, seg, a, b, muscle, 4)
    keys = [(int(muscle[s]), int(s), int(j)) for s, j in zip(mseg, mtq)]
    assert keys == sorted((int(muscle[s]), s, j) for j, s in want)
    assert moff.tolist() == [sum(1 for k in keys if k[0] < m) for m in range(5)]
    assert np.array_equal(ma, start[mtq, mseg]) and np.array_equal(mb, end[mtq, mseg])


def test_layer_validates_its_inputs():
    with pytest.raises(ValueError):
        MuscleMechanics(active_force_type="cubic")
    with pytest.raises(ValueError):
        MuscleMechanics(active_force_lmin=1.2)
    with pytest.raises(NotImplementedError):
        MuscleMechanics(force_velocity_enabled=True)
    layer = fixture_layer()
    with pytest.raises(RuntimeError, match="no CPU path"):
        layer._warp_muscle_dynamics_from_activation_forward(
            torch.zeros(4, 3), torch.from_numpy(fixture_context(layer)), include_passive_force=False
        )


# ---------------------------------------------------------------- oracle pinning


def test_oracle_waypoints_against_rotation_matrices(rig_layer):
    rig, layer = rig_layer
    ctx = synth.make_muscle_context(rig, 16, seed=2)
    xpos, xquat, _, _ = split_context(layer, ctx)
    got = ref.muscle_waypoints(xpos, xquat, layer.waypoint_body, layer.waypoints_local)
    want = waypoints64(layer, xpos, xquat)
    assert np.abs(got - want).max() < 2e-6
    # identity orientation: a pure translation, exactly
    q = np.zeros_like(xquat)
    q[..., 0] = 1.0
    got = ref.muscle_waypoints(xpos, q, layer.waypoint_body, layer.waypoints_local)
    assert np.abs(got - (xpos[:, layer.waypoint_body] + layer.waypoints_local)).max() < 1e-7


@pytest.mark.parametrize("active", ["gaussian", "mujoco"])
@pytest.mark.parametrize("passive", ["exponential", "mujoco"])
def test_oracle_force_magnitudes_against_fp64_curves(active, passive):
    rig = synth.make_muscle_rig(nmuscle=60, seed=5)
    mech = MuscleMechanics(active_force_type=active, passive_force_type=passive, length_norm_min=0.2, length_norm_max=1.8)
    layer = MuscleDynamicsLayer(rig.topology, **rig.dims(), mechanics=mech, device="cpu")
    ctx = synth.make_muscle_context(rig, 32, seed=4)
    ctx[:, : 3 * rig.body_count] *= 0.5  # spread the normalised lengths over every branch of the curves
    xpos, xquat, _, _ = split_context(layer, ctx)
    wp = ref.muscle_waypoints(xpos, xquat, layer.waypoint_body, layer.waypoints_local)
    unit, pas = ref.muscle_force_magnitudes(wp, layer.all_segment_start_idx, layer.all_muscle_segment_offsets,
                                            layer.muscle_params, layer.muscle_rest_length, model9(mech), True)  # fmt: skip
    u64, p64, ln = forces64(layer, wp.astype(np.float64))
    assert (ln < 1).any() and (ln > 1.3).any() and ((ln > 1) & (ln < 1.3)).any()
    scale = layer.muscle_params[:, 0].max()
    assert np.abs(unit - u64).max() < 2e-5 * scale
    assert np.abs(pas - p64).max() < 2e-5 * max(scale, np.abs(p64).max())
    _, zero = ref.muscle_force_magnitudes(wp, layer.all_segment_start_idx, layer.all_muscle_segment_offsets,
                                          layer.muscle_params, layer.muscle_rest_length, model9(mech), False)  # fmt: skip
    assert not zero.any()


def test_oracle_on_the_reference_fixture_closed_form():
    layer = fixture_layer()
    ctx = fixture_context(layer)
    act = np.float32([[0.1, 0.5, 0.9]] * 4)
    out, wp, unit, _ = oracle_forward(layer, ctx, act, False)
    # waypoints (0,1,0) and (2,1,0): length 2, normalised length clamped to 1.4
    assert np.array_equal(wp[0].reshape(-1, 3)[:2], np.float32([[0, 1, 0], [2, 1, 0]]))
    u = np.exp(-(0.4**2) / 0.45)
    assert np.allclose(unit, u, rtol=1e-6)
    # only the child's z rotation sees the muscles: lever (2,1,0), pull along x => torque = +F
    assert np.all(out[:, 0] == 0)
    assert np.allclose(out[:, 1], u * act.sum(1), rtol=1e-6)
    grad = oracle_backward(layer, ctx, np.float32([[0.0, 2.0]] * 4), wp, unit)
    assert np.allclose(grad, 2.0 * u, rtol=1e-6)


def test_oracle_contractions_against_dense_fp64(rig_layer):
    rig, layer = rig_layer
    B = 8
    ctx = synth.make_muscle_context(rig, B, seed=7)
    rng = np.random.default_rng(11)
    act = rng.uniform(0, 1, (B, rig.muscle_count)).astype(np.float32)
    act[:, ::7] = 0.0  # exercises the force == 0 skip
    out, wp, unit, pas = oracle_forward(layer, ctx, act, True)
    _, _, com, cdof = split_context(layer, ctx)
    T = moment_matrix64(layer, wp.astype(np.float64), com, cdof)  # (B, torque, muscle)
    force = unit.astype(np.float64) * act + pas
    want = np.einsum("bjm,bm->bj", T, force)
    assert ref.rel_l2(out, want) < 2e-6
    no_passive, *_ = oracle_forward(layer, ctx, act, False)
    assert ref.rel_l2(no_passive, np.einsum("bjm,bm->bj", T, unit.astype(np.float64) * act)) < 2e-6
    # gradient = transpose of the same linear map, scaled by the unit force
    g = rng.normal(0, 1, (B, rig.torque_dim)).astype(np.float32)
    grad = oracle_backward(layer, ctx, g, wp, unit)
    assert ref.rel_l2(grad, np.einsum("bjm,bj->bm", T, g.astype(np.float64)) * unit) < 2e-6
    # sparse moment: the nonzero pattern of T, entry by entry
    e = layer.sparse_entries
    mom = ref.muscle_sparse_moment(wp, com, cdof, layer.segments_host, e.muscle_dof_torque_idx,
                                   e.muscle_dof_segment_offsets, e.segment_idx, e.start_coeff, e.end_coeff,
                                   layer.root_dof_count)  # fmt: skip
    assert ref.rel_l2(mom, T[:, e.muscle_dof_torque_idx, e.muscle_dof_muscle_idx]) < 2e-6
    dense = np.zeros_like(T)
    dense[:, e.muscle_dof_torque_idx, e.muscle_dof_muscle_idx] = mom
    assert np.abs(dense - T).max() < 1e-5 * np.abs(T).max()  # nothing of T lies off the entry list


def test_oracle_bounds_against_dense_fp64(rig_layer):
    rig, layer = rig_layer
    ctx = synth.make_muscle_context(rig, 8, seed=17)
    _, wp, unit, _ = oracle_forward(layer, ctx, np.ones((8, rig.muscle_count), np.float32), False)
    _, _, com, cdof = split_context(layer, ctx)
    tq = layer.torque_entries_host
    lo, hi = ref.muscle_torque_bounds(wp, com, cdof, layer.segments_host, (tq[0], tq[2], tq[3], tq[4], tq[5]), unit,
                                      layer.root_dof_count)  # fmt: skip
    per_muscle = moment_matrix64(layer, wp.astype(np.float64), com, cdof) * unit[:, None, :]
    assert ref.rel_l2(lo, np.minimum(per_muscle, 0).sum(-1)) < 2e-6
    assert ref.rel_l2(hi, np.maximum(per_muscle, 0).sum(-1)) < 2e-6
    assert (lo <= 0).all() and (hi >= 0).all()


def test_oracle_degenerate_segment_contributes_nothing():
    layer = fixture_layer()
    ctx = fixture_context(layer)
    ctx[:, 3] = -1.0  # child body at x = -1: both waypoints coincide at (0,1,0)
    out, wp, unit, _ = oracle_forward(layer, ctx, np.ones((4, 3), np.float32), False)
    assert np.array_equal(wp[0].reshape(-1, 3)[0], wp[0].reshape(-1, 3)[1])
    assert not out.any()


# ---------------------------------------------------------------- operator registry (no GPU)


def test_operator_schemas_and_registry():
    fwd = torch.ops.instantmimic_muscle.torque_forward.default
    bwd = torch.ops.instantmimic_muscle.torque_backward.default
    assert str(fwd._schema) == (
        "instantmimic_muscle::torque_forward(Tensor activation, Tensor raw_context, SymInt layer_key, "
        "bool include_passive_force) -> Tensor"
    )
    assert str(bwd._schema) == (
        "instantmimic_muscle::torque_backward(Tensor raw_context, Tensor grad_output, SymInt layer_key) -> Tensor"
    )
    layer = fixture_layer()
    key = ops.warp_op_key(layer)
    assert ops.warp_op_key(layer) == key and ops._layer_for(key) is layer
    import copy

    clone = copy.copy(layer)
    assert clone._warp_op_key == key and ops.warp_op_key(clone) != key  # a copy gets its own handle
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        a = torch.empty(5, 3)
        c = torch.empty(5, layer.context_dim)
        assert ops.muscle_torque_forward(a, c, key, False).shape == (5, 2)
        assert ops.muscle_torque_backward(c, torch.empty(5, 2), key).shape == (5, 3)
        u = torch.empty(5, 3)
        assert ops.muscle_torque_cached_lbs_forward(a, c, u, u, key, True).shape == (5, 2)
        assert ops.muscle_torque_cached_lbs_backward(c, u, torch.empty(5, 2), key).shape == (5, 3)
        lo, hi = ops.muscle_torque_bounds(c, key, True)
        assert lo.shape == hi.shape == (5, 2)
    del layer
    gc.collect()
    with pytest.raises(RuntimeError, match="not registered"):
        ops._layer_for(key)


# ---------------------------------------------------------------- GPU parity


def _gpu_layer(rig, **mech):
    m = MuscleMechanics(length_norm_min=0.2, length_norm_max=1.8, **mech)
    return MuscleDynamicsLayer(rig.topology, **rig.dims(), mechanics=m, device="cuda")


@pytest.mark.gpu
@pytest.mark.parametrize("active,passive", [("gaussian", "exponential"), ("mujoco", "mujoco")])
@pytest.mark.parametrize("nworld", [1, 67, 1024])
def test_gpu_geometry_forward_backward_match_oracle(active, passive, nworld):
    rig = synth.make_muscle_rig(nmuscle=284, seed=1003)
    layer = _gpu_layer(rig, active_force_type=active, passive_force_type=passive)
    ctx = synth.make_muscle_context(rig, nworld, seed=9)
    ctx[:, : 3 * rig.body_count] *= 0.5
    rng = np.random.default_rng(13)
    act = rng.uniform(0, 1, (nworld, rig.muscle_count)).astype(np.float32)
    act[:, ::5] = 0.0
    g = rng.normal(0, 1, (nworld, rig.torque_dim)).astype(np.float32)
    ctx_d, act_d = torch.from_numpy(ctx).cuda(), torch.from_numpy(act).cuda()
    for include_passive in (False, True):
        mean, wp_d, unit_d = layer._warp_muscle_dynamics_from_activation_forward(
            act_d, ctx_d, include_passive_force=include_passive
        )
        ws, _ = layer._prepare_waypoint_geometry(ctx_d, include_passive_force_magnitude=include_passive)
        torch.cuda.synchronize()
        wp = wp_d.cpu().numpy().reshape(nworld, -1, 3)
        unit, pas = unit_d.cpu().numpy(), ws["passive_force_magnitude"].cpu().numpy()
        want, wp_o, unit_o, pas_o = oracle_forward(layer, ctx, act, include_passive)
        assert np.array_equal(wp, wp_o)  # IEEE-exact operations only
        scale = np.abs(unit_o).max()
        assert np.abs(unit - unit_o).max() <= FORCE_RTOL * scale
        assert np.abs(pas - pas_o).max() <= FORCE_RTOL * max(scale, np.abs(pas_o).max())
        if not include_passive:
            assert not pas.any()
        # the contraction itself, from the GPU's own force magnitudes: bit exact
        exact, *_ = oracle_forward(layer, ctx, act, include_passive, unit=unit, passive=pas, waypoints=wp)
        assert np.array_equal(mean.cpu().numpy(), exact)
        assert ref.rel_l2(mean.cpu().numpy(), want) < 1e-5
    grad = layer._warp_muscle_dynamics_from_activation_backward(ctx_d, torch.from_numpy(g).cuda())
    assert np.array_equal(grad.cpu().numpy(), oracle_backward(layer, ctx, g, wp, unit))
    cached = layer._warp_muscle_dynamics_from_activation_backward(ctx_d, torch.from_numpy(g).cuda(), unit_d)
    assert torch.equal(cached, grad)


@pytest.mark.gpu
def test_gpu_sparse_moment_matches_oracle_and_feeds_the_projection():
    from instantmimic_amd.muscle import muscle_qfrc_projector as proj

    rig = synth.make_muscle_rig(nmuscle=284, seed=1003)
    layer = _gpu_layer(rig)
    nworld = 257
    ctx = synth.make_muscle_context(rig, nworld, seed=21)
    ctx_d = torch.from_numpy(ctx).cuda()
    mom = layer.eval_muscle_sparse_moment(ctx_d)
    ws, _ = layer._prepare_waypoint_geometry(ctx_d, include_passive_force_magnitude=False)
    wp = ws["transformed_waypoints"].cpu().numpy().reshape(nworld, -1, 3)
    _, _, com, cdof = split_context(layer, ctx)
    e = layer.sparse_entries
    want = ref.muscle_sparse_moment(wp, com, cdof, layer.segments_host, e.muscle_dof_torque_idx,
                                    e.muscle_dof_segment_offsets, e.segment_idx, e.start_coeff, e.end_coeff,
                                    layer.root_dof_count)  # fmt: skip
    assert np.array_equal(mom.cpu().numpy(), want)
    # tau = A' f through the projection kernel equals the operator's torque to rounding
    act = torch.rand(nworld, rig.muscle_count, device="cuda")
    force = ws["unit_force_magnitude"] * act
    offsets, entry_idx = proj.torque_sorted_entries(e.muscle_dof_torque_idx, rig.torque_dim)
    qfrc = torch.zeros(nworld, rig.full_torque_dim, device="cuda")
    proj.project_muscle_sparse_moment_qfrc(
        mom, force, torch.from_numpy(offsets).cuda(), torch.from_numpy(entry_idx).cuda(),
        torch.from_numpy(e.muscle_dof_muscle_idx.astype(np.int32)).cuda(), layer.root_dof_count, qfrc,
    )  # fmt: skip
    torque = layer.forward_from_activation(act, ctx_d, False)
    assert ref.rel_l2(qfrc[:, layer.root_dof_count :].cpu().numpy(), torque.cpu().numpy()) < 1e-5
    assert not qfrc[:, : layer.root_dof_count].any()


@pytest.mark.gpu
def test_gpu_operator_fixture_closed_form_autograd_and_compile():
    layer = fixture_layer("cuda")
    ctx = torch.from_numpy(fixture_context(layer)).cuda()
    key = ops.warp_op_key(layer)
    u = float(np.exp(-(0.4**2) / 0.45))

    def loss(a):
        return ops.muscle_torque_forward(a.sin(), ctx, key, False).square().sum()

    a = torch.full((4, 3), 0.4, device="cuda", requires_grad=True)
    value = loss(a)
    (grad,) = torch.autograd.grad(value, a)
    s, c = np.sin(0.4), np.cos(0.4)
    assert abs(value.item() - 4 * (3 * u * s) ** 2) < 1e-5 * value.item()
    assert torch.allclose(grad, torch.full_like(grad, 2 * (3 * u * s) * u * c), rtol=1e-5)
    assert torch.count_nonzero(grad) > 0
    # strict fullgraph compilation reaches the kernels only through the dispatcher operators
    compiled = torch.compile(loss, fullgraph=True, backend="aot_eager")
    b = torch.full((4, 3), 0.4, device="cuda", requires_grad=True)
    cvalue = compiled(b)
    (cgrad,) = torch.autograd.grad(cvalue, b)
    assert torch.equal(cvalue, value) and torch.equal(cgrad, grad)
    # the autograd node keeps the layer alive after the caller dropped it
    pending = loss(torch.full((4, 3), 0.2, device="cuda", requires_grad=True))
    del layer
    gc.collect()
    pending.backward()


@pytest.mark.gpu
def test_gpu_cached_force_ops_and_bounds():
    rig = synth.make_muscle_rig(nmuscle=284, seed=1003)
    active = np.arange(0, rig.torque_dim, 3)
    layer = MuscleDynamicsLayer(rig.topology, **rig.dims(), mechanics=MuscleMechanics(), active_torque_indices=active,
                                device="cuda")  # fmt: skip
    nworld = 93
    ctx = synth.make_muscle_context(rig, nworld, seed=31)
    ctx_d = torch.from_numpy(ctx).cuda()
    key = ops.warp_op_key(layer)
    act = torch.rand(nworld, rig.muscle_count, device="cuda", requires_grad=True)
    torque = ops.muscle_torque_forward(act, ctx_d, key, True)
    ws, _ = layer._prepare_waypoint_geometry(ctx_d, include_passive_force_magnitude=True)
    unit, pas = ws["unit_force_magnitude"], ws["passive_force_magnitude"]
    cached = ops.muscle_torque_cached_lbs_forward(act, ctx_d, unit, pas, key, True)
    assert torch.equal(cached, torque)
    g = torch.randn_like(torque)
    (g1,) = torch.autograd.grad(torque, act, g, retain_graph=True)
    (g2,) = torch.autograd.grad(cached, act, g)
    assert torch.equal(g1, g2) and torch.count_nonzero(g1) > 0
    lo, hi = ops.muscle_torque_bounds(ctx_d, key, False)
    wp = ws["transformed_waypoints"].cpu().numpy().reshape(nworld, -1, 3)
    _, _, com, cdof = split_context(layer, ctx)
    tq = layer.torque_entries_host
    want_lo, want_hi = ref.muscle_torque_bounds(wp, com, cdof, layer.segments_host,
                                                (tq[0], tq[2], tq[3], tq[4], tq[5]), unit.cpu().numpy(),
                                                layer.root_dof_count)  # fmt: skip
    assert np.array_equal(lo.cpu().numpy(), want_lo) and np.array_equal(hi.cpu().numpy(), want_hi)
    # activations in [0, 1] without passive force stay inside the box
    inside = ops.muscle_torque_forward(act.detach(), ctx_d, key, False)
    tol = 1e-4 * hi.abs().max()
    assert (inside >= lo - tol).all() and (inside <= hi + tol).all()
    slo, shi = ops.muscle_torque_bounds(ctx_d, key, True)
    assert torch.equal(slo, lo[:, active]) and torch.equal(shi, hi[:, active])


@pytest.mark.gpu
def test_gpu_edge_cases():
    layer = fixture_layer("cuda")
    ctx = torch.from_numpy(fixture_context(layer, batch=0)).cuda()
    out, _, _ = layer._warp_muscle_dynamics_from_activation_forward(
        torch.zeros(0, 3, device="cuda"), ctx, include_passive_force=True
    )
    assert out.shape == (0, 2)
    # a context that carries trailing columns (strided rows) and degenerate segments
    full = fixture_context(layer, batch=5)
    full[:, 3] = -1.0
    wide = torch.zeros(5, layer.context_dim + 9, device="cuda")
    wide[:, : layer.context_dim] = torch.from_numpy(full).cuda()
    out, _, _ = layer._warp_muscle_dynamics_from_activation_forward(
        torch.ones(5, 3, device="cuda"), wide[:, : layer.context_dim + 3], include_passive_force=False
    )
    assert not out.any()
    with pytest.raises(ValueError):
        layer._warp_muscle_dynamics_from_activation_forward(
            torch.ones(5, 2, device="cuda"), wide, include_passive_force=False
        )
    with pytest.raises(ValueError, match="columns"):
        layer._warp_muscle_dynamics_from_activation_forward(
            torch.ones(5, 3, device="cuda"), wide[:, :20].contiguous(), include_passive_force=False
        )


@pytest.mark.gpu
def test_gpu_one_thread_per_output_kernels_agree():
    """The contractions have two kernels each (a workgroup per world with the segments staged in
    LDS, and one thread per output for models that do not fit): the second one is forced here
    in a child process and must pass the same oracle comparison."""
    import os
    import subprocess
    import sys

    env = dict(os.environ, IMHIP_MUSCLE_KERNEL="simple")
    code = (
        "import sys; sys.path.insert(0, 'tests'); import test_muscle_dynamics as t;"
        "t.test_gpu_geometry_forward_backward_match_oracle('gaussian', 'exponential', 67);"
        "t.test_gpu_sparse_moment_matches_oracle_and_feeds_the_projection();"
        "t.test_gpu_cached_force_ops_and_bounds(); print('simple kernels ok')"
    )
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "simple kernels ok" in out.stdout, out.stderr[-2000:]


@pytest.mark.gpu
@pytest.mark.parametrize("nworld", [1, 333])
def test_gpu_fused_geometry_equals_the_two_launches(nworld):
    """im_muscle_waypoints_forces against im_muscle_waypoints followed by
    im_muscle_force_magnitudes, through the C-ABI: the same bits, rows beyond the outputs'
    widths untouched."""
    import ctypes as C

    from instantmimic_amd import _lib

    rig = synth.make_muscle_rig(nmuscle=284, seed=1003)
    layer = _gpu_layer(rig, active_force_type="gaussian", passive_force_type="exponential")
    ctx_d = torch.from_numpy(synth.make_muscle_context(rig, nworld, seed=21)).cuda()
    ws, _ = layer._prepare_waypoint_geometry(ctx_d, include_passive_force_magnitude=True)
    d, L = layer._dev, _lib.lib()
    base, ld = ctx_d.data_ptr(), ctx_d.stride(0)
    pad = 5
    wp = torch.full((nworld, 3 * layer.waypoint_count + pad), 7.0, device="cuda")
    unit = torch.full((nworld, layer.muscle_count + pad), 7.0, device="cuda")
    pas = torch.full((nworld, layer.muscle_count + pad), 7.0, device="cuda")
    wp_args = (base + 4 * layer._xpos_off, ld, base + 4 * layer._xquat_off, ld, d["wp_body"].data_ptr(),
               d["wp_local"].data_ptr(), layer.waypoint_count, wp.data_ptr(), wp.stride(0))  # fmt: skip
    frc_args = (d["all_seg_start"].data_ptr(), d["all_seg_off"].data_ptr(), d["params"].data_ptr(),
                layer.muscle_params.shape[1], d["rest"].data_ptr(), C.byref(layer._model), layer.muscle_count,
                unit.data_ptr(), unit.stride(0), pas.data_ptr(), pas.stride(0), nworld, None)  # fmt: skip
    _lib.check(L.im_muscle_waypoints(*wp_args, nworld, None), "im_muscle_waypoints")
    _lib.check(L.im_muscle_force_magnitudes(wp.data_ptr(), wp.stride(0), *frc_args), "im_muscle_force_magnitudes")
    torch.cuda.synchronize()
    assert torch.equal(wp[:, :-pad], ws["transformed_waypoints"])
    assert torch.equal(unit[:, :-pad], ws["unit_force_magnitude"])
    assert torch.equal(pas[:, :-pad], ws["passive_force_magnitude"])
    assert (wp[:, -pad:] == 7.0).all() and (unit[:, -pad:] == 7.0).all() and (pas[:, -pad:] == 7.0).all()
    # the fused call with padded rows as well
    wp2, unit2, pas2 = torch.full_like(wp, 3.0), torch.full_like(unit, 3.0), torch.full_like(pas, 3.0)
    args2 = wp_args[:7] + (wp2.data_ptr(), wp2.stride(0)) + frc_args[:7] + (
        unit2.data_ptr(), unit2.stride(0), pas2.data_ptr(), pas2.stride(0), nworld, None)  # fmt: skip
    _lib.check(L.im_muscle_waypoints_forces(*args2), "im_muscle_waypoints_forces")
    torch.cuda.synchronize()
    assert torch.equal(wp2[:, :-pad], wp[:, :-pad]) and torch.equal(unit2[:, :-pad], unit[:, :-pad])
    assert torch.equal(pas2[:, :-pad], pas[:, :-pad])
    assert (wp2[:, -pad:] == 3.0).all() and (unit2[:, -pad:] == 3.0).all() and (pas2[:, -pad:] == 3.0).all()


@pytest.mark.gpu
def test_gpu_entry_lists_without_a_stated_range_take_the_other_kernels():
    """An entry list whose nother field is 0 sends the contractions to the one-thread-per-output
    kernels; results are the same bits as with the range stated."""
    rig = synth.make_muscle_rig(nmuscle=284, seed=1003)
    layer = _gpu_layer(rig, active_force_type="gaussian", passive_force_type="exponential")
    nworld = 77
    ctx_d = torch.from_numpy(synth.make_muscle_context(rig, nworld, seed=5)).cuda()
    act = torch.rand(nworld, rig.muscle_count, device="cuda")
    g = torch.randn(nworld, rig.torque_dim, device="cuda")

    def run():
        mean, _, unit = layer._warp_muscle_dynamics_from_activation_forward(act, ctx_d, include_passive_force=True)
        grad = layer._warp_muscle_dynamics_from_activation_backward(ctx_d, g)
        moment = layer.eval_muscle_sparse_moment(ctx_d)
        torch.cuda.synchronize()
        return mean.clone(), grad.clone(), moment.clone()

    stated = run()
    for e in (layer._torque_entries, layer._muscle_entries, layer._moment_entries):
        assert e.nother > 0
        e.nother = 0
    for a, b in zip(stated, run()):
        assert torch.equal(a, b)
