"""Sparse muscle moment contractions on MI355X: ``tau = A' f`` and the implicit term
``h * A' diag(s) A`` gathered into M's structure.

Drop-in for the parts of the reference module
``instantmimic.muscle.muscle_qfrc_projector`` that sit on the solver's hot path
(src/instantmimic/muscle/muscle_qfrc_projector.py): metadata builders :535-669 and
:812-972, launchers :777-809 and the projection kernel :2941-2961.  Index tables are
built on the host with NumPy and kept as int32 torch tensors on the GPU; the arithmetic
runs in ``libimhip``'s HIP kernels.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import numpy as np

from .. import _lib

_QDERIV_GATHER_CHUNK = 16
_QDERIV_GATHER_BLOCK_DIM = 256
_QDERIV_GATHER_MAX_SHARED_BYTES = 48 * 1024
_QDERIV_GATHER_MAX_ENTRIES = 0x7FFF


def _np(a, dtype=np.int64) -> np.ndarray:
    if hasattr(a, "detach"):
        a = a.detach().cpu().numpy()
    return np.asarray(a, dtype=dtype)


@dataclass(frozen=True)
class MuscleDofSparseEntries:
    """(muscle, torque dof) entries sorted by muscle then dof, their segments, and the
    lower-triangle entry pairs of every muscle (reference fields, NumPy arrays)."""

    muscle_dof_offsets: np.ndarray
    muscle_dof_muscle_idx: np.ndarray
    muscle_dof_torque_idx: np.ndarray
    muscle_dof_segment_offsets: np.ndarray
    segment_idx: np.ndarray
    start_coeff: np.ndarray
    end_coeff: np.ndarray
    pair_entry_i: np.ndarray
    pair_entry_j: np.ndarray
    pair_muscle_idx: np.ndarray


def _pairs(muscle_dof_offsets: np.ndarray):
    pi, pj, pm = [], [], []
    for muscle in range(len(muscle_dof_offsets) - 1):
        b, e = int(muscle_dof_offsets[muscle]), int(muscle_dof_offsets[muscle + 1])
        n = e - b
        if n <= 0:
            continue
        ii, jj = np.tril_indices(n)
        pi.append(b + ii)
        pj.append(b + jj)
        pm.append(np.full(ii.size, muscle))
    if not pi:
        z = np.zeros(0, np.int32)
        return z, z.copy(), z.copy()
    return (np.concatenate(a).astype(np.int32) for a in (pi, pj, pm))


def build_muscle_dof_sparse_entries(
    torque_active_entry_offsets, torque_active_segment_idx, torque_active_muscle_idx, torque_active_start_coeff,
    torque_active_end_coeff, muscle_count: int,
) -> MuscleDofSparseEntries:  # fmt: skip
    """Group active segments by (muscle, dof) and list each muscle's entry pairs i >= j."""
    offsets = _np(torque_active_entry_offsets)
    seg = _np(torque_active_segment_idx)
    mus = _np(torque_active_muscle_idx)
    c0 = _np(torque_active_start_coeff, np.float32)
    c1 = _np(torque_active_end_coeff, np.float32)
    torque_dim = max(offsets.size - 1, 0)
    if torque_dim == 0 or seg.size == 0:
        z = np.zeros(0, np.int32)
        return MuscleDofSparseEntries(
            np.zeros(muscle_count + 1, np.int32), z, z.copy(), np.zeros(1, np.int32), z.copy(),
            np.zeros(0, np.float32), np.zeros(0, np.float32), z.copy(), z.copy(), z.copy(),
        )  # fmt: skip
    torque = np.repeat(np.arange(torque_dim), np.diff(offsets))
    order = np.lexsort((seg, torque, mus))  # by muscle, then dof, then segment
    mus, torque, seg, c0, c1 = mus[order], torque[order], seg[order], c0[order], c1[order]
    new = np.ones(seg.size, bool)
    new[1:] = (mus[1:] != mus[:-1]) | (torque[1:] != torque[:-1])
    start = np.flatnonzero(new)
    group_muscle, group_torque = mus[start], torque[start]
    muscle_dof_offsets = np.zeros(muscle_count + 1, np.int32)
    muscle_dof_offsets[1:] = np.cumsum(np.bincount(group_muscle, minlength=muscle_count))
    pi, pj, pm = _pairs(muscle_dof_offsets)
    return MuscleDofSparseEntries(
        muscle_dof_offsets, group_muscle.astype(np.int32), group_torque.astype(np.int32),
        np.concatenate((start, [seg.size])).astype(np.int32), seg.astype(np.int32), c0, c1, pi, pj, pm,
    )  # fmt: skip


def entries_from_muscle_dofs(muscle_dofs, muscle_count: int) -> MuscleDofSparseEntries:
    """Entries for a plain list of (muscle, torque dof) couplings, one segment each."""
    md = np.unique(np.asarray(muscle_dofs, np.int64).reshape(-1, 2), axis=0)
    torque_dim = int(md[:, 1].max()) + 1 if md.size else 0
    order = np.argsort(md[:, 1], kind="stable")
    offsets = np.zeros(torque_dim + 1, np.int64)
    offsets[1:] = np.cumsum(np.bincount(md[:, 1], minlength=torque_dim))
    n = md.shape[0]
    return build_muscle_dof_sparse_entries(
        offsets, np.arange(n), md[order, 0], np.ones(n, np.float32), np.zeros(n, np.float32), muscle_count
    )


def torque_sorted_entries(muscle_dof_torque_idx, torque_dim: int):
    """Entry order per torque dof, ascending entry index
    (src/instantmimic/envs/controls/fast_muscle/torque_runtime.py:617-629)."""
    t = _np(muscle_dof_torque_idx)
    order = np.argsort(t, kind="stable").astype(np.int32)
    offsets = np.zeros(torque_dim + 1, np.int32)
    offsets[1:] = np.cumsum(np.bincount(t, minlength=torque_dim))
    return offsets, order


@dataclass(frozen=True)
class PreparedMuscleImplicitQderivPairs:
    pair_elem_id: np.ndarray
    pair_entry_i: np.ndarray
    pair_entry_j: np.ndarray
    pair_muscle_idx: np.ndarray
    dropped_pair_count: int


def prepare_muscle_implicit_qderiv_pairs(
    *, pair_entry_i, pair_entry_j, pair_muscle_idx, muscle_dof_torque_idx, matrix_elemid, root_dof_count: int
) -> PreparedMuscleImplicitQderivPairs:
    """The packed M element of every damping pair; pairs without one are dropped."""
    pi, pj, pm = _np(pair_entry_i), _np(pair_entry_j), _np(pair_muscle_idx)
    dof, elemid = _np(muscle_dof_torque_idx), _np(matrix_elemid)
    if pi.shape != pj.shape or pi.shape != pm.shape:
        raise ValueError("Implicit muscle pair arrays must have matching shapes")
    if pi.size == 0:
        z = np.zeros(0, np.int32)
        return PreparedMuscleImplicitQderivPairs(z, z.copy(), z.copy(), z.copy(), 0)
    mapped = elemid[dof[pi] + int(root_dof_count), dof[pj] + int(root_dof_count)]
    valid = mapped >= 0
    return PreparedMuscleImplicitQderivPairs(
        mapped[valid].astype(np.int32), pi[valid].astype(np.int32), pj[valid].astype(np.int32),
        pm[valid].astype(np.int32), int((~valid).sum()),
    )  # fmt: skip


@dataclass(frozen=True)
class MuscleImplicitQderivGather:
    """Gather tables on the device: pairs grouped by M element, cut into chunks of 16,
    packed ``i | j << 16`` chunk-interleaved (pair k of chunk c at ``k * chunk_count + c``),
    padded with the entry count."""

    kernel: Any
    cuda: bool
    entry_muscle: Any
    elem_ids: Any
    chunk_offsets: Any
    chunk_pairs: Any
    entry_count: int
    chunk_count: int


def gather_tables(prepared: PreparedMuscleImplicitQderivPairs, entry_muscle_idx):
    """Host tables of the deterministic gather: (elem_ids, chunk_offsets, chunk_pairs, entry_count,
    chunk_count) from ``im_muscle_gather_tables``; ``None`` when there is nothing to gather or the
    index limit is hit."""
    import ctypes as C

    elem = np.ascontiguousarray(_np(prepared.pair_elem_id), np.int32)
    entry_muscle = _np(entry_muscle_idx)
    entry_count = int(entry_muscle.size)
    if elem.size == 0 or entry_count >= _QDERIV_GATHER_MAX_ENTRIES:
        return None
    pi, pj, pm = (np.ascontiguousarray(_np(a), np.int32) for a in (prepared.pair_entry_i, prepared.pair_entry_j, prepared.pair_muscle_idx))
    if not (np.array_equal(entry_muscle[pi], pm) and np.array_equal(entry_muscle[pj], pm)):
        raise ValueError("every implicit qDeriv pair must join entries of its muscle")
    nelem, nchunk = C.c_int(0), C.c_int(0)
    lib = _lib.lib()
    _lib.check(lib.im_muscle_gather_tables(elem.ctypes.data, None, None, int(elem.size), entry_count, None, None, None, C.byref(nelem), C.byref(nchunk)), "im_muscle_gather_tables")
    elem_ids, chunk_offsets = np.zeros(nelem.value, np.int32), np.zeros(nelem.value + 1, np.int32)
    chunk_pairs = np.zeros(_QDERIV_GATHER_CHUNK * nchunk.value, np.int32)
    _lib.check(
        lib.im_muscle_gather_tables(elem.ctypes.data, pi.ctypes.data, pj.ctypes.data, int(elem.size), entry_count, elem_ids.ctypes.data,
                                    chunk_offsets.ctypes.data, chunk_pairs.ctypes.data, C.byref(nelem), C.byref(nchunk)),
        "im_muscle_gather_tables",
    )  # fmt: skip
    return elem_ids, chunk_offsets, chunk_pairs, entry_count, int(nchunk.value)


def build_muscle_implicit_qderiv_gather(prepared, entry_muscle_idx, device) -> MuscleImplicitQderivGather | None:
    """The gather tables on ``device``, or ``None`` when they exceed the index or LDS limits."""
    import torch

    tables = gather_tables(prepared, entry_muscle_idx)
    if tables is None:
        return None
    elem_ids, chunk_offsets, chunk_pairs, entry_count, chunk_count = tables
    if 4 * (2 * (entry_count + 1) + chunk_count) > _QDERIV_GATHER_MAX_SHARED_BYTES:
        return None
    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError("the HIP gather runs on the GPU only (no CPU fallback)")

    def i32(a):
        return torch.from_numpy(np.ascontiguousarray(a, np.int32)).to(dev)

    return MuscleImplicitQderivGather(
        kernel="im_muscle_implicit_gather", cuda=True, entry_muscle=i32(_np(entry_muscle_idx)), elem_ids=i32(elem_ids),
        chunk_offsets=i32(chunk_offsets), chunk_pairs=i32(chunk_pairs), entry_count=entry_count,
        chunk_count=chunk_count,
    )  # fmt: skip


def _stream(t) -> int:
    import torch

    return int(torch.cuda.current_stream(t.device).cuda_stream)


def _f32_rows(*tensors):
    import torch

    for t in tensors:
        if t.dtype != torch.float32 or not t.is_cuda or t.dim() != 2 or t.stride(1) != 1:
            raise TypeError("expected 2-D float32 CUDA tensors with contiguous rows")


def apply_muscle_implicit_qderiv_gather(gather: MuscleImplicitQderivGather, moment, force_velocity_slope, timestep: float, qderiv) -> None:
    """Add ``timestep * sum_m slope_m r_m r_m'`` to qDeriv in M structure."""
    import torch

    _f32_rows(moment, force_velocity_slope, qderiv)
    with torch.cuda.device(moment.device):
        status = _lib.lib().im_muscle_implicit_gather(
            moment.data_ptr(), moment.stride(0), force_velocity_slope.data_ptr(), force_velocity_slope.stride(0),
            gather.entry_muscle.data_ptr(), gather.entry_count, gather.elem_ids.data_ptr(), int(gather.elem_ids.numel()),
            gather.chunk_offsets.data_ptr(), gather.chunk_pairs.data_ptr(), gather.chunk_count, float(timestep),
            qderiv.data_ptr(), qderiv.stride(0), int(moment.shape[0]), _stream(moment),
        )  # fmt: skip
    _lib.check(status, "im_muscle_implicit_gather")


def project_muscle_sparse_moment_qfrc(
    moment, muscle_force_magnitude, torque_entry_offsets, torque_entry_idx, muscle_dof_muscle_idx, root_dof_count: int,
    qfrc_applied,
) -> None:  # fmt: skip
    """``qfrc_applied[w, root + j] = sum_e moment[w, e] * force[w, muscle(e)]`` over the
    entries of torque dof j in torque-sorted order (arguments of the reference kernel)."""
    import torch

    _f32_rows(moment, muscle_force_magnitude, qfrc_applied)
    for t in (torque_entry_offsets, torque_entry_idx, muscle_dof_muscle_idx):
        if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
            raise TypeError("index tables must be contiguous int32 CUDA tensors")
    ntorque = int(torque_entry_offsets.numel()) - 1
    with torch.cuda.device(moment.device):
        status = _lib.lib().im_muscle_project(
            moment.data_ptr(), moment.stride(0), muscle_force_magnitude.data_ptr(), muscle_force_magnitude.stride(0),
            torque_entry_offsets.data_ptr(), torque_entry_idx.data_ptr(), muscle_dof_muscle_idx.data_ptr(),
            int(muscle_dof_muscle_idx.numel()), int(muscle_force_magnitude.shape[1]), ntorque, int(root_dof_count),
            qfrc_applied.data_ptr(), qfrc_applied.stride(0), int(moment.shape[0]), _stream(moment),
        )  # fmt: skip
    _lib.check(status, "im_muscle_project")


def eval_muscle_force_velocity_state(
    transformed_waypoints, muscle_waypoint_start, muscle_params, muscle_rest_length, force_velocity_length_scale,
    activation, qvel, moment, muscle_dof_offsets, muscle_dof_torque_idx, root_dof_count: int, *,
    muscle_force_scale: float, muscle_length_norm_min: float, muscle_length_norm_max: float, vmax: float,
    fvmax: float, clamp_activation: bool, include_active: bool, active_force_model_params,
    muscle_length, effective_activation, length_velocity, force_velocity_multiplier, force_velocity_slope,
) -> None:  # fmt: skip
    """Launch of ``eval_muscle_force_velocity_state_kernel`` with the reference's arrays
    (src/instantmimic/muscle/muscle_qfrc_projector.py:2816-2884): waypoints (nworld, nwaypoint, 3),
    activation and the five outputs (nworld, nmuscle), qvel (nworld, nv), moment (nworld, nentry);
    the index tables int32 tensors on the same GPU.  ``force_velocity_slope`` is what
    :func:`apply_muscle_implicit_qderiv_gather` takes."""
    import torch

    nworld, nmuscle = int(activation.shape[0]), int(activation.shape[1])
    outs = (muscle_length, effective_activation, length_velocity, force_velocity_multiplier, force_velocity_slope)
    wp2 = transformed_waypoints.reshape(nworld, -1)
    _f32_rows(wp2, activation, qvel, moment, muscle_params, *outs)
    for t in outs:
        if tuple(t.shape) != (nworld, nmuscle) or t.stride(0) != outs[0].stride(0):
            raise ValueError("the five outputs must be (nworld, nmuscle) with one row stride")
    for t in (muscle_waypoint_start, muscle_dof_offsets, muscle_dof_torque_idx):
        if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
            raise TypeError("index tables must be contiguous int32 CUDA tensors")
    if muscle_waypoint_start.numel() != nmuscle + 1 or muscle_dof_offsets.numel() != nmuscle + 1:
        raise ValueError("muscle_waypoint_start and muscle_dof_offsets need nmuscle + 1 entries")
    if qvel.shape[0] != nworld or moment.shape[0] != nworld or moment.shape[1] < muscle_dof_torque_idx.numel():
        raise ValueError("qvel and moment do not match the batch or the entry table")
    if muscle_rest_length.numel() != nmuscle or force_velocity_length_scale.numel() != nmuscle or muscle_params.shape[0] != nmuscle:
        raise ValueError("per-muscle arrays need nmuscle rows")
    model = _lib.MuscleForceModel()
    model.force_scale, model.length_norm_min, model.length_norm_max = muscle_force_scale, muscle_length_norm_min, muscle_length_norm_max
    for k, v in enumerate(active_force_model_params):
        model.active[k] = float(v)
    fv = _lib.MuscleForceVelocityModel(float(vmax), float(fvmax), float(bool(clamp_activation)), float(bool(include_active)))
    import ctypes as C

    with torch.cuda.device(activation.device):
        status = _lib.lib().im_muscle_force_velocity_state(
            wp2.data_ptr(), wp2.stride(0), muscle_waypoint_start.data_ptr(), muscle_params.data_ptr(),
            muscle_params.stride(0), muscle_rest_length.data_ptr(), force_velocity_length_scale.data_ptr(),
            activation.data_ptr(), activation.stride(0), qvel.data_ptr(), qvel.stride(0), moment.data_ptr(),
            moment.stride(0), muscle_dof_offsets.data_ptr(), muscle_dof_torque_idx.data_ptr(), int(root_dof_count),
            C.byref(model), C.byref(fv), nmuscle, *[t.data_ptr() for t in outs], outs[0].stride(0), nworld,
            _stream(activation),
        )  # fmt: skip
    _lib.check(status, "im_muscle_force_velocity_state")
