"""Waypoint muscle layer on MI355X: pose context -> path geometry -> activation-to-torque
projection and its activation gradient.

Drop-in for the waypoint projection of the reference's ``MuscleDynamicsLayer``
(src/instantmimic/muscle/muscle_dynamics.py): static sparsity built as in
``muscle_qfrc_projector.py:336-510`` and ``muscle_dynamics.py:1318-1392``, raw context
layout of ``muscle_dynamics.py:4824-4838``, launch sequence of
``_warp_muscle_dynamics_from_activation_forward`` (:4958-5009 and the waypoint tail) and
``_warp_muscle_dynamics_from_activation_backward``.  Linear-blend-skinned attachments, the
force-velocity factor and the native body-wrench tiles of the reference are other paths of
that class and are not provided here; asking for them raises.

The arithmetic runs in ``libimhip``; tensors must live on the GPU.  Index tables are built
once on the host with NumPy.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field

import numpy as np

from .. import _lib
from .muscle_qfrc_projector import MuscleDofSparseEntries, _np, build_muscle_dof_sparse_entries


@dataclass(frozen=True)
class MuscleMechanics:
    """The fields of the reference's MuscleMechanicsRuntimeSpec that the waypoint path reads
    (src/instantmimic/muscle/runtime_specs.py:66-96)."""

    force_scale: float = 1.0
    active_force_type: str = "gaussian"
    active_force_gamma: float = 0.45
    active_force_lmin: float = 0.5
    active_force_lmax: float = 1.6
    passive_force_type: str = "exponential"
    passive_force_k_pe: float = 5.5
    passive_force_e_mo: float = 0.3
    passive_force_lmax: float = 1.6
    passive_force_fpmax: float = 1.3
    length_norm_min: float = 0.2
    length_norm_max: float = 1.8
    include_passive_force_in_output: bool = False
    force_velocity_enabled: bool = False

    def __post_init__(self):
        # the reference's checks, muscle_dynamics.py:523-573
        if self.active_force_type not in {"gaussian", "mujoco"}:
            raise ValueError("muscle_active_force_type must be 'gaussian' or 'mujoco'")
        if self.active_force_gamma <= 0.0:
            raise ValueError("Gaussian active-force gamma must be positive")
        if not (0.0 < self.active_force_lmin < 1.0 and self.active_force_lmax > 1.0):
            raise ValueError("MuJoCo active-force lmin/lmax must satisfy 0 < lmin < 1 < lmax")
        if self.passive_force_type not in {"exponential", "mujoco"}:
            raise ValueError("muscle_passive_force_type must be 'exponential' or 'mujoco'")
        if self.passive_force_k_pe <= 0.0 or self.passive_force_e_mo <= 0.0:
            raise ValueError("exponential passive-force k_pe and e_mo must be positive")
        if self.passive_force_lmax <= 1.0 or self.passive_force_fpmax < 0.0:
            raise ValueError("MuJoCo passive-force lmax must exceed 1 and fpmax must be nonnegative")
        if self.force_velocity_enabled:
            raise NotImplementedError("the force-velocity factor is not part of this library")

    def active_params(self) -> tuple[float, float, float]:
        if self.active_force_type == "gaussian":
            return (0.0, self.active_force_gamma, 0.0)
        return (1.0, self.active_force_lmin, self.active_force_lmax)

    def passive_params(self) -> tuple[float, float, float]:
        if self.passive_force_type == "exponential":
            return (0.0, self.passive_force_k_pe, self.passive_force_e_mo)
        return (1.0, self.passive_force_lmax, self.passive_force_fpmax)


@dataclass(frozen=True)
class MuscleTopology:
    """The waypoint fields of the reference's MuscleTopologySpec (runtime_specs.py), as
    NumPy-convertible arrays."""

    muscle_params: np.ndarray  # (M, >= 4): f0, l_m0, l_t0, pennation
    muscle_rest_length: np.ndarray  # (M,)
    muscle_waypoints_local: np.ndarray  # (W, 3)
    muscle_waypoint_body: np.ndarray  # (W,)
    all_segment_muscle_idx: np.ndarray  # (S_all,) nondecreasing
    all_segment_start_idx: np.ndarray  # (S_all,) waypoint id; the end is start + 1
    apply_segment_muscle_idx: np.ndarray  # (S,)
    apply_segment_start_idx: np.ndarray
    apply_segment_end_idx: np.ndarray
    apply_segment_body_start_idx: np.ndarray
    apply_segment_body_end_idx: np.ndarray
    body_parentid: np.ndarray  # (nbody,)
    body_rootid: np.ndarray
    dof_bodyid: np.ndarray  # (>= full_torque_dim,)
    uses_lbs_waypoint_attachments: bool = False


def build_dof_subtree_mask(body_parentid, dof_bodyid, body_count: int, full_torque_dim: int) -> np.ndarray:
    """mask[dof, body] = 1 when the dof's body is the body or one of its ancestors below
    the world; world-body dofs move everything (muscle_qfrc_projector.py:336-356)."""
    parent = _np(body_parentid)
    ancestor = np.zeros((body_count, body_count), bool)
    for b in range(body_count):
        p = b
        while p != 0:
            ancestor[b, p] = True
            p = int(parent[p])
    dof_body = _np(dof_bodyid)[:full_torque_dim]
    mask = ancestor[:, dof_body].T.astype(np.float32)
    mask[dof_body == 0] = 1.0
    return mask


def build_muscle_segment_offsets(segment_muscle_idx, muscle_count: int) -> np.ndarray:
    """muscle_qfrc_projector.py:321-333"""
    counts = np.bincount(_np(segment_muscle_idx), minlength=muscle_count)
    return np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)


def build_torque_sparse_segment_entries(segment_start_dof_mask, segment_end_dof_mask, apply_segment_muscle_idx):
    """Per torque dof, the segments whose start or end coefficient is nonzero, ascending
    (muscle_qfrc_projector.py:378-456).  Returns offsets, torque, segment, muscle, start and
    end coefficient."""
    start = np.asarray(segment_start_dof_mask, np.float32)
    end = np.asarray(segment_end_dof_mask, np.float32)
    muscle = _np(apply_segment_muscle_idx)
    torque_idx, segment_idx = np.nonzero((start != 0) | (end != 0))  # row-major: torque, then segment
    offsets = np.concatenate([[0], np.cumsum(np.bincount(torque_idx, minlength=start.shape[0]))])
    return (
        offsets.astype(np.int32),
        torque_idx.astype(np.int32),
        segment_idx.astype(np.int32),
        muscle[segment_idx].astype(np.int32),
        start[torque_idx, segment_idx],
        end[torque_idx, segment_idx],
    )


def build_muscle_sparse_torque_entries(
    torque_entry_offsets, torque_segment_idx, torque_start_coeff, torque_end_coeff, apply_segment_muscle_idx,
    muscle_count: int,
):  # fmt: skip
    """The same entries sorted by (muscle, segment, torque) (muscle_qfrc_projector.py:459-510).
    Returns offsets, segment, torque, start and end coefficient."""
    offsets = _np(torque_entry_offsets)
    segment = _np(torque_segment_idx)
    if len(offsets) <= 1 or len(segment) == 0:
        z = np.zeros(0, np.int32)
        return np.zeros(muscle_count + 1, np.int32), z, z.copy(), np.zeros(0, np.float32), np.zeros(0, np.float32)
    torque = np.repeat(np.arange(len(offsets) - 1), np.diff(offsets))
    muscle = _np(apply_segment_muscle_idx)[segment]
    order = np.lexsort((torque, segment, muscle))
    return (
        build_muscle_segment_offsets(muscle, muscle_count),
        segment[order].astype(np.int32),
        torque[order].astype(np.int32),
        np.asarray(torque_start_coeff, np.float32)[order],
        np.asarray(torque_end_coeff, np.float32)[order],
    )


@dataclass
class _Tables:
    keep: list = field(default_factory=list)


def _stream(t) -> int:
    import torch

    return torch.cuda.current_stream(t.device).cuda_stream


class MuscleDynamicsLayer:
    """Static tables of one musculoskeletal model on one GPU and the launchers that use them."""

    def __init__(
        self,
        topology: MuscleTopology,
        *,
        body_count: int,
        full_torque_dim: int,
        torque_dim: int,
        muscle_count: int,
        mechanics: MuscleMechanics | None = None,
        active_torque_indices=None,
        device="cuda",
    ):
        import torch

        if topology.uses_lbs_waypoint_attachments:
            raise NotImplementedError("linear-blend-skinned waypoint attachments are not part of this library")
        if body_count <= 0 or muscle_count <= 0 or torque_dim <= 0:
            raise ValueError("muscle body, muscle, and torque dimensions must be positive")
        if full_torque_dim < torque_dim:
            raise ValueError("full_torque_dim must be at least torque_dim")
        self.mechanics = mechanics or MuscleMechanics()
        self.body_count, self.muscle_count = int(body_count), int(muscle_count)
        self.torque_dim, self.full_torque_dim = int(torque_dim), int(full_torque_dim)
        self.root_dof_count = self.full_torque_dim - self.torque_dim
        self.include_passive_force_in_output = self.mechanics.include_passive_force_in_output
        self.muscle_force_velocity_enabled = False
        self.device = torch.device(device)
        # MuscleOutputSpec.active_torque_indices of the reference (runtime_specs.py:53-63)
        self.active_torque_indices = None if active_torque_indices is None else _np(active_torque_indices)
        self.active_output_dim = self.torque_dim if self.active_torque_indices is None else len(self.active_torque_indices)
        # raw context = xpos | xquat | xipos | subtree_com | cdof (muscle_dynamics.py:4824-4838)
        nb, nvf = self.body_count, self.full_torque_dim
        self._xpos_off, self._xquat_off = 0, 3 * nb
        self._xipos_off, self._com_off, self._cdof_off = 7 * nb, 10 * nb, 13 * nb
        self.context_dim = 13 * nb + 6 * nvf

        t = topology
        self.waypoint_count = len(_np(t.muscle_waypoint_body))
        mask = build_dof_subtree_mask(t.body_parentid, t.dof_bodyid, nb, nvf)
        self.dof_subtree_mask = mask
        body0, body1 = _np(t.apply_segment_body_start_idx), _np(t.apply_segment_body_end_idx)
        self.segment_start_dof_mask = mask[self.root_dof_count :, body0]
        self.segment_end_dof_mask = mask[self.root_dof_count :, body1]
        rootid = _np(t.body_rootid)
        self.apply_segment_muscle_idx = _np(t.apply_segment_muscle_idx, np.int32)
        tq = build_torque_sparse_segment_entries(
            self.segment_start_dof_mask, self.segment_end_dof_mask, t.apply_segment_muscle_idx
        )
        ms = build_muscle_sparse_torque_entries(tq[0], tq[2], tq[4], tq[5], t.apply_segment_muscle_idx, self.muscle_count)
        self.torque_entries_host = tq
        self.muscle_entries_host = ms
        self.sparse_entries: MuscleDofSparseEntries = build_muscle_dof_sparse_entries(
            tq[0], tq[2], tq[3], tq[4], tq[5], self.muscle_count
        )
        self.segments_host = (
            _np(t.apply_segment_start_idx, np.int32), _np(t.apply_segment_end_idx, np.int32),
            rootid[body0].astype(np.int32), rootid[body1].astype(np.int32),
        )  # fmt: skip
        self.all_segment_start_idx = _np(t.all_segment_start_idx, np.int32)
        self.all_muscle_segment_offsets = build_muscle_segment_offsets(t.all_segment_muscle_idx, self.muscle_count)
        self.muscle_params = np.ascontiguousarray(np.asarray(t.muscle_params, np.float32))
        self.muscle_rest_length = np.ascontiguousarray(np.asarray(t.muscle_rest_length, np.float32))
        self.waypoints_local = np.ascontiguousarray(np.asarray(t.muscle_waypoints_local, np.float32))
        self.waypoint_body = _np(t.muscle_waypoint_body, np.int32)
        last = self.all_segment_start_idx.max(initial=-1) + 1
        if max(last, self.segments_host[0].max(initial=-1), self.segments_host[1].max(initial=-1)) >= self.waypoint_count:
            raise ValueError("a segment names a waypoint beyond the waypoint list")
        if self.waypoint_body.max(initial=-1) >= nb or max(self.segments_host[2].max(initial=-1), self.segments_host[3].max(initial=-1)) >= nb:
            raise ValueError("a waypoint or segment names a body beyond body_count")

        m = self.mechanics
        self._model = _lib.MuscleForceModel(
            m.force_scale, m.length_norm_min, m.length_norm_max, (C.c_float * 3)(*m.active_params()),
            (C.c_float * 3)(*m.passive_params()), 1,
        )  # fmt: skip
        self._dev = {}
        if self.device.type == "cuda":
            self._upload()

    # ------------------------------------------------------------------ device tables
    def _upload(self):
        import torch

        def up(a):
            return torch.from_numpy(np.ascontiguousarray(a)).to(self.device)

        d = self._dev
        d["seg"] = [up(a) for a in self.segments_host]
        d["tq"] = [up(a) for a in (self.torque_entries_host[i] for i in (0, 2, 3, 4, 5))]
        d["ms"] = [up(a) for a in self.muscle_entries_host]
        e = self.sparse_entries
        d["mom"] = [up(a.astype(np.int32)) for a in (e.muscle_dof_segment_offsets, e.segment_idx)] + [
            up(np.asarray(e.start_coeff, np.float32)),
            up(np.asarray(e.end_coeff, np.float32)),
        ]
        d["mom_torque"] = up(e.muscle_dof_torque_idx.astype(np.int32))
        d["all_seg_start"] = up(self.all_segment_start_idx)
        d["all_seg_off"] = up(self.all_muscle_segment_offsets)
        d["params"], d["rest"] = up(self.muscle_params), up(self.muscle_rest_length)
        d["wp_local"], d["wp_body"] = up(self.waypoints_local), up(self.waypoint_body)
        p = [t.data_ptr() for t in d["seg"]]
        self._segments = _lib.MuscleSegments(*p, len(self.segments_host[0]))

        def entries(ts, nrow, nother, other=True):
            off, seg = ts[0], ts[1]
            rest = ts[2:]
            o = rest[0].data_ptr() if other else None
            a, b = (rest[1], rest[2]) if other else (rest[0], rest[1])
            return _lib.MuscleEntries(off.data_ptr(), seg.data_ptr(), o, a.data_ptr(), b.data_ptr(), nrow, seg.numel(), nother)

        self._torque_entries = entries(d["tq"], self.torque_dim, self.muscle_count)
        self._muscle_entries = entries(d["ms"], self.muscle_count, self.torque_dim)
        self._moment_entries = entries(d["mom"], len(e.muscle_dof_torque_idx), self.torque_dim, other=False)

    def _need_gpu(self, *tensors):
        import torch

        if not self._dev:
            raise RuntimeError("this layer was built without a GPU; its kernels exist only in libimhip (no CPU path)")
        for t in tensors:
            if t is None:
                continue
            if not t.is_cuda or t.dtype != torch.float32:
                raise ValueError("muscle tensors must be float32 tensors on the GPU")
            if t.dim() != 2 or (t.numel() and t.shape[1] > 1 and t.stride(1) != 1):
                raise ValueError("muscle tensors must be 2-D with contiguous rows")

    # ------------------------------------------------------------------ geometry
    def _prepare_waypoint_geometry(self, raw_context, *, include_passive_force_magnitude: bool, compute_force_magnitudes: bool = True):
        """Waypoints in the world frame and the per-muscle force magnitudes of a batch of
        contexts (reference _prepare_warp_waypoint_geometry).  Returns a workspace dict and
        the geometry descriptor that the contraction launchers take."""
        import torch

        self._need_gpu(raw_context)
        if raw_context.shape[1] < self.context_dim:
            raise ValueError(f"raw_context has {raw_context.shape[1]} columns, the layer needs {self.context_dim}")
        B, ld = raw_context.shape[0], raw_context.stride(0)
        base, d, s = raw_context.data_ptr(), self._dev, _stream(raw_context)
        ws = {"transformed_waypoints": torch.empty((B, 3 * self.waypoint_count), device=raw_context.device)}
        wp = ws["transformed_waypoints"]
        L = _lib.lib()
        wp_args = (
            base + 4 * self._xpos_off, ld, base + 4 * self._xquat_off, ld, d["wp_body"].data_ptr(),
            d["wp_local"].data_ptr(), self.waypoint_count, wp.data_ptr(), wp.stride(0),
        )  # fmt: skip
        if compute_force_magnitudes:
            # both steps in one launch: a world's waypoints stay on chip between them
            ws["unit_force_magnitude"] = torch.empty((B, self.muscle_count), device=raw_context.device)
            ws["passive_force_magnitude"] = torch.empty((B, self.muscle_count), device=raw_context.device)
            self._model.include_passive = 1 if include_passive_force_magnitude else 0
            u, p = ws["unit_force_magnitude"], ws["passive_force_magnitude"]
            _lib.check(
                L.im_muscle_waypoints_forces(
                    *wp_args, d["all_seg_start"].data_ptr(), d["all_seg_off"].data_ptr(), d["params"].data_ptr(),
                    self.muscle_params.shape[1], d["rest"].data_ptr(), C.byref(self._model), self.muscle_count,
                    u.data_ptr(), u.stride(0), p.data_ptr(), p.stride(0), B, s,
                ),
                "im_muscle_waypoints_forces",
            )  # fmt: skip
        else:
            _lib.check(L.im_muscle_waypoints(*wp_args, B, s), "im_muscle_waypoints")
        geo = _lib.MuscleGeometry(
            wp.data_ptr(), wp.stride(0), base + 4 * self._com_off, ld, base + 4 * self._cdof_off, ld
        )
        return ws, geo

    # ------------------------------------------------------------------ launchers
    def _warp_muscle_dynamics_from_activation_forward(self, activation, raw_context, *, include_passive_force: bool, mean_out=None):
        """(torque, transformed_waypoints, unit_force_magnitude), as the reference's method of
        this name (muscle_dynamics.py:4958-5009)."""
        import torch

        activation, raw_context = activation.float(), raw_context.float()
        self._need_gpu(activation, raw_context, mean_out)
        if activation.shape != (raw_context.shape[0], self.muscle_count):
            raise ValueError("activation must be (batch, muscle_count)")
        ws, geo = self._prepare_waypoint_geometry(raw_context, include_passive_force_magnitude=include_passive_force)
        B = activation.shape[0]
        mean = mean_out if mean_out is not None else torch.empty((B, self.torque_dim), device=activation.device)
        u, p = ws["unit_force_magnitude"], ws["passive_force_magnitude"]
        _lib.check(
            _lib.lib().im_muscle_torque_forward(
                C.byref(geo), C.byref(self._segments), C.byref(self._torque_entries), u.data_ptr(), u.stride(0),
                p.data_ptr() if include_passive_force else None, p.stride(0), activation.data_ptr(),
                activation.stride(0), self.root_dof_count, mean.data_ptr(), mean.stride(0), B, _stream(activation),
            ),
            "im_muscle_torque_forward",
        )  # fmt: skip
        return mean, ws["transformed_waypoints"], u

    def _warp_muscle_dynamics_from_activation_backward(self, raw_context, grad_output, unit_force_magnitude=None):
        """Activation gradient; geometry is rebuilt from the context unless the unit forces
        are handed in."""
        import torch

        raw_context, grad_output = raw_context.float(), grad_output.float().contiguous()
        self._need_gpu(raw_context, grad_output, unit_force_magnitude)
        if grad_output.shape != (raw_context.shape[0], self.torque_dim):
            raise ValueError("grad_output must be (batch, torque_dim)")
        ws, geo = self._prepare_waypoint_geometry(
            raw_context, include_passive_force_magnitude=False, compute_force_magnitudes=unit_force_magnitude is None
        )
        u = ws["unit_force_magnitude"] if unit_force_magnitude is None else unit_force_magnitude
        B = raw_context.shape[0]
        grad = torch.empty((B, self.muscle_count), device=raw_context.device)
        _lib.check(
            _lib.lib().im_muscle_activation_grad(
                C.byref(geo), C.byref(self._segments), C.byref(self._muscle_entries), u.data_ptr(), u.stride(0),
                grad_output.data_ptr(), grad_output.stride(0), self.root_dof_count, grad.data_ptr(), grad.stride(0), B,
                _stream(raw_context),
            ),
            "im_muscle_activation_grad",
        )  # fmt: skip
        return grad

    def _warp_muscle_dynamics_from_activation_forward_cached_lbs_force(
        self, activation, raw_context, unit_force_magnitude, passive_force_magnitude, *, include_passive_force: bool
    ):
        """Torque from force magnitudes computed outside this call (the reference method of
        this name behind instantmimic_muscle::torque_cached_lbs_forward)."""
        import torch

        activation, raw_context = activation.float(), raw_context.float()
        self._need_gpu(activation, raw_context, unit_force_magnitude, passive_force_magnitude)
        B = activation.shape[0]
        for t in (activation, unit_force_magnitude, passive_force_magnitude):
            if tuple(t.shape) != (B, self.muscle_count):
                raise ValueError("activation and force magnitudes must be (batch, muscle_count)")
        _, geo = self._prepare_waypoint_geometry(raw_context, include_passive_force_magnitude=False, compute_force_magnitudes=False)
        mean = torch.empty((B, self.torque_dim), device=activation.device)
        u, p = unit_force_magnitude, passive_force_magnitude
        _lib.check(
            _lib.lib().im_muscle_torque_forward(
                C.byref(geo), C.byref(self._segments), C.byref(self._torque_entries), u.data_ptr(), u.stride(0),
                p.data_ptr() if include_passive_force else None, p.stride(0), activation.data_ptr(),
                activation.stride(0), self.root_dof_count, mean.data_ptr(), mean.stride(0), B, _stream(activation),
            ),
            "im_muscle_torque_forward",
        )  # fmt: skip
        return mean

    def _compute_activation_torque_bounds_warp(self, raw_context, *, select_active: bool):
        """(lower, upper) of the torque over activations in [0, 1] at the context's geometry
        (reference muscle_dynamics.py:4810-4822); ``select_active`` keeps the layer's
        active torque indices."""
        import torch

        raw_context = raw_context.float()
        self._need_gpu(raw_context)
        ws, geo = self._prepare_waypoint_geometry(raw_context, include_passive_force_magnitude=False)
        B = raw_context.shape[0]
        lower = torch.empty((B, self.torque_dim), device=raw_context.device)
        upper = torch.empty_like(lower)
        u = ws["unit_force_magnitude"]
        _lib.check(
            _lib.lib().im_muscle_torque_bounds(
                C.byref(geo), C.byref(self._segments), C.byref(self._torque_entries), u.data_ptr(), u.stride(0),
                self.root_dof_count, lower.data_ptr(), upper.data_ptr(), lower.stride(0), B, _stream(raw_context),
            ),
            "im_muscle_torque_bounds",
        )  # fmt: skip
        if select_active and self.active_torque_indices is not None:
            idx = torch.from_numpy(self.active_torque_indices.astype(np.int64)).to(raw_context.device)
            return lower.index_select(1, idx), upper.index_select(1, idx)
        return lower, upper

    def eval_muscle_sparse_moment(self, raw_context, moment_out=None):
        """moment (batch, entries) of the (muscle, dof) entries in ``sparse_entries``
        (reference eval_muscle_sparse_moment_kernel, muscle_qfrc_projector.py:2617-2662)."""
        import torch

        raw_context = raw_context.float()
        self._need_gpu(raw_context, moment_out)
        ws, geo = self._prepare_waypoint_geometry(raw_context, include_passive_force_magnitude=False, compute_force_magnitudes=False)
        B, ne = raw_context.shape[0], len(self.sparse_entries.muscle_dof_torque_idx)
        moment = moment_out if moment_out is not None else torch.empty((B, ne), device=raw_context.device)
        _lib.check(
            _lib.lib().im_muscle_sparse_moment(
                C.byref(geo), C.byref(self._segments), self._dev["mom_torque"].data_ptr(), C.byref(self._moment_entries),
                self.root_dof_count, moment.data_ptr(), moment.stride(0), B, _stream(raw_context),
            ),
            "im_muscle_sparse_moment",
        )  # fmt: skip
        return moment

    def forward_from_activation(self, activation, raw_context, include_passive_force: bool | None = None):
        """Differentiable torque through the dispatcher operator."""
        from .warp_custom_ops import muscle_torque_forward, warp_op_key

        inc = self.include_passive_force_in_output if include_passive_force is None else bool(include_passive_force)
        return muscle_torque_forward(activation, raw_context, warp_op_key(self), inc)
