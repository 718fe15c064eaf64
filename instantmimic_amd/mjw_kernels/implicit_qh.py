"""The implicit-fast integrator's matrix ``qH = M - h dF/dv`` on M's pattern and the solve that
follows it: the host side of ``deriv_smooth_vel``, ``_prepare_implicit_qh`` and
``implicit_factor_optimized`` (src/instantmimic/utils/mjw_step_optimized.py:3803-3900, 3734-3745,
4936-4968).

The reference assembles qH with upstream's derivative kernels, which are not in its tree; the
terms here are the ones MuJoCo's ``mjd_smooth_vel`` documents for this integrator:

* joint damping: ``+ h dof_damping`` on the diagonal (``im_implicit_qh_base``),
* actuators with affine gain / bias: ``- h moment' diag(gain) moment`` with the gain of
  ``im_actuator_velocity_gain``,
* tendon damping: ``+ h J' diag(tendon_damping) J``,
* polynomial dampers (``dof_dampingpoly``, ``tendon_dampingpoly``): a damper whose force is
  ``-v (b + p_1 |v| + ... + p_K |v|^K)`` enters with its slope at the current velocity,
  ``b + 2 p_1 |v| + ... + (K + 1) p_K |v|^K``, in place of ``b`` (``im_polynomial_damping``),
* rows of free bodies reset to M (``_implicit_free_body_reset_m``): here those rows never receive
  a term, which leaves them equal to M,
* the registered contributors (the muscles' ``h A' diag(s) A``) on top.

The three pair sums over sparse rows go through the deterministic gather of
:mod:`instantmimic_amd.muscle.muscle_qfrc_projector` (``im_muscle_implicit_gather``), element by
element in a fixed order.  Fluid forces are not assembled: a model that has them is refused.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

import numpy as np

from .. import _lib
from ..muscle import muscle_qfrc_projector as MQ

# mjtDisableBit of MuJoCo 3.4 on (spring and damper split); a caller on another version passes its own
DISABLE_DAMPER = 1 << 6
DISABLE_ACTUATION = 1 << 11
GAIN_AFFINE = 1  # mjGAIN_AFFINE
BIAS_AFFINE = 1  # mjBIAS_AFFINE


def _host(a, dtype=np.int32) -> np.ndarray:
    if hasattr(a, "numpy") and not isinstance(a, np.ndarray):
        a = a.cpu().numpy() if hasattr(a, "cpu") else a.numpy()
    return np.ascontiguousarray(np.asarray(a), dtype)


def free_dofs(m: Any) -> np.ndarray:
    """Dofs of the model's free bodies (``m.body_freeadr`` lists the bodies, six dofs each from
    ``body_dofadr``), ascending."""
    free = getattr(m, "body_freeadr", None)
    if free is None or len(_host(free)) == 0:
        return np.zeros(0, np.int32)
    adr = _host(m.body_dofadr)[_host(free)]
    return np.sort((adr[:, None] + np.arange(6)[None, :]).reshape(-1)).astype(np.int32)


def element_dofs(m: Any, damper: bool = True) -> np.ndarray:
    """Per element of M's CSR: the dof whose damping it receives (its own diagonal, outside free
    bodies), else -1."""
    rowadr, rownnz, colind = _host(m.M_rowadr), _host(m.M_rownnz), _host(m.M_colind)
    rowi = np.repeat(np.arange(len(rowadr)), rownnz)
    out = np.where(rowi == colind, rowi, -1).astype(np.int32)
    if not damper:
        out[:] = -1
    free = free_dofs(m)
    out[np.isin(rowi, free)] = -1
    return out


def matrix_elemid(m: Any) -> np.ndarray:
    """(nv, nv) table: CSR index of M's element (i, j) in either order, -1 off the pattern and for
    every element in a free body's rows (those rows stay equal to M)."""
    rowadr, rownnz, colind = _host(m.M_rowadr), _host(m.M_rownnz), _host(m.M_colind)
    nv = len(rowadr)
    rowi = np.repeat(np.arange(nv), rownnz)
    keep = ~np.isin(rowi, free_dofs(m))
    out = np.full((nv, nv), -1, np.int32)
    idx = np.arange(len(colind), dtype=np.int32)
    out[rowi[keep], colind[keep]] = idx[keep]
    out[colind[keep], rowi[keep]] = idx[keep]
    return out


@dataclass
class RowPairGather:
    """Gather tables of ``sum_r weight_r row_r' row_r`` for sparse rows with a fixed pattern
    (actuator moments, tendon Jacobians): entries sorted by (row, dof)."""

    gather: Any  # MuscleImplicitQderivGather or None when no pair lands on the pattern
    entry_source: Any  # int64 tensor: position of every sorted entry in the caller's value array
    nrow: int
    dropped_pair_count: int


def row_pair_gather(rownnz, rowadr, colind, elemid: np.ndarray, device) -> RowPairGather:
    """Tables for rows given in CSR form (``rownnz``, ``rowadr``, ``colind`` as the model or the
    first world holds them; the pattern must be the same in every world)."""
    import torch

    rownnz, rowadr, colind = _host(rownnz), _host(rowadr), _host(colind)
    nrow = len(rownnz)
    rows = np.repeat(np.arange(nrow), rownnz)
    pos = np.concatenate([np.arange(a, a + n) for a, n in zip(rowadr, rownnz)]) if nrow else np.zeros(0, np.int64)
    dofs = colind[pos]
    order = np.lexsort((dofs, rows))
    rows, dofs, pos = rows[order], dofs[order], pos[order]
    if len(rows) and (np.diff(rows * (int(dofs.max()) + 1) + dofs) <= 0).any():
        raise ValueError("a sparse row lists a dof twice")
    ent = MQ.entries_from_muscle_dofs(np.stack([rows, dofs], 1), nrow) if len(rows) else None
    if ent is None:
        return RowPairGather(None, torch.zeros(0, dtype=torch.int64, device=device), nrow, 0)
    prepared = MQ.prepare_muscle_implicit_qderiv_pairs(
        pair_entry_i=ent.pair_entry_i, pair_entry_j=ent.pair_entry_j, pair_muscle_idx=ent.pair_muscle_idx,
        muscle_dof_torque_idx=ent.muscle_dof_torque_idx, matrix_elemid=elemid, root_dof_count=0,
    )  # fmt: skip
    gather = MQ.build_muscle_implicit_qderiv_gather(prepared, ent.muscle_dof_muscle_idx, device)
    if gather is None and len(prepared.pair_elem_id):
        raise ValueError("the pair tables exceed the gather kernel's limits")
    return RowPairGather(gather, torch.from_numpy(pos.astype(np.int64)).to(device), nrow, prepared.dropped_pair_count)


@dataclass
class ImplicitQhScratch:
    """What the implicit-fast step keeps between calls (the reference's ``implicit_qderiv``,
    ``implicit_qacc`` and ``implicit_qh_contributors`` of its position scratch, :505-520)."""

    elem_dof: Any
    actuators: RowPairGather | None
    tendons: RowPairGather | None
    tendon_damping: Any
    implicit_qderiv: Any
    implicit_qacc: Any
    actuator_gain: Any
    timestep: float
    implicit_qh_contributors: tuple = ()
    dense_factor_solve: Any = None
    tree_factor_solve: Any = None
    implicit_factor_workspace: Any = None
    tables: dict = field(default_factory=dict)


def _flag(m: Any, bit: int) -> bool:
    return bool(int(getattr(getattr(m, "opt", None), "disableflags", 0)) & bit)


def create_implicit_qh_scratch(m: Any, d: Any, device, *, disable_damper=DISABLE_DAMPER, disable_actuation=DISABLE_ACTUATION) -> ImplicitQhScratch:
    """Tables and buffers for a model: ``m`` needs M's CSR, ``dof_damping``, ``opt.timestep`` and,
    where present, ``body_freeadr`` / ``body_dofadr``, the actuator arrays (``nactuator``,
    ``actuator_gaintype``, ``actuator_biastype``, ``actuator_gainprm``, ``actuator_biasprm``) and
    the tendon arrays (``ntendon``, ``ten_J_rownnz / rowadr / colind``, ``tendon_damping``);
    ``d`` the moment pattern (``moment_rownnz / rowadr / colind``) and ``nworld``."""
    import torch

    if getattr(m, "has_fluid", False):
        raise NotImplementedError("fluid forces are not part of this qH")
    dev = torch.device(device)
    nworld, nM = int(d.nworld), len(_host(m.M_colind))
    damper = not _flag(m, disable_damper)
    elemid = matrix_elemid(m)
    actuators = tendons = tendon_damping = gain = None
    nu = int(getattr(m, "nactuator", 0) or 0)
    if nu > 0 and not _flag(m, disable_actuation):
        for name, allowed in (("actuator_gaintype", (0, GAIN_AFFINE)), ("actuator_biastype", (0, BIAS_AFFINE))):
            if not np.isin(_host(getattr(m, name)), allowed).all():
                raise NotImplementedError(f"{name}: only fixed and affine actuators have a velocity gain here")
        actuators = row_pair_gather(_host(d.moment_rownnz).reshape(-1, nu)[0], _host(d.moment_rowadr).reshape(-1, nu)[0],
                                    _host(d.moment_colind).reshape(nworld if _host(d.moment_colind).ndim > 1 else 1, -1)[0], elemid, dev)  # fmt: skip
        gain = torch.zeros((nworld, nu), device=dev)
    nt = int(getattr(m, "ntendon", 0) or 0)
    tables = {}
    tendon_poly = _polynomial(getattr(m, "tendon_dampingpoly", None), nt, dev) if nt > 0 and damper else None
    if nt > 0 and damper and (np.any(_host(m.tendon_damping, np.float32) != 0) or tendon_poly is not None):
        tendons = row_pair_gather(m.ten_J_rownnz, m.ten_J_rowadr, m.ten_J_colind, elemid, dev)
        td = torch.from_numpy(_host(m.tendon_damping, np.float32).reshape(-1, nt)).to(dev)
        tendon_damping = td.expand(nworld, nt).contiguous()
        if tendon_poly is not None:
            tables["tendon_poly"], tables["tendon_base"] = tendon_poly, tendon_damping.clone()
    dof_poly = _polynomial(getattr(m, "dof_dampingpoly", None), int(m.nv), dev) if damper else None
    if dof_poly is not None:
        tables["dof_poly"], tables["dof_effective"] = dof_poly, torch.zeros((nworld, int(m.nv)), device=dev)
    return ImplicitQhScratch(
        elem_dof=torch.from_numpy(element_dofs(m, damper)).to(dev), actuators=actuators, tendons=tendons,
        tendon_damping=tendon_damping, implicit_qderiv=torch.zeros((nworld, nM), device=dev),
        implicit_qacc=torch.zeros((nworld, int(m.nv)), device=dev), actuator_gain=gain,
        timestep=float(np.asarray(_host(m.opt.timestep, np.float32)).reshape(-1)[0]), tables=tables,
    )  # fmt: skip


def _polynomial(poly, n: int, dev):
    """The coefficients of |v|, |v|^2, ... of a polynomial damper as a (1 or nworld, n, K) device
    tensor; ``None`` when the model has none or all are zero."""
    import torch

    if poly is None:
        return None
    p = _host(poly, np.float32)
    if p.size == 0 or not np.any(p != 0):
        return None
    if p.size % n:
        raise ValueError("polynomial damping coefficients do not match the number of dofs or tendons")
    if p.ndim == 3:
        p = p.reshape(p.shape[0], n, -1)
    else:
        p = p.reshape(1, n, -1)
    return torch.from_numpy(np.ascontiguousarray(p)).to(dev)


def polynomial_damping(base, poly, velocity, out) -> None:
    """``out[w, i] = base[w, i] + sum_k (k + 1) poly[w, i, k - 1] |velocity[w, i]|^k``
    (``im_polynomial_damping``): the damping coefficient the implicit matrix sees."""
    import torch

    nworld, n = int(velocity.shape[0]), int(out.shape[1])
    for t in (base, poly, velocity, out):
        if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
            raise TypeError("polynomial damping takes contiguous float32 CUDA tensors")
    with torch.cuda.device(out.device):
        status = _lib.lib().im_polynomial_damping(
            base.data_ptr(), base.stride(0) if base.shape[0] > 1 else 0, poly.data_ptr(),
            poly.stride(0) if poly.shape[0] > 1 else 0, int(poly.shape[2]), velocity.data_ptr(), velocity.stride(0),
            out.data_ptr(), out.stride(0), n, nworld, _stream(out),
        )  # fmt: skip
    _lib.check(status, "im_polynomial_damping")


def _stream(t) -> int:
    import torch

    return int(torch.cuda.current_stream(t.device).cuda_stream)


def actuator_velocity_gain(m: Any, d: Any, scratch: ImplicitQhScratch) -> None:
    """``scratch.actuator_gain[w, a]``: d force / d velocity of every actuator."""
    import torch

    t, inp, force = _actuator_inputs(m, d, scratch)
    gain, nu = scratch.actuator_gain, scratch.actuator_gain.shape[1]
    with torch.cuda.device(gain.device):
        status = _lib.lib().im_actuator_velocity_gain(
            t["gaintype"].data_ptr(), t["biastype"].data_ptr(), t["gainprm"].data_ptr(), t["biasprm"].data_ptr(),
            int(t["gainprm"].shape[1]), None if t["forcelimited"] is None else t["forcelimited"].data_ptr(),
            None if t["forcerange"] is None else t["forcerange"].data_ptr(), inp.data_ptr(), inp.stride(0),
            None if force is None else force.data_ptr(), 0 if force is None else force.stride(0), gain.data_ptr(),
            gain.stride(0), int(nu), int(gain.shape[0]), _stream(gain),
        )  # fmt: skip
    _lib.check(status, "im_actuator_velocity_gain")


def _actuator_inputs(m: Any, d: Any, scratch: ImplicitQhScratch):
    """The actuators' parameter tables on the device (made once), what drives each gain, and the
    forces that the force range is tested against (or None)."""
    import torch

    dev = scratch.actuator_gain.device
    t = scratch.tables
    if "gaintype" not in t:
        nu = scratch.actuator_gain.shape[1]
        t["gaintype"] = torch.from_numpy(_host(m.actuator_gaintype)).to(dev)
        t["biastype"] = torch.from_numpy(_host(m.actuator_biastype)).to(dev)
        t["gainprm"] = torch.from_numpy(_host(m.actuator_gainprm, np.float32).reshape(-1, nu, _host(m.actuator_gainprm, np.float32).shape[-1])[0].copy()).to(dev)
        t["biasprm"] = torch.from_numpy(_host(m.actuator_biasprm, np.float32).reshape(-1, nu, _host(m.actuator_biasprm, np.float32).shape[-1])[0].copy()).to(dev)
        limited = getattr(m, "actuator_forcelimited", None)
        t["forcelimited"] = None if limited is None else torch.from_numpy(_host(limited, np.uint8)).to(dev)
        t["forcerange"] = None if limited is None else torch.from_numpy(_host(m.actuator_forcerange, np.float32).reshape(-1, nu, 2)[0].copy()).to(dev)
        # what drives the gain: the control, or the last activation variable of a stateful actuator
        actadr, actnum = getattr(m, "actuator_actadr", None), getattr(m, "actuator_actnum", None)
        t["act_index"] = None
        if actadr is not None and actnum is not None and (_host(actnum) > 0).any():
            adr, num = _host(actadr), _host(actnum)
            t["act_index"] = (torch.from_numpy(np.flatnonzero(num > 0)).to(dev), torch.from_numpy((adr + num - 1)[num > 0].astype(np.int64)).to(dev))
    inp = d.ctrl
    if t["act_index"] is not None:
        inp = d.ctrl.clone()
        inp[:, t["act_index"][0]] = d.act[:, t["act_index"][1]]
    force = getattr(d, "actuator_force", None) if t["forcelimited"] is not None else None
    if inp.dtype != torch.float32 or inp.stride(1) != 1 or inp.shape != scratch.actuator_gain.shape:
        raise TypeError("ctrl must be a float32 (nworld, nactuator) tensor with contiguous rows")
    return t, inp, force


def _pair_term(rows: RowPairGather, values, weight, scale: float):
    """im_row_pair_term of a row set: the caller's values are read through ``entry_source``."""
    g = rows.gather
    if g is None:
        return None
    if "source32" not in rows.__dict__:
        import torch

        rows.source32 = rows.entry_source.to(dtype=torch.int32)
    term = _lib.RowPairTerm()
    term.values, term.ld_values = values.data_ptr(), values.stride(0)
    term.entry_source, term.entry_row, term.nentry = rows.source32.data_ptr(), g.entry_muscle.data_ptr(), int(g.entry_count)
    term.elem_ids, term.nelem = g.elem_ids.data_ptr(), int(g.elem_ids.numel())
    term.chunk_offsets, term.chunk_pairs, term.chunk_count = g.chunk_offsets.data_ptr(), g.chunk_pairs.data_ptr(), int(g.chunk_count)
    term.weight, term.ld_weight = (None, 0) if weight is None else (weight.data_ptr(), weight.stride(0))
    term.scale = float(scale)
    return term


def _deriv_smooth_vel_fused(m, d, out, scratch: ImplicitQhScratch, damping, nworld: int, nM: int) -> bool:
    """The whole of ``deriv_smooth_vel`` through im_implicit_qh; False when a world's rows do not
    fit the kernel's LDS (the caller then makes the separate calls)."""
    import ctypes as C

    import torch

    acts = scratch.actuators is not None and scratch.actuators.gather is not None
    tens = scratch.tendons is not None and scratch.tendons.gather is not None
    if scratch.actuators is not None:
        t, inp, force = _actuator_inputs(m, d, scratch)
        gain = scratch.actuator_gain
        gain_args = [t["gaintype"].data_ptr(), t["biastype"].data_ptr(), t["gainprm"].data_ptr(), t["biasprm"].data_ptr(),
                     int(t["gainprm"].shape[1]), None if t["forcelimited"] is None else t["forcelimited"].data_ptr(),
                     None if t["forcerange"] is None else t["forcerange"].data_ptr(), inp.data_ptr(), inp.stride(0),
                     None if force is None else force.data_ptr(), 0 if force is None else force.stride(0), gain.data_ptr(),
                     gain.stride(0), int(gain.shape[1])]  # fmt: skip
    else:
        gain_args = [None, None, None, None, 0, None, None, None, 0, None, 0, None, 0, 0]
    ta = tt = None
    if acts:
        values = d.actuator_moment.reshape(nworld, -1)
        if values.dtype != torch.float32 or values.stride(1) != 1:
            return False
        ta = _pair_term(scratch.actuators, values, None, -scratch.timestep)
    if tens:
        values = d.ten_J.reshape(nworld, -1)
        if values.dtype != torch.float32 or values.stride(1) != 1:
            return False
        tt = _pair_term(scratch.tendons, values, scratch.tendon_damping, scratch.timestep)
    with torch.cuda.device(out.device):
        status = _lib.lib().im_implicit_qh(
            d.M.data_ptr(), d.M.stride(0), nM, scratch.elem_dof.data_ptr(), damping.data_ptr(),
            damping.stride(0) if damping.shape[0] > 1 else 0, scratch.timestep, *gain_args,
            None if ta is None else C.byref(ta), None if tt is None else C.byref(tt), out.data_ptr(), out.stride(0), nworld,
            _stream(out),
        )  # fmt: skip
    if status == _lib.IM_ERR_UNSUPPORTED:
        return False
    _lib.check(status, "im_implicit_qh")
    return True


def deriv_smooth_vel(m: Any, d: Any, out, scratch: ImplicitQhScratch, *, fused: bool = True) -> None:
    """``out = M - h qDeriv`` on M's pattern (:3803-3900): damping, actuators, tendon damping.
    ``fused``: one launch (im_implicit_qh) where a world's rows fit its LDS; otherwise, and with
    ``fused=False``, the base, the gains and one gather per term as separate launches.  The two
    forms give the same bits."""
    import torch

    M = d.M
    damping = scratch.tables.get("damping")
    if damping is None:
        damping = scratch.tables["damping"] = torch.from_numpy(_host(m.dof_damping, np.float32).reshape(-1, int(m.nv))).to(out.device)
    if M.dtype != torch.float32 or out.dtype != torch.float32 or M.stride(1) != 1 or out.stride(1) != 1 or M.shape != out.shape:
        raise TypeError("M and out must be float32 (nworld, nM) tensors with contiguous rows")
    nworld, nM = int(M.shape[0]), int(scratch.elem_dof.numel())
    # polynomial dampers (dof_dampingpoly, tendon_dampingpoly): their slope at the current velocity
    # takes the place of the constant coefficient
    if "dof_poly" in scratch.tables:
        polynomial_damping(damping, scratch.tables["dof_poly"], d.qvel.reshape(nworld, -1), scratch.tables["dof_effective"])
        damping = scratch.tables["dof_effective"]
    if "tendon_poly" in scratch.tables:
        polynomial_damping(scratch.tables["tendon_base"], scratch.tables["tendon_poly"], d.ten_velocity.reshape(nworld, -1), scratch.tendon_damping)
    if fused and _deriv_smooth_vel_fused(m, d, out, scratch, damping, nworld, nM):
        return
    with torch.cuda.device(out.device):
        status = _lib.lib().im_implicit_qh_base(
            M.data_ptr(), M.stride(0), nM, scratch.elem_dof.data_ptr(), damping.data_ptr(),
            damping.stride(0) if damping.shape[0] > 1 else 0, scratch.timestep, out.data_ptr(), out.stride(0), nworld,
            _stream(out),
        )  # fmt: skip
    _lib.check(status, "im_implicit_qh_base")
    if scratch.actuators is not None and scratch.actuators.gather is not None:
        actuator_velocity_gain(m, d, scratch)
        moment = d.actuator_moment.reshape(nworld, -1).index_select(1, scratch.actuators.entry_source)
        MQ.apply_muscle_implicit_qderiv_gather(scratch.actuators.gather, moment, scratch.actuator_gain, -scratch.timestep, out)
    if scratch.tendons is not None and scratch.tendons.gather is not None:
        ten_J = d.ten_J.reshape(nworld, -1).index_select(1, scratch.tendons.entry_source)
        MQ.apply_muscle_implicit_qderiv_gather(scratch.tendons.gather, ten_J, scratch.tendon_damping, scratch.timestep, out)


def _prepare_implicit_qh(m: Any, d: Any, scratch: ImplicitQhScratch, qh) -> None:
    """The registered contributors on top of ``deriv_smooth_vel`` (:3727-3745).  The free bodies'
    rows need no reset: no table of this module writes to them."""
    for contributor in getattr(scratch, "implicit_qh_contributors", ()):
        contributor.apply(qh)


def implicit_factor_optimized(m: Any, d: Any, scratch: ImplicitQhScratch, rhs=None):
    """``scratch.implicit_qacc = qH^-1 rhs`` (``d.efc.Ma`` by default) with the tree L'DL or the
    blocked Cholesky, whichever ``_factor_solve_i_dense`` takes (:4936-4968, without the
    free-body correction and the integration step that follow it there)."""
    from . import blocked_dense as BD

    qderiv, qacc = scratch.implicit_qderiv, scratch.implicit_qacc
    if qderiv is None or qacc is None:
        raise RuntimeError("implicit factor integration requires qDeriv/qacc scratch")
    deriv_smooth_vel(m, d, qderiv, scratch)
    _prepare_implicit_qh(m, d, scratch, qderiv)
    BD._factor_solve_i_dense(
        m, d, qderiv, qacc, d.efc.Ma if rhs is None else rhs, scratch.dense_factor_solve,
        factor_workspace=scratch.implicit_factor_workspace, tree_factor_solve=scratch.tree_factor_solve,
    )  # fmt: skip
    return qacc
