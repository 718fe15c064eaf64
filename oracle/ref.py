"""ctypes front end of ``cpu_ref.c`` plus fp64 NumPy references (oracle only).

Pinning status

* ``assemble_csr``            pinned: fp64 ``einsum`` of ``M + J' diag(D active) J``
                              gathered on the CSR entries (tests/test_oracle.py).
* ``tree_ldl_solve``          pinned: fp64 ``numpy.linalg.solve`` on well-conditioned
                              matrices (the reference's own check,
                              tests/test_tree_ldl.py:119-120), the invariant
                              ``L' D L == H`` rebuilt from the returned factor, brute force
                              Gaussian elimination on tiny trees, and independence of the
                              result (to rounding) from the number of groups.
* ``assemble_tree_ldl_solve`` composition of the two above; pinned through them.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build() -> str:
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return os.path.join(_HERE, "_build", "liboracle.so")


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "_build", "liboracle.so")
        src = os.path.join(_HERE, "cpu_ref.c")
        if not os.path.exists(path) or os.path.getmtime(path) < os.path.getmtime(src):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _i(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _f(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def max_threads() -> int:
    return int(lib().orc_max_threads())


def set_threads(n: int) -> None:
    lib().orc_set_threads(int(n))


def _plan_arrays(plan):
    gptr = [0]
    gd = []
    for g in plan.groups:
        gd += list(g)
        gptr.append(len(gd))
    return _i(gptr), _i(gd if gd else [0]), _i(plan.trunk if plan.trunk else [0])


def rows_of(rownnz):
    return np.repeat(np.arange(len(rownnz)), np.asarray(rownnz)).astype(np.int32)


def assemble_csr(rowadr, rownnz, colind, M, J, D, state, nefc=None, quad=1):
    M, J, D = _f(M), _f(J), _f(D)
    state = _i(state)
    nworld, nM = M.shape
    njmax, nv = J.shape[1], J.shape[2]
    H = np.empty_like(M)
    ne = _i(nefc) if nefc is not None else None
    lib().orc_assemble_csr(
        nworld, nv, nM, _p(rows_of(rownnz)), _p(_i(colind)), _p(M), _p(J), njmax, _p(D), _p(state), _p(ne), quad, _p(H)
    )
    return H


def tree_ldl_solve(rowadr, rownnz, colind, plan, H, y, want_factor=False):
    H, y = _f(H), _f(y)
    nworld, nM = H.shape
    nv = y.shape[1]
    gptr, gd, trunk = _plan_arrays(plan)
    x = np.empty_like(y)
    ld = np.empty_like(H) if want_factor else None
    lib().orc_tree_ldl_solve(
        nworld, nv, nM, _p(_i(rowadr)), _p(_i(rownnz)), _p(_i(colind)), len(plan.groups), _p(gptr), _p(gd),
        len(plan.trunk), _p(trunk), _p(H), _p(y), _p(x), _p(ld),
    )  # fmt: skip
    return (x, ld) if want_factor else x


def assemble_tree_ldl_solve(rowadr, rownnz, colind, plan, M, J, D, state, nefc, grad, quad=1, want_h=False):
    M, J, D, grad = _f(M), _f(J), _f(D), _f(grad)
    state = _i(state)
    nworld, nM = M.shape
    njmax, nv = J.shape[1], J.shape[2]
    gptr, gd, trunk = _plan_arrays(plan)
    x = np.empty_like(grad)
    H = np.empty_like(M) if want_h else None
    ne = _i(nefc) if nefc is not None else None
    lib().orc_assemble_tree_ldl_solve(
        nworld, nv, nM, _p(_i(rowadr)), _p(_i(rownnz)), _p(_i(colind)), _p(rows_of(rownnz)), len(plan.groups),
        _p(gptr), _p(gd), len(plan.trunk), _p(trunk), _p(M), _p(J), njmax, _p(D), _p(state), _p(ne), quad,
        _p(grad), _p(x), _p(H),
    )  # fmt: skip
    return (x, H) if want_h else x


# ---------------------------------------------------------------- fp64 references


def dense_from_csr(values, rowadr, rownnz, colind):
    nv = len(rowadr)
    rowi = rows_of(rownnz)
    out = np.zeros((values.shape[0], nv, nv), np.float64)
    out[:, rowi, colind] = values
    out[:, colind, rowi] = values
    return out


def assemble_dense64(rowadr, rownnz, colind, M, J, D, state, nefc=None, quad=1):
    """fp64 dense ``M + J' diag(D [state == quad]) J`` (all rows, no pattern)."""
    J64 = np.asarray(J, np.float64)
    w = np.where(np.asarray(state) == quad, np.asarray(D, np.float64), 0.0)
    if nefc is not None:
        w = w * (np.arange(J64.shape[1])[None, :] < np.asarray(nefc)[:, None])
    return dense_from_csr(np.asarray(M, np.float64), rowadr, rownnz, colind) + np.einsum("wri,wr,wrj->wij", J64, w, J64)


def solve64(Hd, y):
    return np.linalg.solve(Hd, np.asarray(y, np.float64)[..., None])[..., 0]


def rel_l2(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


# ---------------------------------------------------------------- muscle contractions
# Pinning: `muscle_project` against a dense fp64 A' f, `muscle_implicit_gather` against a
# dense fp64 h A' diag(s) A restricted to M's pattern (tests/test_muscle.py); the index
# tables against brute-force enumeration there as well.  The reference's own tests do not
# cover these kernels.


def muscle_project(moment, force, offsets, entry_idx, entry_muscle, root, nv):
    moment, force = _f(moment), _f(force)
    nworld, nentry = moment.shape
    qfrc = np.zeros((nworld, nv), np.float32)
    lib().orc_muscle_project(
        nworld, nentry, force.shape[1], len(offsets) - 1, _p(moment), _p(force), _p(_i(offsets)), _p(_i(entry_idx)),
        _p(_i(entry_muscle)), int(root), _p(qfrc), nv,
    )  # fmt: skip
    return qfrc


def muscle_implicit_gather(moment, slope, entry_muscle, elem_ids, chunk_offsets, chunk_pairs, chunk_count, timestep, qderiv):
    moment, slope = _f(moment), _f(slope)
    out = np.array(qderiv, np.float32, copy=True, order="C")
    lib().orc_muscle_implicit_gather.argtypes = None
    lib().orc_muscle_implicit_gather(
        moment.shape[0], moment.shape[1], slope.shape[1], len(elem_ids), int(chunk_count), 16, _p(moment), _p(slope),
        _p(_i(entry_muscle)), _p(_i(elem_ids)), _p(_i(chunk_offsets)), _p(_i(chunk_pairs)), ctypes.c_float(timestep),
        _p(out), out.shape[1],
    )  # fmt: skip
    return out


# ---------------------------------------------------------------- static-pattern sparse L'DL
# Pinning: the level/run/backward tables are executed in fp64 as parallel sweeps with a
# race check per level (the executor the reference's own test holds,
# tests/test_mjw_sparse_hessian.py:199-262) and must solve H x = g to 1e-10; the fp32
# lane-by-lane C executor is then checked against that fp64 result within conditioning.

TABLE_ORDER = ("SH_LP", "SH_LT", "SH_ES", "SH_EC", "SH_RP", "SH_RAB", "SH_RKL", "SH_ORIG", "SH_BL", "SH_BS", "SH_BI",
               "SH_BJ", "SH_PM", "SH_SA", "SH_SB", "SH_SM")  # fmt: skip


def run_tables64(T, nv, nslots, H, g):
    """Factor and solve through the tables in fp64, each level as one parallel sweep
    (every lane reads the level's input snapshot); asserts that no level writes what
    another lane of it reads or writes.  Returns x = H^-1 g."""
    nfac = nslots - nv
    u = lambda k: T[k].astype(np.int64) & 0xFFFFFFFF  # noqa: E731
    N, iD = np.zeros(nslots), np.zeros(nv)
    pair = T["SH_PAIR"].reshape(nv, nv)
    for s in range(nfac):
        a, b = T["SH_SA"][s], T["SH_SB"][s]
        assert pair[a, b] == s
        N[s] = H[a, b]
    words = (nv + 31) // 32
    pm = u("SH_PM")
    for a in range(nv):
        for b in range(a, nv):
            in_mask = (pm[a * words + b // 32] >> (b % 32)) & 1
            assert bool(in_mask) == (pair[a, b] >= 0 or a == b)
            assert H[a, b] == 0.0 or pair[a, b] >= 0
    orig = T["SH_ORIG"]
    N[nfac:] = g[orig]
    LP, ES, EC, RP = T["SH_LP"], T["SH_ES"], T["SH_EC"], T["SH_RP"]
    RAB, RKL = u("SH_RAB"), u("SH_RKL")
    for lvl in range(len(LP) - 1):
        n0, d0 = N.copy(), iD.copy()
        written, read = set(), set()
        for e in range(LP[lvl], LP[lvl + 1]):
            v = 0.0
            for r in range(RP[e], RP[e + 1]):
                a, b, k, ln = RAB[r] & 0xFFFF, RAB[r] >> 16, RKL[r] & 0xFFFF, RKL[r] >> 16
                v += float(np.sum(n0[a : a + ln] * n0[b : b + ln] * d0[k : k + ln]))
                read |= {*range(a, a + ln), *range(b, b + ln), *range(-k - ln, -k)}
            assert ES[e] not in written
            written.add(int(ES[e]))
            N[ES[e]] = n0[ES[e]] - v
            if EC[e] >= 0:
                iD[EC[e]] = 1.0 / N[ES[e]]
                written.add(-1 - int(EC[e]))
        assert not written & read
    BL, BS, BI, BJ = T["SH_BL"], T["SH_BS"], T["SH_BI"], T["SH_BJ"]
    for lvl in range(len(BL) - 1):
        z = N[nfac:].copy()
        src, dst = set(), set()
        for p in range(BL[lvl], BL[lvl + 1]):
            i, j = int(BI[p]), int(BJ[p])
            assert j not in dst, "two pushes to one unknown in a level"
            src.add(i)
            dst.add(j)
            N[nfac + j] = z[j] - N[BS[p]] * (z[i] * iD[i])
        assert not src & dst
    x = np.zeros(nv)
    x[orig] = N[nfac:] * iD
    return x


def sparse_plan(m, body_groups, block, path="fused"):
    """The oracle's own plan of a model (planner.sparse_pattern + planner.sparse_tables): what
    ``sparse_init_factor`` / ``sparse_update_factor`` execute, independent of the product's planner."""
    from . import planner

    return planner.sparse_tables(int(m.nv), int(m.nv_pad), planner.sparse_pattern(m, body_groups), m.M_hinit_i, m.M_colind, block, path)


def sparse_init_factor(plan, nefc, J, D, state, M, grad, hfactor=None, done=None, quad=1):
    """fp32 lane-by-lane restatement of the initial assemble + factor + solve kernel."""
    J, D, M, grad = _f(J), _f(D), _f(M), _f(grad)
    state, nefc = _i(state), _i(nefc)
    nworld, njmax, nv = J.shape
    tabs = [np.ascontiguousarray(plan.tables[k], np.int32) for k in TABLE_ORDER]
    ptrs = (ctypes.c_void_p * len(tabs))(*[t.ctypes.data for t in tabs])
    hf = np.zeros((nworld, plan.nv_pad, plan.nv_pad), np.float32) if hfactor is None else np.array(hfactor, np.float32, order="C")
    search = np.zeros((nworld, nv), np.float32)
    sdot = np.zeros(nworld, np.float32)
    decr = np.zeros(nworld, np.float32)
    dn = None if done is None else np.ascontiguousarray(done, np.uint8)
    status = lib().orc_sparse_init_factor(
        plan.nv, plan.nv_pad, plan.block, plan.nslots, plan.levels, ptrs, nworld, _p(dn), _p(nefc), _p(J), njmax, _p(D),
        _p(state), quad, _p(M), M.shape[1], _p(grad), grad.shape[1], _p(hf), _p(search), _p(sdot), _p(decr),
    )  # fmt: skip
    assert status == 0
    return hf, search, sdot, decr


# ---------------------------------------------------------------- blocked dense Cholesky, dense J'DJ
# Pinning: `blocked_factor_solve` against scipy.linalg.cho_factor / cho_solve in fp64 and the
# invariant U'U == M; the order inside a tile operation is this oracle's own convention (the
# reference's tile arithmetic is Warp's, third party): bit-level parity with the reference is
# UNPINNED for this function, tolerance parity is pinned.  `jtdj_dense` against fp64 einsum.


def blocked_factor_solve(M, block_idx, nv, pad, B, y, want_factor=True):
    M, y = _f(M), _f(y)
    nworld, nM = M.shape
    U = np.zeros((nworld, pad, pad), np.float32) if want_factor else None
    x = np.zeros((nworld, nv), np.float32)
    lib().orc_blocked_factor_solve(nworld, nv, pad, B, nM, _p(M), nM, _p(_i(block_idx)), _p(y), _p(U), _p(x))
    return (x, U) if want_factor else x


def tile_cholesky_solve(M, adr, size, y, elemid=None):
    """x = tile^-1 y for every diagonal tile of ``size`` dofs starting at ``adr[t]``: ``M`` dense
    (nworld, n, n) without ``elemid``, else (nworld, nM) values gathered through ``elemid``
    (ntile * size * size ids).  Pinned by tests/test_tile_cholesky.py: scipy's ``cho_solve`` in
    fp64 within conditioning, ``L L' == A`` through the blocked factor of the same matrix (up to
    16 dofs the two are the same operations: bit-equal), dofs outside every tile untouched."""
    M, y, adr = _f(M), _f(y), _i(adr)
    nworld = M.shape[0]
    x = np.zeros_like(y)
    L = ctypes.c_long
    if elemid is None:
        n = M.shape[1]
        st = lib().orc_tile_cholesky_solve(nworld, int(size), adr.size, _p(adr), _p(M), L(n * n), L(n), None, 0, _p(y),
                                           L(y.shape[1]), _p(x), L(x.shape[1]))  # fmt: skip
    else:
        ids = _i(elemid)
        st = lib().orc_tile_cholesky_solve(nworld, int(size), adr.size, _p(adr), _p(M), L(M.shape[1]), L(0), _p(ids),
                                           M.shape[1], _p(y), L(y.shape[1]), _p(x), L(x.shape[1]))  # fmt: skip
    assert st == 0
    return x


def blocked_multi_solve(U, nv, B, y, active=None, x=None):
    """Solve with stored factors U (nworld, pad, pad) for y (nworld, nv, nrhs); inactive worlds
    keep ``x`` (zeros when not given)."""
    U, y = _f(U), _f(y)
    nworld, pad, _ = U.shape
    nrhs = y.shape[2]
    x = np.zeros_like(y) if x is None else _f(x).copy()
    act = _i(active) if active is not None else None
    lib().orc_blocked_multi_solve(nworld, nv, pad, B, _p(U), _p(y), nrhs, _p(act), _p(x))
    return x


def jtdj_dense(Mdense, J, D, state, nefc, nv_pad, quad=1):
    Mdense, J, D = _f(Mdense), _f(J), _f(D)
    state = _i(state)
    nworld, njmax, nv = J.shape
    H = np.zeros((nworld, nv_pad, nv_pad), np.float32)
    ne = _i(nefc) if nefc is not None else None
    lib().orc_jtdj_dense(nworld, nv, nv_pad, _p(Mdense), _p(J), njmax, _p(D), _p(state), _p(ne), quad, _p(H))
    return H


# ---------------------------------------------------------------- muscle geometry, torque ops
# Pinning (tests/test_muscle_dynamics.py): `muscle_waypoints` against fp64 rotation matrices
# built from the quaternions; `muscle_force_magnitudes` against an fp64 evaluation of the
# four curves and the closed form of the reference's two-body fixture
# (tests/muscle_warp_fixtures.py:17-180: one segment (0,1,0)->(2,1,0), gaussian gamma 0.45,
# normalised length clamped to 1.4, unit force exp(-0.16/0.45)); `muscle_torque_forward`
# against the same fixture's closed form (torque[1] = sum_m unit_m act_m, torque[0] = 0) and
# a dense fp64 evaluation from the unsparsified subtree masks; `muscle_activation_grad`
# against central finite differences of the forward in fp64 and the transpose identity
# <g, T a> = <T' g, a>; `muscle_sparse_moment` against d torque / d force in fp64.
# Bit-level agreement with the reference's Warp build is unpinned: Warp's lowering of the
# vec3 expressions (operation association, contraction under NVRTC) is not visible from its
# Python source and `rot_vec_quat` lives in mujoco_warp, which is not in the tree.


def muscle_waypoints(xpos, xquat, wp_body, wp_local):
    xpos, xquat, wp_local = _f(xpos), _f(xquat), _f(wp_local)
    nworld, nbody = xpos.shape[0], xpos.shape[1]
    out = np.zeros((nworld, len(wp_body), 3), np.float32)
    lib().orc_muscle_waypoints(nworld, nbody, len(wp_body), _p(xpos), _p(xquat), _p(_i(wp_body)), _p(wp_local), _p(out))
    return out


def muscle_force_magnitudes(waypoints, seg_start, seg_offsets, params, rest, model, include_passive=True):
    """model = (force_scale, lnorm_min, lnorm_max, active[3], passive[3]) flattened to 9 floats."""
    waypoints, params = _f(waypoints), _f(params)
    nworld, nwp = waypoints.shape[0], waypoints.shape[1]
    nmuscle = len(seg_offsets) - 1
    unit = np.zeros((nworld, nmuscle), np.float32)
    passive = np.zeros((nworld, nmuscle), np.float32)
    lib().orc_muscle_force_magnitudes(
        nworld, nwp, nmuscle, _p(waypoints), _p(_i(seg_start)), _p(_i(seg_offsets)), _p(params), params.shape[1],
        _p(_f(rest)), _p(_f(model)), int(bool(include_passive)), _p(unit), _p(passive),
    )  # fmt: skip
    return unit, passive


def muscle_force_velocity_state(waypoints, wp_start, params, rest, length_scale, act, qvel, moment, dof_offsets,
                                dof_torque, root, model, fv):
    """model = the 9 floats of muscle_force_magnitudes; fv = (vmax, fvmax, clamp_activation,
    include_active).  Returns (length, effective_activation, velocity, multiplier, slope)."""
    waypoints, params, act, qvel, moment = _f(waypoints), _f(params), _f(act), _f(qvel), _f(moment)
    nworld, nwp = waypoints.shape[0], waypoints.shape[1]
    nmuscle = len(wp_start) - 1
    out = np.zeros((5, nworld, nmuscle), np.float32)
    lib().orc_muscle_force_velocity_state(
        nworld, nwp, nmuscle, moment.shape[1], qvel.shape[1], _p(waypoints), _p(_i(wp_start)), _p(params),
        params.shape[1], _p(_f(rest)), _p(_f(length_scale)), _p(act), _p(qvel), _p(moment), _p(_i(dof_offsets)),
        _p(_i(dof_torque)), int(root), _p(_f(model)), _p(_f(fv)), _p(out),
    )  # fmt: skip
    return tuple(out)


def _geo(waypoints, com, cdof):
    waypoints, com, cdof = _f(waypoints), _f(com), _f(cdof)
    return waypoints, com, cdof, (waypoints.shape[0], waypoints.shape[1], com.shape[1], cdof.shape[1])


def muscle_torque_forward(waypoints, com, cdof, seg, entries, unit, passive, act, root):
    """seg = (p0, p1, b0, b1); entries = (offsets, segment, muscle, start_coeff, end_coeff)."""
    waypoints, com, cdof, (nworld, nwp, nbody, nv) = _geo(waypoints, com, cdof)
    unit, act = _f(unit), _f(act)
    passive = None if passive is None else _f(passive)
    off, es, em, ea, eb = entries
    ntorque = len(off) - 1
    out = np.zeros((nworld, ntorque), np.float32)
    s = [_i(a) for a in seg]
    keep = [_i(off), _i(es), _i(em), _f(ea), _f(eb)]
    lib().orc_muscle_torque_forward(
        nworld, nwp, nbody, nv, unit.shape[1], ntorque, _p(waypoints), _p(com), _p(cdof), *[_p(a) for a in s],
        *[_p(a) for a in keep], _p(unit), _p(passive), _p(act), int(root), _p(out),
    )  # fmt: skip
    return out


def muscle_activation_grad(waypoints, com, cdof, seg, entries, unit, gout, root):
    """entries = (offsets, segment, torque, start_coeff, end_coeff) per muscle."""
    waypoints, com, cdof, (nworld, nwp, nbody, nv) = _geo(waypoints, com, cdof)
    unit, gout = _f(unit), _f(gout)
    off, es, et, ea, eb = entries
    nmuscle = len(off) - 1
    out = np.zeros((nworld, nmuscle), np.float32)
    s = [_i(a) for a in seg]
    keep = [_i(off), _i(es), _i(et), _f(ea), _f(eb)]
    lib().orc_muscle_activation_grad(
        nworld, nwp, nbody, nv, nmuscle, gout.shape[1], _p(waypoints), _p(com), _p(cdof), *[_p(a) for a in s],
        *[_p(a) for a in keep], _p(unit), _p(gout), int(root), _p(out),
    )  # fmt: skip
    return out


def muscle_sparse_moment(waypoints, com, cdof, seg, entry_torque, offsets, segment, start_coeff, end_coeff, root):
    waypoints, com, cdof, (nworld, nwp, nbody, nv) = _geo(waypoints, com, cdof)
    nentry = len(entry_torque)
    out = np.zeros((nworld, nentry), np.float32)
    s = [_i(a) for a in seg]
    keep = [_i(entry_torque), _i(offsets), _i(segment), _f(start_coeff), _f(end_coeff)]
    lib().orc_muscle_sparse_moment(
        nworld, nwp, nbody, nv, nentry, _p(waypoints), _p(com), _p(cdof), *[_p(a) for a in s],
        *[_p(a) for a in keep], int(root), _p(out),
    )  # fmt: skip
    return out


# ---------------------------------------------------------------- per-iteration factor stage
# Pinning (tests/test_newton_stages.py): the updated H against a fresh fp64 assembly with the
# new states; the dof union against a NumPy any() over the changed rows; the solve against
# fp64 `numpy.linalg.solve` within conditioning; the stored augmented factor against
# U'U == [[H, g], [g', 1e30]] in fp64; solve-only equals refactor-with-no-change to
# rounding.  Tile arithmetic and the order of the two sums on the dense path are this
# oracle's own conventions (Warp tile library / mujoco_warp block_cholesky are third party):
# bit-level parity with the reference UNPINNED there, tolerance parity pinned.

UPDATE_TABLES = TABLE_ORDER + ("SH_PAIR", "SH_FL", "SH_FR", "SH_RS", "SH_RKP", "SH_RK")


def sparse_update_factor(plan, state_changes, changes, ids, J, D, state, grad, hfactor, done=None, quad=1):
    J, D, grad = _f(J), _f(D), _f(grad)
    state, ids, changes, state_changes = _i(state), _i(ids), _i(changes), _i(state_changes)
    nworld, njmax, nv = J.shape
    tabs = [np.ascontiguousarray(plan.tables[k], np.int32) for k in UPDATE_TABLES]
    ptrs = (ctypes.c_void_p * len(tabs))(*[t.ctypes.data for t in tabs])
    hf = np.array(hfactor, np.float32, order="C")
    uni = np.zeros((nworld, nv + 1), np.int32)
    search = np.zeros((nworld, nv), np.float32)
    sdot, decr = np.zeros(nworld, np.float32), np.zeros(nworld, np.float32)
    dn = None if done is None else np.ascontiguousarray(done, np.uint8)
    status = lib().orc_sparse_update_factor(
        plan.nv, plan.nv_pad, plan.block, plan.nslots, plan.levels, ptrs, nworld, _p(dn), _p(state_changes),
        _p(changes), _p(ids), ids.shape[1], _p(J), njmax, _p(D), _p(state), quad, _p(grad), grad.shape[1], _p(hf),
        _p(uni), _p(search), _p(sdot), _p(decr),
    )  # fmt: skip
    assert status == 0
    return hf, uni, search, sdot, decr


def sparse_dense_factor(plan, grad, H, hfactor, quad_changed=None, state_changed=None, skip_unchanged=False,
                        skip_noflip=False, done=None):
    """Factor step of the upstream iteration on a plan of path "nonfused": lane-by-lane fp32
    restatement of sparse_hessian.py:639-679 (modes 4 / 5) under the dispatch of :849-894."""
    grad, H = _f(grad), _f(H)
    nworld, nv = grad.shape[0], plan.nv
    tabs = [np.ascontiguousarray(plan.tables[k], np.int32) for k in UPDATE_TABLES + ("SH_GAT",)]
    ptrs = (ctypes.c_void_p * len(tabs))(*[t.ctypes.data for t in tabs])
    hf = np.array(hfactor, np.float32, order="C")
    assert H.shape == (nworld, plan.nv_pad, plan.nv_pad) and hf.shape == H.shape
    search = np.zeros((nworld, nv), np.float32)
    sdot, decr = np.zeros(nworld, np.float32), np.zeros(nworld, np.float32)
    dn = None if done is None else np.ascontiguousarray(done, np.uint8)
    qc = None if quad_changed is None else _i(quad_changed)
    sc = None if state_changed is None else _i(state_changed)
    status = lib().orc_sparse_dense_factor(
        plan.nv, plan.nv_pad, plan.block, plan.nslots, plan.levels, ptrs, nworld, _p(dn), _p(grad), grad.shape[1], _p(H),
        _p(qc), _p(sc), int(skip_unchanged), int(skip_noflip), _p(hf), _p(search), _p(sdot), _p(decr),
    )  # fmt: skip
    assert status == 0
    return hf, search, sdot, decr


def dense_update_factor(state_changes, changes, ids, J, D, state, grad, H, U, done=None, quad=1):
    J, D, grad = _f(J), _f(D), _f(grad)
    state, ids, changes, state_changes = _i(state), _i(ids), _i(changes), _i(state_changes)
    nworld, njmax, nv = J.shape
    H, U = np.array(H, np.float32, order="C"), np.array(U, np.float32, order="C")
    pad = H.shape[1]
    uni = np.zeros((nworld, nv + 1), np.int32)
    search = np.zeros((nworld, nv), np.float32)
    sdot, decr = np.zeros(nworld, np.float32), np.zeros(nworld, np.float32)
    dn = None if done is None else np.ascontiguousarray(done, np.uint8)
    status = lib().orc_dense_update_factor(
        nworld, nv, pad, _p(dn), _p(state_changes), _p(changes), _p(ids), ids.shape[1], _p(J), njmax, _p(D),
        _p(state), quad, _p(grad), grad.shape[1], _p(H), _p(U), _p(uni), _p(search), _p(sdot), _p(decr),
    )  # fmt: skip
    assert status == 0
    return H, U, uni, search, sdot, decr


def muscle_torque_bounds(waypoints, com, cdof, seg, entries, unit, root):
    """Pinned by tests/test_muscle_dynamics.py: lower / upper = the negative / positive
    parts of the dense fp64 moment matrix times the unit forces, summed over muscles."""
    waypoints, com, cdof, (nworld, nwp, nbody, nv) = _geo(waypoints, com, cdof)
    unit = _f(unit)
    off, es, em, ea, eb = entries
    ntorque = len(off) - 1
    lower = np.zeros((nworld, ntorque), np.float32)
    upper = np.zeros((nworld, ntorque), np.float32)
    s = [_i(a) for a in seg]
    keep = [_i(off), _i(es), _i(em), _f(ea), _f(eb)]
    lib().orc_muscle_torque_bounds(
        nworld, nwp, nbody, nv, unit.shape[1], ntorque, _p(waypoints), _p(com), _p(cdof), *[_p(a) for a in s],
        *[_p(a) for a in keep], _p(unit), int(root), _p(lower), _p(upper),
    )  # fmt: skip
    return lower, upper


# ---- steps either side of the solve that walk a world's small trees -------------------------
# Pinning: `mul_m_sparse` against the dense fp64 product with the symmetric matrix of the CSR
# and by linearity; `tree_accumulate` against subtree sums taken from the ancestor relation in
# fp64 (and exactly, on integer-valued inputs, where every order of additions gives the same
# bits); `project_body_wrenches` against the masked sum of the reference's legacy kernel
# (muscle_dynamics_kernels.py:2906-2955) in fp64.  Bit-level agreement with the reference build
# is unpinned for all three: the first one's term order comes from upstream tables that are not
# in the tree, the other two add siblings with atomics in the reference's default kernels.


def mul_m_sparse(M, vec, rowadr, col, madr, skip=None, out=None):
    M, vec = _f(M), _f(vec)
    nworld, nM = M.shape
    nv = vec.shape[1]
    out = np.zeros((nworld, nv), np.float32) if out is None else out
    sk = None if skip is None else np.ascontiguousarray(skip, np.uint8)
    lib().orc_mul_m_sparse(nworld, nv, nM, _p(_i(rowadr)), _p(_i(col)), _p(_i(madr)), _p(M), _p(vec),
                           None if sk is None else _p(sk), _p(out))  # fmt: skip
    return out


def tree_accumulate(values, components, parent, bodies, offsets, skip_root_parent=False):
    """Returns the accumulated copy of values (nworld, nbody, components)."""
    out = _f(values).copy()
    nworld, nbody = out.shape[0], out.shape[1]
    lib().orc_tree_accumulate(nworld, nbody, components, _p(_i(parent)), _p(_i(bodies)), _p(_i(offsets)),
                              len(offsets) - 1, int(bool(skip_root_parent)), _p(out))  # fmt: skip
    return out


def project_body_wrenches(body_force, body_torque, xipos, subtree_com, cdof, rootid, dof_body, parent, bodies, offsets,
                          root, ntorque, out_offset=0, mean=None):  # fmt: skip
    body_force, body_torque, xipos, subtree_com, cdof = (_f(a) for a in (body_force, body_torque, xipos, subtree_com, cdof))
    nworld, nbody, nvfull = body_force.shape[0], body_force.shape[1], cdof.shape[1]
    mean = np.zeros((nworld, ntorque + out_offset), np.float32) if mean is None else mean
    lib().orc_project_body_wrenches(
        nworld, nbody, nvfull, _p(body_force), _p(body_torque), _p(xipos), _p(subtree_com), _p(cdof), _p(_i(rootid)),
        _p(_i(dof_body)), _p(_i(parent)), _p(_i(bodies)), _p(_i(offsets)), len(offsets) - 1, root, ntorque, out_offset,
        mean.shape[1], _p(mean),
    )  # fmt: skip
    return mean


# `newton_gradient`: pinned by the fp64 product J' f and grad = Ma - qfrc_smooth - J' f, by
# grad_dot against the fp64 dot product, and by the closed form of the rescaling branch; the
# order in which a block adds its lanes' partial sums is unpinned (Warp's tile_sum).
def newton_gradient(J, force, smooth, Ma, changed, alpha, grad_dot, decrement, scale, nefc=None, done=None, block=64):
    """Returns (qfrc_constraint, grad, grad_dot, decrement, scale, search_unchanged); the three
    per-world scalars start from the arrays passed in (copied)."""
    J, force, smooth, Ma, alpha = (_f(a) for a in (J, force, smooth, Ma, alpha))
    nworld, njmax, nv = J.shape
    qc, grad = np.zeros((nworld, nv), np.float32), np.zeros((nworld, nv), np.float32)
    gd, de, sc = (_f(a).copy() for a in (grad_dot, decrement, scale))
    un = np.zeros(nworld, np.uint8)
    dn = None if done is None else np.ascontiguousarray(done, np.uint8)
    lib().orc_newton_gradient(
        nworld, nv, njmax, block, None if nefc is None else _p(_i(nefc)), _p(J), _p(force), _p(smooth), _p(Ma),
        _p(_i(changed)), _p(alpha), None if dn is None else _p(dn), _p(qc), _p(grad), _p(gd), _p(de), _p(sc), _p(un),
    )  # fmt: skip
    return qc, grad, gd, de, sc, un


# `newton_jv`: pinned by the fp64 product J v; the chunking rule above 50 dofs is the
# reference's own statement and is exercised on both sides of the threshold.
def newton_jv(J, search, nefc=None, skip=None, out=None):
    J, search = _f(J), _f(search)
    nworld, njmax, nv = J.shape
    out = np.zeros((nworld, njmax), np.float32) if out is None else out
    sk = None if skip is None else np.ascontiguousarray(skip, np.uint8)
    lib().orc_newton_jv(nworld, nv, njmax, None if nefc is None else _p(_i(nefc)), _p(J), _p(search),
                        None if sk is None else _p(sk), _p(out))  # fmt: skip
    return out


def newton_init_jaref(J, qacc, aref, nefc=None):
    """Jaref = J qacc - aref: the row sums of `newton_jv`, then one float32 subtraction (rows at
    or past nefc stay zero).  Pinned by the fp64 product."""
    jv = newton_jv(J, qacc, nefc=nefc)
    njmax = jv.shape[1]
    ne = np.full(len(jv), njmax) if nefc is None else np.minimum(np.asarray(nefc), njmax)
    rows = np.arange(njmax)[None, :] < ne[:, None]
    return np.where(rows, jv - _f(aref), np.float32(0.0)).astype(np.float32)


def newton_search_sums(grad, search, block=32, skip=None, sdot=None, decr=None):
    """(search_dot, decrement) of the tree stage; skipped worlds keep what was passed in.  Pinned
    by the fp64 dot products and, where every lane holds one dof, by the tree's association."""
    grad, search = _f(grad), _f(search)
    nworld, nv = search.shape
    sdot = np.zeros(nworld, np.float32) if sdot is None else _f(sdot).copy()
    decr = np.zeros(nworld, np.float32) if decr is None else _f(decr).copy()
    sk = None if skip is None else np.ascontiguousarray(skip, np.uint8)
    lib().orc_newton_search_sums(nworld, nv, block, None if sk is None else _p(sk), _p(grad), grad.shape[1], _p(search),
                                 nv, _p(sdot), _p(decr))  # fmt: skip
    return sdot, decr


def newton_tree_stage(rowadr, rownnz, colind, plan, M, J, D, state, nefc, grad, skip, search, sdot, decr, block=32, quad=1):
    """The tree factor stage: for the worlds that are not skipped search = -(M + J' D_act J)^-1 grad
    by the fused assembly + tree L'DL, and the two dot products.  Returns (search, search_dot,
    decrement) with the skipped worlds' entries as passed in."""
    nv = len(rowadr)
    x = assemble_tree_ldl_solve(rowadr, rownnz, colind, plan, M, J, D, state, nefc, _f(grad)[:, :nv], quad=quad)
    run = np.ones(len(x), bool) if skip is None else np.asarray(skip) == 0
    new = np.where(run[:, None], -x, _f(search)).astype(np.float32)
    sd, de = newton_search_sums(_f(grad)[:, :nv], new, block=block, skip=skip, sdot=sdot, decr=decr)
    return new, sd, de


# The step along the search direction and the listing of changed rows
# (src/instantmimic/utils/mjw_kernels/newton_stages.py:373-381, 403-426), in NumPy.  `advance`
# is pinned by its closed form in fp64 and, bit for bit, by an exact-product-one-rounding sum;
# `changed_rows` is integer work, pinned by brute force over the rows.
def newton_advance(alpha, search, mv, jv, qacc, Ma, jaref, nefc=None, done=None):
    """Returns the advanced copies (qacc, Ma, jaref)."""
    a = _f(alpha)[:, None]
    live = np.ones(len(a), bool) if done is None else np.asarray(done) == 0
    q64 = (np.float64(a) * _f(search).astype(np.float64) + _f(qacc)).astype(np.float32)  # one rounding: a fused multiply-add
    m64 = (np.float64(a) * _f(mv).astype(np.float64) + _f(Ma)).astype(np.float32)
    njmax = jv.shape[1]
    ne = np.full(len(a), njmax) if nefc is None else np.minimum(np.asarray(nefc), njmax)
    rows = np.arange(njmax)[None, :] < ne[:, None]
    j2 = _f(jaref) + (a * _f(jv))  # float32 product, then float32 sum
    sel = live[:, None]
    return np.where(sel, q64, qacc), np.where(sel, m64, Ma), np.where(sel & rows, j2, jaref)


def newton_changed_rows(old_state, new_state, quad=1, nefc=None, done=None, ids=None, quad_count=None, state_count=None):
    old_state, new_state = np.asarray(old_state), np.asarray(new_state)
    nworld, njmax = old_state.shape
    ids = np.zeros((nworld, njmax), np.int32) if ids is None else ids.copy()
    qc = np.zeros(nworld, np.int32) if quad_count is None else quad_count.copy()
    sc = np.zeros(nworld, np.int32) if state_count is None else state_count.copy()
    for w in range(nworld):
        if done is not None and done[w]:
            continue
        ne = njmax if nefc is None else min(int(nefc[w]), njmax)
        flips = [r for r in range(ne) if (old_state[w, r] == quad) != (new_state[w, r] == quad)]
        ids[w, : len(flips)] = flips
        qc[w] = len(flips)
        sc[w] = int(np.count_nonzero(old_state[w, :ne] != new_state[w, :ne]))
    return ids, qc, sc


# The convergence test of an iteration (src/instantmimic/utils/mjw_kernels/newton_fusion.py:265-296)
# in NumPy float32; pinned by worlds built to meet exactly one criterion each.
def newton_converged(alpha, improvement, grad_dot, decrement, tolerance, meaninertia, nv, maxiter, niter, done, overflow_bit=0):
    """Returns (niter, done, overflow, newly_done_count)."""
    nworld = len(alpha)
    niter, done = np.asarray(niter, np.int32).copy(), np.asarray(done, np.uint8).copy()
    overflow = np.zeros(nworld, np.int32)
    w = np.arange(nworld)
    tol = _f(tolerance)[w % len(tolerance)]
    scale = _f(meaninertia)[w % len(meaninertia)] * np.float32(nv)
    a, imp, gd, de = (_f(x) for x in (alpha, improvement, grad_dot, decrement))
    with np.errstate(invalid="ignore", divide="ignore"):
        conv = (a == 0) | ((imp > 0) & (imp / scale < tol)) | (np.sqrt(gd) / scale < tol) | (np.float32(0.5) * de / scale < tol)
    live = done == 0
    niter[live] += 1
    stop = live & (conv | (niter == maxiter))
    overflow[stop & ~conv] = overflow_bit
    done[stop] = 1
    return niter, done, overflow, int(stop.sum())


# The scalar line search and the constraint re-evaluation of the line-search stage
# (newton_stages.py:179-444).  The stage's flow is the reference's; the per-row cost model is
# upstream's and restated from MuJoCo's primal line search: parity with upstream's bits is
# UNPINNED.  Pinned by tests/test_newton_linesearch.py: against the exact minimiser of the line's
# cost in fp64 (slope at alpha within the stage's tolerance, cost decrease equal to the reported
# improvement), by the closed form without one-sided rows (alpha = -p'(0) / p''(0)), and the
# states / forces by brute force from their definitions.
def newton_linesearch(tolerance, ls_tolerance, meaninertia, ne, nf, nefc, smooth, D, frictionloss, Jaref, search, search_dot,
                      mv, jv, Ma, done=None, ls_iterations=50, overflow_bit=4):  # fmt: skip
    """Returns (alpha, improvement, ls_exhausted, overflow)."""
    smooth, D, Jaref, search, search_dot, mv, jv, Ma = (_f(a) for a in (smooth, D, Jaref, search, search_dot, mv, jv, Ma))
    nworld, nv = search.shape
    njmax = D.shape[1]
    alpha, imp = np.zeros(nworld, np.float32), np.zeros(nworld, np.float32)
    ex, ov = np.zeros(nworld, np.uint8), np.zeros(nworld, np.int32)
    tol, lst, mi = _f(tolerance), _f(ls_tolerance), _f(meaninertia)
    fl = None if frictionloss is None else _f(frictionloss)
    dn = None if done is None else np.ascontiguousarray(done, np.uint8)
    opt = lambda a: None if a is None else _p(_i(a))  # noqa: E731
    status = lib().orc_newton_linesearch(
        nworld, nv, njmax, _p(tol), len(tol), _p(lst), len(lst), _p(mi), len(mi), opt(ne), opt(nf), opt(nefc), _p(smooth), _p(D),
        _p(fl), _p(Jaref), _p(search), _p(search_dot), _p(mv), _p(jv), _p(Ma), _p(dn), int(ls_iterations), int(overflow_bit),
        _p(alpha), _p(imp), _p(ex), _p(ov),
    )  # fmt: skip
    assert status == 0
    return alpha, imp, ex, ov


def newton_eval_constraints(Jaref, D, frictionloss, ne, nf, nefc, state, done=None, exhausted=None):
    """Returns (force, new state, ids, quad_changed_count, state_changed_count)."""
    Jaref, D = _f(Jaref), _f(D)
    nworld, njmax = D.shape
    force = np.zeros((nworld, njmax), np.float32)
    st = np.array(state, np.int32, order="C")
    ids = np.zeros((nworld, njmax), np.int32)
    qc, sc = np.zeros(nworld, np.int32), np.zeros(nworld, np.int32)
    fl = None if frictionloss is None else _f(frictionloss)
    dn = None if done is None else np.ascontiguousarray(done, np.uint8)
    ex = None if exhausted is None else np.ascontiguousarray(exhausted, np.uint8)
    opt = lambda a: None if a is None else _p(_i(a))  # noqa: E731
    status = lib().orc_newton_eval_constraints(nworld, njmax, _p(Jaref), _p(D), _p(fl), opt(ne), opt(nf), opt(nefc), _p(dn), _p(ex),
                                               _p(force), _p(st), _p(ids), njmax, _p(qc), _p(sc))  # fmt: skip
    assert status == 0
    return force, st, ids, qc, sc


# ---------------------------------------------------------------- implicit-fast integrator matrix
# Pinned by tests/test_implicit_qh.py against the dense fp64 statement
# qH = M + h diag(b) - h A' diag(g) A + h Jt' diag(bt) Jt on M's pattern with free-body rows reset to M.
# Upstream's kernels are absent from the reference tree: bit-level parity with them is UNPINNED.


def implicit_qh_base(M, elem_dof, damping, timestep):
    M, damping = _f(M), _f(damping)
    elem_dof = _i(elem_dof)
    nworld, nM = M.shape
    out = np.zeros_like(M)
    ld = 0 if damping.ndim == 1 else damping.shape[1]
    assert lib().orc_implicit_qh_base(nworld, nM, _p(M), nM, _p(elem_dof), _p(damping), ld, ctypes.c_float(timestep), _p(out), nM) == 0
    return out


def polynomial_damping(base, poly, velocity):
    """``base + sum_k (k + 1) poly[..., k - 1] |velocity|^k`` per (world, item); ``base`` (n,) or
    (nworld, n), ``poly`` (n, K) or (nworld, n, K).  Pinned by tests/test_implicit_qh.py: the
    central difference of the damper's force in fp64, and K = 0 returning ``base``."""
    base, poly, velocity = _f(base), _f(poly), _f(velocity)
    nworld, n = velocity.shape
    nterm = poly.shape[-1]
    out = np.zeros_like(velocity)
    L = ctypes.c_long
    assert lib().orc_polynomial_damping(nworld, n, nterm, _p(base), L(0 if base.ndim == 1 else n), _p(poly),
                                        L(0 if poly.ndim == 2 else n * nterm), _p(velocity), L(n), _p(out), L(n)) == 0  # fmt: skip
    return out


def actuator_velocity_gain(gaintype, biastype, gainprm, biasprm, inp, forcelimited=None, forcerange=None, force=None):
    gainprm, biasprm, inp = _f(gainprm), _f(biasprm), _f(inp)
    gaintype, biastype = _i(gaintype), _i(biastype)
    nworld, nu = inp.shape
    out = np.zeros_like(inp)
    fl = None if forcelimited is None else np.ascontiguousarray(forcelimited, np.uint8)
    fr = None if forcerange is None else _f(forcerange)
    fo = None if force is None else _f(force)
    assert lib().orc_actuator_velocity_gain(nworld, nu, _p(gaintype), _p(biastype), _p(gainprm), _p(biasprm), gainprm.shape[1],
                                            _p(fl), _p(fr), _p(inp), _p(fo), _p(out)) == 0  # fmt: skip
    return out
