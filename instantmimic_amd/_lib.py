"""ctypes binding of ``libimhip.so`` (the C ABI declared in ``include/imhip.h``).

The library must have been built (``python -m instantmimic_amd.build`` or
``__graft_entry__.build()``); there is no fallback path when it is missing.
"""

from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libimhip.so")

IM_OK = 0
IM_ERR_ARG = 1
IM_ERR_STRUCTURE = 2
IM_ERR_UNSUPPORTED = 3
IM_ERR_HIP = 4
IM_ERR_STRIDE = 5
IM_ERR_SCRATCH = 6
IM_FLAG_NEGATE = 1


class TreePlanInfo(C.Structure):
    _fields_ = [
        (name, C.c_int32)
        for name in (
            "nv", "nM", "ngroups", "ntrunk", "span", "dense_cost", "shared_bytes", "beats_dense", "max_depth",
            "device_ready",
        )
    ]  # fmt: skip


_vp, _i, _i64, _u = C.c_void_p, C.c_int, C.c_int64, C.c_uint


class SparsePlanInfo(C.Structure):
    _fields_ = [
        ("nv", C.c_int32), ("nv_pad", C.c_int32), ("block", C.c_int32), ("path", C.c_int32),
        ("nslots", C.c_int32), ("nfac", C.c_int32), ("nterms", C.c_int32), ("nlevels", C.c_int32),
        ("device_ready", C.c_int32), ("density", C.c_double),
    ]  # fmt: skip


# order of the IM_SH_* table ids of imhip.h
SPARSE_TABLES = ("SH_LP", "SH_LT", "SH_ES", "SH_EC", "SH_RP", "SH_RAB", "SH_RKL", "SH_ORIG", "SH_BL", "SH_BS",
                 "SH_BI", "SH_BJ", "SH_PM", "SH_SA", "SH_SB", "SH_SM", "SH_PAIR", "SH_FL", "SH_FR", "SH_RS",
                 "SH_RKP", "SH_RK", "SH_GAT")  # fmt: skip


class MuscleForceModel(C.Structure):
    _fields_ = [
        ("force_scale", C.c_float),
        ("length_norm_min", C.c_float),
        ("length_norm_max", C.c_float),
        ("active", C.c_float * 3),
        ("passive", C.c_float * 3),
        ("include_passive", C.c_int32),
    ]


class MuscleForceVelocityModel(C.Structure):
    _fields_ = [("vmax", C.c_float), ("fvmax", C.c_float), ("clamp_activation", C.c_float), ("include_active", C.c_float)]


class NewtonArgs(C.Structure):
    """im_newton_args"""

    _fields_ = [
        ("opt_tolerance", C.c_void_p), ("opt_ls_tolerance", C.c_void_p), ("stat_meaninertia", C.c_void_p),
        ("ntolerance", C.c_int32), ("nls_tolerance", C.c_int32), ("nmeaninertia", C.c_int32),
        ("ls_iterations", C.c_int32), ("iterations", C.c_int32), ("block", C.c_int32), ("quad", C.c_int32),
        ("ls_overflow_bit", C.c_int32), ("iterations_overflow_bit", C.c_int32),
        ("M_mulm_rowadr", C.c_void_p), ("M_mulm_col", C.c_void_p), ("M_mulm_madr", C.c_void_p), ("nterm", C.c_int32),
        ("ne", C.c_void_p), ("nf", C.c_void_p), ("nefc", C.c_void_p),
        ("M", C.c_void_p), ("ldM", C.c_int64), ("efc_J", C.c_void_p), ("njmax", C.c_int32),
        ("efc_D", C.c_void_p), ("efc_frictionloss", C.c_void_p), ("qfrc_smooth", C.c_void_p),
        ("qacc", C.c_void_p), ("efc_Ma", C.c_void_p), ("efc_force", C.c_void_p), ("efc_state", C.c_void_p),
        ("Jaref", C.c_void_p), ("search", C.c_void_p), ("search_dot", C.c_void_p), ("mv", C.c_void_p), ("jv", C.c_void_p),
        ("alpha", C.c_void_p), ("improvement", C.c_void_p), ("grad", C.c_void_p), ("ld_grad", C.c_int64),
        ("grad_dot", C.c_void_p), ("grad_scale", C.c_void_p), ("newton_decrement", C.c_void_p),
        ("qfrc_constraint", C.c_void_p), ("quad_changed_ids", C.c_void_p), ("ld_ids", C.c_int32),
        ("quad_changed_count", C.c_void_p), ("state_changed_count", C.c_void_p), ("solver_niter", C.c_void_p),
        ("overflow", C.c_void_p), ("nsolving", C.c_void_p),
        ("done", C.c_void_p), ("ls_exhausted", C.c_void_p), ("search_unchanged", C.c_void_p), ("nworld", C.c_int32),
    ]  # fmt: skip


class RowPairTerm(C.Structure):
    """im_row_pair_term"""

    _fields_ = [
        ("values", C.c_void_p), ("ld_values", C.c_int64), ("entry_source", C.c_void_p), ("entry_row", C.c_void_p),
        ("nentry", C.c_int32), ("elem_ids", C.c_void_p), ("nelem", C.c_int32), ("chunk_offsets", C.c_void_p),
        ("chunk_pairs", C.c_void_p), ("chunk_count", C.c_int32), ("weight", C.c_void_p), ("ld_weight", C.c_int64),
        ("scale", C.c_float),
    ]  # fmt: skip


class MuscleGeometry(C.Structure):
    _fields_ = [
        ("waypoints", _vp), ("ld_waypoints", _i64),
        ("subtree_com", _vp), ("ld_subtree_com", _i64),
        ("cdof", _vp), ("ld_cdof", _i64),
    ]  # fmt: skip


class MuscleSegments(C.Structure):
    _fields_ = [
        ("start_waypoint", _vp), ("end_waypoint", _vp), ("start_root_body", _vp), ("end_root_body", _vp),
        ("nsegment", C.c_int32),
    ]  # fmt: skip


class MuscleEntries(C.Structure):
    _fields_ = [
        ("offsets", _vp), ("segment", _vp), ("other", _vp), ("start_coeff", _vp), ("end_coeff", _vp),
        ("nrow", C.c_int32), ("nentry", C.c_int32), ("nother", C.c_int32),
    ]  # fmt: skip


class BodyWrenches(C.Structure):
    _fields_ = [
        ("body_force", _vp), ("body_torque", _vp), ("xipos", _vp), ("subtree_com", _vp), ("cdof", _vp),
        ("ld_body_force", C.c_int64), ("ld_body_torque", C.c_int64), ("ld_xipos", C.c_int64),
        ("ld_subtree_com", C.c_int64), ("ld_cdof", C.c_int64), ("body_rootid", _vp),
    ]  # fmt: skip


class WrenchTopology(C.Structure):
    _fields_ = [
        ("dof_bodyid", _vp), ("body_parentid", _vp), ("level_bodies", _vp), ("level_offsets", _vp),
        ("levels", C.c_int32), ("body_count", C.c_int32),
    ]  # fmt: skip


_pgeo, _pseg, _pent = C.POINTER(MuscleGeometry), C.POINTER(MuscleSegments), C.POINTER(MuscleEntries)

# name -> (restype, argtypes); the single list of symbols the header declares
SIGNATURES = {
    "im_version": (_i, []),
    "im_status_string": (C.c_char_p, [_i]),
    "im_last_hip_error": (_i, []),
    "im_tree_structure_check": (_i, [_i, _vp, _vp, _vp, _i]),
    "im_tree_plan_create": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, C.POINTER(_vp)]),
    "im_tree_plan_destroy": (None, [_vp]),
    "im_tree_plan_get_info": (_i, [_vp, C.POINTER(TreePlanInfo)]),
    "im_tree_plan_get_arrays": (_i, [_vp, _vp, _vp, _vp, _vp]),
    "im_tree_factor_solve": (_i, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _i, _vp]),
    "im_assemble_tree_ldl_solve": (
        _i,
        [_vp, _vp, _i64, _vp, _i, _vp, _vp, _vp, _i, _vp, _i64, _vp, _i64, _vp, _i, _u, _vp],
    ),
    "im_assemble_tree_ldl_solve_iters": (
        _i,
        [_vp, _vp, _i64, _vp, _i, _vp, _vp, _i64, _vp, _i, _vp, _i64, _i64, _vp, _i64, _i64, _i, _i, _u, _vp],
    ),
    "im_tree_pattern_violations": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _i, _vp, _i, _vp]),
    "im_check_reciprocal": (_i, [C.c_uint32, C.c_uint32, _vp, _vp]),
    "im_dof_pattern_create": (_i, [_i, _vp, _i, _vp, _vp, _vp, C.POINTER(_vp)]),
    "im_dof_pattern_destroy": (None, [_vp]),
    "im_dof_pattern_couple_bodies": (_i, [_vp, _vp, _i]),
    "im_dof_pattern_couple_dofs": (_i, [_vp, _vp, _i]),
    "im_dof_pattern_get": (_i, [_vp, _vp]),
    "im_sparse_plan_build": (_i, [_vp, _i, _i, _i, _vp, _vp, _i, _i, C.POINTER(_i), C.POINTER(_vp)]),
    "im_sparse_plan_get_info": (_i, [_vp, C.POINTER(SparsePlanInfo)]),
    "im_sparse_plan_table_size": (_i, [_vp, _i]),
    "im_sparse_plan_get_table": (_i, [_vp, _i, _vp, _i]),
    "im_sparse_plan_get_structure": (_i, [_vp, _vp, _vp, _vp]),
    "im_sparse_plan_destroy": (None, [_vp]),
    "im_sparse_init_factor": (
        _i,
        [_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp],
    ),
    "im_sparse_update_factor": (
        _i,
        [_vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp],
    ),
    "im_sparse_dense_factor": (_i, [_vp, _vp, _vp, _i, _vp, _i64, _vp, _vp, _i, _i, _vp, _vp, _i, _vp, _vp, _i, _vp]),
    "im_implicit_qh_base": (_i, [_vp, _i64, _i, _vp, _vp, _i64, C.c_float, _vp, _i64, _i, _vp]),
    "im_actuator_velocity_gain": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _i, _i, _vp]),
    "im_implicit_qh": (
        _i,
        [_vp, _i64, _i, _vp, _vp, _i64, C.c_float, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _i,
         C.POINTER(RowPairTerm), C.POINTER(RowPairTerm), _vp, _i64, _i, _vp],
    ),  # fmt: skip
    "im_newton_linesearch": (
        _i,
        [_vp, _i, _vp, _i, _vp, _i, _vp, _vp, _vp, _i, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _i64,
         _vp, _i64, _vp, _i64, _vp, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _vp],
    ),  # fmt: skip
    "im_newton_eval_constraints": (
        _i,
        [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i, _vp, _vp, _i, _vp],
    ),
    "im_check_pivot_sqrt": (_i, [_u, _u, _vp, _vp]),
    "im_jtdj_factor_solve": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _i, _vp, _i, _i, _vp, _i64, _vp, _i, _vp, _i64, _i, _vp]),
    "im_tree_plan_kernel_key": (_i, [_vp, _vp, _vp]),
    "im_tree_plan_attach_kernels": (_i, [_vp, _vp]),
    "im_dense_update_factor": (
        _i,
        [_vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _i, _vp, _i64, _vp, _vp, _i, _i, _vp, _vp, _i64, _vp, _vp, _i, _vp],
    ),
    "im_dense_update_column": (
        _i,
        [_vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _i, _vp, _i64, _vp, _vp, _i, _i, _vp, _vp, _i64, _vp, _vp, _i, _vp],
    ),
    "im_dense_init_factor": (
        _i,
        [_vp, _vp, _vp, _i, _vp, _vp, _i, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _i, _i, _vp, _vp, _i64, _vp, _vp, _i, _vp],
    ),
    "im_dense_init_tile": (
        _i,
        [_vp, _vp, _vp, _i, _vp, _vp, _i, _vp, _i64, _vp, _vp, _i64, _vp, _i, _i, _vp, _vp, _i64, _vp, _vp, _i, _vp],
    ),
    "im_newton_init_context": (_i, [C.POINTER(NewtonArgs), _vp, _i64, _vp, _i64, _i, _i, _vp]),
    "im_polynomial_damping": (_i, [_vp, _i64, _vp, _i64, _i, _vp, _i64, _vp, _i64, _i, _i, _vp]),
    "im_dense_update_tile": (
        _i,
        [_vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _i, _vp, _i64, _vp, _i, _i, _vp, _vp, _i64, _vp, _vp, _i, _vp],
    ),
    "im_tile_cholesky_solve": (_i, [_vp, _i64, _i64, _vp, _i, _i, _vp, _i64, _vp, _i64, _i, _vp]),
    "im_tile_cholesky_solve_m": (_i, [_vp, _i64, _i, _vp, _vp, _i, _i, _vp, _i64, _vp, _i64, _i, _vp]),
    "im_blocked_factor_solve": (_i, [_vp, _i64, _i, _vp, _i, _i, _i, _vp, _i64, _vp, _vp, _i64, _i, _vp]),
    "im_blocked_index_layout": (_i, [_vp, _i, _i, _i, _vp, _vp]),
    "im_blocked_multi_solve": (_i, [_vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _vp]),
    "im_blocked_factor_multi_solve": (_i, [_vp, _i64, _i, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _vp, _i, _vp]),
    "im_blocked_factor_multi_solve_static": (_i, [_vp, _i64, _i, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _vp]),
    "im_copy_dense_factor": (_i, [_vp, _i, _vp, _i, _vp, _i64, _i, _vp]),
    "im_jtdj_mfma": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _vp]),
    "im_muscle_project": (_i, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i64, _i, _vp]),
    "im_muscle_gather_tables": (_i, [_vp, _vp, _vp, _i, _i, _vp, _vp, _vp, C.POINTER(_i), C.POINTER(_i)]),
    "im_muscle_implicit_gather": (
        _i,
        [_vp, _i64, _vp, _i64, _vp, _i, _vp, _i, _vp, _vp, _i, C.c_float, _vp, _i64, _i, _vp],
    ),
    "im_muscle_waypoints": (_i, [_vp, _i64, _vp, _i64, _vp, _vp, _i, _vp, _i64, _i, _vp]),
    "im_muscle_force_magnitudes": (
        _i,
        [_vp, _i64, _vp, _vp, _vp, _i, _vp, C.POINTER(MuscleForceModel), _i, _vp, _i64, _vp, _i64, _i, _vp],
    ),
    "im_muscle_force_velocity_state": (
        _i,
        [_vp, _i64, _vp, _vp, _i, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _i, C.POINTER(MuscleForceModel),
         C.POINTER(MuscleForceVelocityModel), _i, _vp, _vp, _vp, _vp, _vp, _i64, _i, _vp],
    ),  # fmt: skip
    "im_muscle_waypoints_forces": (
        _i,
        [_vp, _i64, _vp, _i64, _vp, _vp, _i, _vp, _i64, _vp, _vp, _vp, _i, _vp, C.POINTER(MuscleForceModel), _i,
         _vp, _i64, _vp, _i64, _i, _vp],
    ),  # fmt: skip
    "im_muscle_torque_forward": (
        _i,
        [_pgeo, _pseg, _pent, _vp, _i64, _vp, _i64, _vp, _i64, _i, _vp, _i64, _i, _vp],
    ),
    "im_muscle_activation_grad": (_i, [_pgeo, _pseg, _pent, _vp, _i64, _vp, _i64, _i, _vp, _i64, _i, _vp]),
    "im_muscle_torque_bounds": (_i, [_pgeo, _pseg, _pent, _vp, _i64, _i, _vp, _vp, _i64, _i, _vp]),
    "im_muscle_sparse_moment": (_i, [_pgeo, _pseg, _vp, _pent, _i, _vp, _i64, _i, _vp]),
    "im_mul_m_sparse": (_i, [_vp, _i64, _i, _vp, _vp, _vp, _i, _vp, _i64, _vp, _vp, _i64, _i, _i, _vp]),
    "im_tree_accumulate": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp, _i64, _i, _i, _vp]),
    "im_newton_gradient": (
        _i,
        [_vp, _vp, _i, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i, _i,
         _i, _vp],
    ),  # fmt: skip
    "im_newton_jv": (_i, [_vp, _i, _vp, _vp, _i64, _vp, _vp, _i64, _i, _i, _vp]),
    "im_newton_init_jaref": (_i, [_vp, _i, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _i, _i, _vp]),
    "im_dense_from_csr": (_i, [_vp, _i64, _vp, _i, _i, _vp, _i, _vp]),
    "im_newton_tree_stage": (
        _i,
        [_vp, _vp, _vp, _i64, _vp, _i, _vp, _vp, _vp, _i, _vp, _i64, _vp, _i64, _vp, _vp, _i, _i, _vp],
    ),
    "im_newton_solve_tree": (_i, [_vp, C.POINTER(NewtonArgs), _vp]),
    "im_newton_solve_dense_tile": (_i, [C.POINTER(NewtonArgs), _vp, _vp, _i, _i, _i, _vp, _vp]),
    "im_newton_solve_dense_column": (_i, [C.POINTER(NewtonArgs), _vp, _vp, _vp, _i, _i, _i, _vp, _vp]),
    "im_newton_solve_sparse": (_i, [_vp, C.POINTER(NewtonArgs), _vp, _vp, _vp]),
    "im_newton_advance": (
        _i,
        [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _i, _i, _i, _vp],
    ),
    "im_newton_changed_rows": (_i, [_vp, _vp, _i, _vp, _i, _vp, _vp, _i, _vp, _vp, _i, _vp]),
    "im_newton_converged": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _vp]),
    "im_newton_init_empty_worlds": (_i, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i, _i, _vp]),
    "im_qfrc_constraint_from_grad": (_i, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _i64, _i, _i, _vp]),
    "im_project_body_wrenches": (
        _i,
        [C.POINTER(BodyWrenches), C.POINTER(WrenchTopology), _i, _i, _i, _vp, _i64, _i, _vp],
    ),
}

_lib = None


class ImhipError(RuntimeError):
    def __init__(self, status: int, where: str):
        self.status = status
        msg = lib().im_status_string(status).decode()
        if status == IM_ERR_HIP:
            msg += f" (hipError {lib().im_last_hip_error()})"
        super().__init__(f"{where}: {msg}")


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m instantmimic_amd.build` "
                "(there is no CPU fallback for the HIP kernels)"
            )
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status: int, where: str) -> None:
    if status != IM_OK:
        raise ImhipError(status, where)
