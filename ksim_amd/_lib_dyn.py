"""ctypes signatures of the model / control-step entry points (include/ksim_hip.h)."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_double, c_float, c_int32, c_int64, c_void_p

import numpy as np

MAXB, MAXQ, MAXV, MAXU, MAXS = 32, 40, 32, 32, 16
KS_ACT_TORQUE, KS_ACT_POSITION, KS_ACT_POSITION_VELOCITY = 0, 1, 2


class KsModelDesc(ctypes.Structure):
    _fields_ = [
        ("nb", c_int32), ("nq", c_int32), ("nv", c_int32), ("nu", c_int32), ("ns", c_int32),
        ("iterations", c_int32), ("ls_iterations", c_int32), ("eulerdamp", c_int32), ("condim", c_int32),
        ("dt", c_double), ("gravity", c_double * 3), ("tolerance", c_double), ("ls_tolerance", c_double),
        ("impratio", c_double), ("meaninertia", c_double), ("friction", c_double),
        ("solref", c_double * 2), ("solimp", c_double * 5),
        ("body_parent", c_int32 * MAXB), ("body_jtype", c_int32 * MAXB), ("body_qadr", c_int32 * MAXB),
        ("body_dofadr", c_int32 * MAXB), ("body_subtree_end", c_int32 * MAXB),
        ("body_pos", c_double * 3 * MAXB), ("body_quat", c_double * 4 * MAXB), ("body_mass", c_double * MAXB),
        ("body_ipos", c_double * 3 * MAXB), ("body_iquat", c_double * 4 * MAXB), ("body_inertia", c_double * 3 * MAXB),
        ("jnt_axis", c_double * 3 * MAXB), ("jnt_pos", c_double * 3 * MAXB), ("body_invweight0", c_double * MAXB),
        ("qpos0", c_double * MAXQ),
        ("dof_body", c_int32 * MAXV), ("dof_parent", c_int32 * MAXV), ("dof_damping", c_double * MAXV),
        ("dof_armature", c_double * MAXV),
        ("act_dof", c_int32 * MAXU), ("act_gear", c_double * MAXU), ("act_lo", c_double * MAXU),
        ("act_hi", c_double * MAXU),
        ("sph_body", c_int32 * MAXS), ("sph_pos", c_double * 3 * MAXS), ("sph_radius", c_double * MAXS),
        ("jnt_limited", c_int32 * MAXB), ("jnt_range", c_double * 2 * MAXB), ("dof_invweight0", c_double * MAXV),
        ("dof_frictionloss", c_double * MAXV), ("dof_solref", c_double * 2), ("dof_solimp", c_double * 5),
        ("dof_stiffness", c_double * MAXV),
    ]


from . import _lib_terms as _T  # noqa: E402  (event and random-number structs)

_P = c_void_p
STEP_IO_POINTERS = (
    "qpos", "qvel", "qacc_warmstart", "time", "last_ctrl",
    "action", "ctrl_in", "latency", "zero_offset", "drop", "kp", "kd", "ctrl_clip", "kp_scale", "kd_scale",
    "torque_limit_scale", "action_bias", "torque_bias", "action_noise", "torque_noise", "friction", "mass_scale",
    "env_mask",
    "qacc", "ctrl_out", "xpos", "xquat", "cvel", "traj_ctrl", "traj_xpos", "traj_xquat", "solver_niter", "nefc",
    "dbg_M", "dbg_bias", "dbg_qacc_smooth", "contact_dist", "cinert", "cfrc_ext", "armature_scale", "damping_scale",
    "frictionloss", "body_ipos", "body_inertia", "sph_pos", "sph_radius", "env_order", "work",
)


class KsStepIO(ctypes.Structure):
    _fields_ = [("N", c_int64), ("substeps", c_int32), ("actuator_period", c_int32), ("actuator_type", c_int32),
                ("action_scale", c_float)] + [(name, _P) for name in STEP_IO_POINTERS] + [
                    ("n_events", c_int32), ("events", _T.KsEventDesc * _T.KS_MAX_EVENTS), ("event_state", _P),
                    ("event_uniform", _P), ("event_rng", _T.KsRng), ("event_force", _P), ("fresh", _P)]


def model_desc(m) -> KsModelDesc:
    """KinematicModel -> KsModelDesc."""
    d = KsModelDesc()
    for k in ("nb", "nq", "nv", "nu", "ns", "iterations", "ls_iterations"):
        setattr(d, k, int(getattr(m, k)))
    d.eulerdamp = int(bool(m.eulerdamp))
    d.condim = int(getattr(m, "condim", 3))
    for k in ("dt", "tolerance", "ls_tolerance", "impratio", "meaninertia", "friction"):
        setattr(d, k, float(getattr(m, k)))

    def fill(field, arr):
        arr = np.asarray(arr)
        if arr.size == 0:
            return
        dst = np.ctypeslib.as_array(getattr(d, field))
        if dst.ndim == 1:
            dst[: arr.size] = arr.reshape(-1)
        else:
            dst[: arr.shape[0], :] = arr

    for k in ("gravity", "solref", "solimp", "body_parent", "body_jtype", "body_qadr", "body_dofadr",
              "body_subtree_end", "body_pos", "body_quat", "body_mass", "body_ipos", "body_iquat", "body_inertia",
              "jnt_axis", "jnt_pos", "qpos0", "dof_body", "dof_parent", "dof_damping", "dof_armature", "act_dof",
              "act_gear", "sph_body", "sph_pos", "sph_radius", "jnt_limited", "jnt_range", "dof_invweight0",
              "dof_frictionloss", "dof_solref", "dof_solimp", "dof_stiffness"):
        fill(k, getattr(m, k))
    fill("body_invweight0", m.body_invweight0[:, 0])
    fill("act_lo", m.act_ctrlrange.reshape(-1, 2)[:, 0])
    fill("act_hi", m.act_ctrlrange.reshape(-1, 2)[:, 1])
    return d


def bind(lib) -> None:
    lib.ks_model_create.argtypes = [POINTER(KsModelDesc), POINTER(c_void_p)]
    lib.ks_model_destroy.argtypes = [c_void_p]
    lib.ks_model_lds_bytes.argtypes = [c_void_p]
    lib.ks_step.argtypes = [c_void_p, c_void_p, POINTER(KsStepIO)]
    lib.ks_forward.argtypes = [c_void_p, c_void_p, POINTER(KsStepIO)]
    lib.ks_work_order.argtypes = [c_void_p, c_int64, c_void_p, c_void_p]
    for name in ("ks_model_create", "ks_model_destroy", "ks_model_lds_bytes", "ks_step", "ks_forward", "ks_work_order"):
        getattr(lib, name).restype = c_int32
