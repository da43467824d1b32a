"""ctypes front-end of the C dynamics oracle (oracle/ks_dyn_oracle.c) — TEST INFRASTRUCTURE.

``Oracle(model_arrays, dtype)`` wraps one precision of the oracle; ``Oracle.data()`` makes a
per-env data block whose fields are numpy views of the C struct.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import c_double, c_float, c_int

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libksoracle.so")
FLOPS_LIB = os.path.join(HERE, "libksoracle_flops.so")
MAXB, MAXQ, MAXV, MAXU, MAXS, MAXR = 32, 40, 32, 32, 16, 128


def build(force: bool = False) -> str:
    src = [os.path.join(HERE, f) for f in ("ks_dyn_oracle.c", "ks_dyn_oracle.h", "flop_count.cpp", "Makefile")]
    if force or not os.path.exists(LIB) or not os.path.exists(FLOPS_LIB) or any(os.path.getmtime(s) > os.path.getmtime(LIB) for s in src):
        subprocess.run(["make", "-C", HERE, "-B"], check=True, capture_output=True)
    return LIB


class KsorModel(ctypes.Structure):
    _fields_ = [
        ("nb", c_int), ("nq", c_int), ("nv", c_int), ("nu", c_int), ("ns", c_int),
        ("iterations", c_int), ("ls_iterations", c_int), ("eulerdamp", c_int), ("condim", c_int),
        ("dt", c_double), ("gravity", c_double * 3), ("tolerance", c_double), ("ls_tolerance", c_double),
        ("impratio", c_double), ("meaninertia", c_double), ("solref", c_double * 2), ("solimp", c_double * 5),
        ("body_parent", c_int * MAXB), ("body_jtype", c_int * MAXB), ("body_qadr", c_int * MAXB),
        ("body_dofadr", c_int * MAXB), ("body_subtree_end", c_int * MAXB),
        ("body_pos", c_double * 3 * MAXB), ("body_quat", c_double * 4 * MAXB), ("body_mass", c_double * MAXB),
        ("body_ipos", c_double * 3 * MAXB), ("body_iquat", c_double * 4 * MAXB), ("body_inertia", c_double * 3 * MAXB),
        ("jnt_axis", c_double * 3 * MAXB), ("jnt_pos", c_double * 3 * MAXB), ("body_invweight0", c_double * MAXB),
        ("qpos0", c_double * MAXQ),
        ("dof_body", c_int * MAXV), ("dof_parent", c_int * MAXV), ("dof_damping", c_double * MAXV),
        ("dof_armature", c_double * MAXV),
        ("jnt_limited", c_int * MAXB), ("jnt_range", c_double * 2 * MAXB), ("dof_invweight0", c_double * MAXV),
        ("dof_frictionloss", c_double * MAXV), ("dof_solref", c_double * 2), ("dof_solimp", c_double * 5),
        ("dof_stiffness", c_double * MAXV),
        ("act_dof", c_int * MAXU), ("act_gear", c_double * MAXU), ("act_lo", c_double * MAXU),
        ("act_hi", c_double * MAXU),
        ("sph_body", c_int * MAXS), ("sph_pos", c_double * 3 * MAXS), ("sph_radius", c_double * MAXS),
    ]


def _data_struct(real):
    class KsorData(ctypes.Structure):
        _fields_ = [
            ("qpos", real * MAXQ), ("qvel", real * MAXV), ("ctrl", real * MAXU), ("qacc_warmstart", real * MAXV),
            ("time", real),
            ("mass_scale", real * MAXB), ("friction", real), ("armature_scale", real * MAXV),
            ("damping_scale", real * MAXV),
            ("has_ipos", c_int), ("has_inertia", c_int), ("has_frictionloss", c_int), ("has_spheres", c_int),
            ("body_ipos", real * 3 * MAXB), ("body_inertia", real * 3 * MAXB), ("dof_frictionloss", real * MAXV),
            ("sph_pos", real * 3 * MAXS), ("sph_radius", real * MAXS),
            ("xfrc_applied", real * 6 * MAXB),
            ("xpos", real * 3 * MAXB), ("xquat", real * 4 * MAXB), ("xmat", real * 9 * MAXB),
            ("xipos", real * 3 * MAXB), ("ximat", real * 9 * MAXB), ("xanchor", real * 3 * MAXB),
            ("xaxis", real * 3 * MAXB), ("com", real * 3),
            ("cinert", real * 10 * MAXB), ("crb", real * 10 * MAXB), ("cdof", real * 6 * MAXV),
            ("M", real * (MAXV * MAXV)), ("L", real * (MAXV * MAXV)),
            ("cvel", real * 6 * MAXB), ("cdof_dot", real * 6 * MAXV),
            ("qfrc_bias", real * MAXV), ("qfrc_passive", real * MAXV), ("qfrc_actuator", real * MAXV),
            ("actuator_force", real * MAXU), ("qfrc_smooth", real * MAXV), ("qacc_smooth", real * MAXV),
            ("nefc", c_int), ("solver_niter", c_int),
            ("con_dist", real * MAXS), ("con_pos", real * 3 * MAXS),
            ("efc_J", real * (MAXR * MAXV)), ("efc_pos", real * MAXR), ("efc_aref", real * MAXR),
            ("efc_D", real * MAXR), ("efc_force", real * MAXR), ("efc_floss", real * MAXR),
            ("qfrc_constraint", real * MAXV), ("qacc", real * MAXV), ("cfrc_ext", real * 6 * MAXB),
        ]

    return KsorData


DataF64 = _data_struct(c_double)
DataF32 = _data_struct(c_float)


def make_model(a: dict) -> KsorModel:
    m = KsorModel()
    for k in ("nb", "nq", "nv", "nu", "ns", "iterations", "ls_iterations"):
        setattr(m, k, int(a[k]))
    m.eulerdamp = int(bool(a["eulerdamp"]))
    m.condim = int(a.get("condim", 3))
    for k in ("dt", "tolerance", "ls_tolerance", "impratio", "meaninertia"):
        setattr(m, k, float(a[k]))

    def fill(field, arr):
        arr = np.asarray(arr)
        dst = np.ctypeslib.as_array(getattr(m, field))
        if arr.size == 0:
            return
        if dst.ndim == 1:
            dst[: arr.size] = arr.reshape(-1)
        else:
            dst[: arr.shape[0], :] = arr

    fill("gravity", a["gravity"]); fill("solref", a["solref"]); fill("solimp", a["solimp"])
    for k in ("body_parent", "body_jtype", "body_qadr", "body_dofadr", "body_subtree_end", "body_mass", "qpos0",
              "dof_body", "dof_parent", "dof_damping", "dof_armature", "act_dof", "act_gear", "sph_body",
              "sph_radius"):
        fill(k, a[k])
    for k in ("body_pos", "body_quat", "body_ipos", "body_iquat", "body_inertia", "jnt_axis", "jnt_pos", "sph_pos"):
        fill(k, a[k])
    fill("body_invweight0", np.asarray(a["body_invweight0"])[:, 0])
    for k in ("jnt_limited", "jnt_range", "dof_invweight0", "dof_frictionloss", "dof_solref", "dof_solimp", "dof_stiffness"):
        if k in a:  # absent: no limits, no dry friction
            fill(k, a[k])
    fill("act_lo", np.asarray(a["act_ctrlrange"]).reshape(-1, 2)[:, 0])
    fill("act_hi", np.asarray(a["act_ctrlrange"]).reshape(-1, 2)[:, 1])
    return m


class DataView:
    """numpy views of one KsorData block, trimmed to the model's sizes."""

    def __init__(self, raw, a: dict):
        object.__setattr__(self, "raw", raw)
        object.__setattr__(self, "_a", a)

    def __getattr__(self, name):
        raw, a = self.raw, self._a
        v = getattr(raw, name)
        if isinstance(v, (int, float)):
            return v
        arr = np.ctypeslib.as_array(v)
        nb, nq, nv, nu, ns = a["nb"], a["nq"], a["nv"], a["nu"], a["ns"]
        trim = {"qpos": nq, "qvel": nv, "ctrl": nu, "qacc_warmstart": nv, "mass_scale": nb, "armature_scale": nv, "damping_scale": nv, "xfrc_applied": nb, "cfrc_ext": nb, "xpos": nb, "xquat": nb,
                "xmat": nb, "xipos": nb, "ximat": nb, "xanchor": nb, "xaxis": nb, "cinert": nb, "crb": nb, "cdof": nv,
                "cvel": nb, "cdof_dot": nv, "qfrc_bias": nv, "qfrc_passive": nv, "qfrc_actuator": nv,
                "actuator_force": nu, "qfrc_smooth": nv, "qacc_smooth": nv, "con_dist": ns, "con_pos": ns,
                "qfrc_constraint": nv, "qacc": nv}
        if name in ("M", "L"):
            return arr[: nv * nv].reshape(nv, nv)
        if name == "efc_J":
            return arr[: raw.nefc * nv].reshape(raw.nefc, nv)
        if name in ("efc_pos", "efc_aref", "efc_D", "efc_force", "efc_floss"):
            return arr[: raw.nefc]
        if name in trim:
            return arr[: trim[name]]
        return arr

    def __setattr__(self, name, value):
        if name == "time" or name == "friction":
            setattr(self.raw, name, float(value))
            return
        getattr(self, name)[...] = value


class Oracle:
    def __init__(self, model_arrays: dict, dtype=np.float64, count_flops: bool = False):
        """`count_flops`: the float64 oracle built with a scalar type that counts its floating-point operations
        (flop_count.cpp); `flops()` reads the count, `flops_reset()` clears it.  One thread only."""
        build()
        self.lib = ctypes.CDLL(FLOPS_LIB if count_flops else LIB)
        self.a = model_arrays
        self.model = make_model(model_arrays)
        self.dtype = np.dtype(dtype)
        if count_flops and self.dtype != np.float64:
            raise ValueError("the counting oracle computes in float64")
        self.suf = "_cnt" if count_flops else "_f64" if self.dtype == np.float64 else "_f32"
        self.Data = DataF64 if self.dtype == np.float64 else DataF32
        size = getattr(self.lib, "ksor_sizeof_data" + self.suf)()
        assert size == ctypes.sizeof(self.Data), (size, ctypes.sizeof(self.Data))

    def fn(self, name):
        f = getattr(self.lib, name + self.suf)
        f.restype = None
        return f

    def data(self, qpos=None, qvel=None, friction=None, mass_scale=None, armature_scale=None, damping_scale=None,
             body_ipos=None, body_inertia=None, dof_frictionloss=None, sph_pos=None, sph_radius=None) -> DataView:
        raw = self.Data()
        d = DataView(raw, self.a)
        d.qpos = self.a["qpos0"] if qpos is None else qpos
        if qvel is not None:
            d.qvel = qvel
        d.mass_scale = 1.0 if mass_scale is None else mass_scale
        d.raw.armature_scale[:] = [1.0] * MAXV
        d.raw.damping_scale[:] = [1.0] * MAXV
        if armature_scale is not None:
            d.armature_scale = armature_scale
        if damping_scale is not None:
            d.damping_scale = damping_scale
        d.friction = self.a["friction"] if friction is None else friction
        # per-env replacements of model fields (None: the model's own)
        nb, nv, ns = self.a["nb"], self.a["nv"], self.a["ns"]
        for flag, fields in (("has_ipos", (("body_ipos", body_ipos, nb),)), ("has_inertia", (("body_inertia", body_inertia, nb),)),
                             ("has_frictionloss", (("dof_frictionloss", dof_frictionloss, nv),)),
                             ("has_spheres", (("sph_pos", sph_pos, ns), ("sph_radius", sph_radius, ns)))):
            given = [v is not None for _, v, _ in fields]
            if any(given):
                if not all(given):
                    raise ValueError("sph_pos and sph_radius come together")
                for name, v, n in fields:
                    np.ctypeslib.as_array(getattr(raw, name))[:n] = np.asarray(v)
                setattr(raw, flag, 1)
        return d

    def flops(self) -> float:
        f = self.lib.ksor_flops
        f.restype = c_double
        return float(f())

    def flops_reset(self) -> None:
        self.lib.ksor_flops_reset()

    def call(self, name, d: DataView):
        self.fn(name)(ctypes.byref(self.model), ctypes.byref(d.raw))

    def forward(self, d):
        self.call("ksor_forward", d)

    def step(self, d):
        self.call("ksor_step", d)

    def position_stage(self, d):
        for n in ("ksor_kinematics", "ksor_com_pos", "ksor_crb"):
            self.call(n, d)

    def velocity_stage(self, d):
        for n in ("ksor_com_vel", "ksor_rne"):
            self.call(n, d)

    # ---- batched control step (N envs, env-major arrays) used by parity tests and the CPU baseline
    def batch(self, N: int):
        block = (self.Data * N)()
        ones = [1.0] * MAXV
        for e in range(N):  # neutral per-env parameters; the caller sets state, mass scales and friction
            block[e].armature_scale[:] = ones
            block[e].damping_scale[:] = ones
        return block

    def ctrl_step_batch(self, block, S, actuator_period, action, last_ctrl, latency, zero_offset, kp, kd, ctrl_clip,
                        nthreads=1, qvel_impulse=None):
        N = len(block)
        dt = self.dtype
        c = lambda x: None if x is None else np.ascontiguousarray(x, dtype=dt)  # noqa: E731
        action, latency, zero_offset, kp, kd, ctrl_clip, qvel_impulse = map(c, (action, latency, zero_offset, kp, kd, ctrl_clip, qvel_impulse))
        assert last_ctrl.dtype == dt and last_ctrl.flags.c_contiguous
        p = lambda x: None if x is None else x.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
        f = self.fn("ksor_ctrl_step_batch")
        f.argtypes = [ctypes.c_void_p, c_int, c_int, c_int, ctypes.c_void_p] + [ctypes.c_void_p] * 7 + [c_int, ctypes.c_void_p]
        f(ctypes.byref(self.model), N, S, actuator_period, ctypes.byref(block), p(action), p(last_ctrl), p(latency),
          p(zero_offset), p(kp), p(kd), p(ctrl_clip), nthreads, p(qvel_impulse))
