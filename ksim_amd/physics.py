"""Device-resident physics model and the batched control-step call (thin layer over the C ABI).

``DeviceModel`` plays the part of the ``mjx.Model`` that ``mjx.put_model`` returns
(ksim/utils/mujoco.py:388-391); ``control_step`` / ``forward`` are the batched forms of
``MjxEngine.step`` / the ``mjx.forward`` inside ``MjxEngine.reset`` (ksim/engine.py:205-361).
"""
from __future__ import annotations

import ctypes
from typing import Mapping

import torch

from . import _lib, _lib_dyn
from .model import KinematicModel


class DeviceModel:
    """Handle of a model uploaded to the current GPU. Immutable; hashable by identity."""

    def __init__(self, model: KinematicModel):
        lib = _lib.load()
        if not torch.cuda.is_available():
            raise _lib.KsError("DeviceModel needs a GPU (there is no CPU path)")
        torch.cuda.current_device()  # make sure a HIP context exists
        torch.zeros(1, device="cuda")
        self.model = model
        self._lib = lib
        self._handle = ctypes.c_void_p()
        desc = _lib_dyn.model_desc(model)
        _lib.check(lib.ks_model_create(ctypes.byref(desc), ctypes.byref(self._handle)))

    @property
    def handle(self) -> ctypes.c_void_p:
        if not self._handle:
            raise _lib.KsError("model handle was closed")
        return self._handle

    @property
    def lds_bytes(self) -> int:
        return int(self._lib.ks_model_lds_bytes(self.handle))

    def close(self) -> None:
        if self._handle:
            self._lib.ks_model_destroy(self._handle)
            self._handle = ctypes.c_void_p()

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass


_F32 = ("qpos", "qvel", "qacc_warmstart", "time", "last_ctrl", "action", "ctrl_in", "latency", "zero_offset", "kp",
        "kd", "ctrl_clip", "kp_scale", "kd_scale", "torque_limit_scale", "action_bias", "torque_bias", "action_noise",
        "torque_noise", "friction", "mass_scale", "qacc", "ctrl_out", "xpos", "xquat", "cvel", "dbg_M", "dbg_bias",
        "dbg_qacc_smooth", "contact_dist", "cinert", "cfrc_ext", "armature_scale", "damping_scale", "frictionloss", "body_ipos",
        "body_inertia", "sph_pos", "sph_radius")
_I32 = ("solver_niter", "nefc", "env_order", "work")


def _expected_shapes(m: KinematicModel, N: int, S: int, actuator_type: int = _lib_dyn.KS_ACT_POSITION) -> dict:
    nb, nq, nv, nu, ns = m.nb, m.nq, m.nv, m.nu, m.ns
    na = 2 * nu if actuator_type == _lib_dyn.KS_ACT_POSITION_VELOCITY else nu  # width of the action vector
    return {
        "qpos": (N, nq), "qvel": (N, nv), "qacc_warmstart": (N, nv), "time": (N,), "last_ctrl": (N, na),
        "action": (N, na), "ctrl_in": (N, nu), "latency": (N,), "zero_offset": (N, nu), "drop": (N, na),
        "kp": (nu,), "kd": (nu,), "ctrl_clip": (nu,), "kp_scale": (N,), "kd_scale": (N,),
        "torque_limit_scale": (N,), "action_bias": (N, nu), "torque_bias": (N, nu), "action_noise": (S, N, na),
        "torque_noise": (S, N, nu), "friction": (N,), "mass_scale": (N, nb), "env_mask": (N,), "fresh": (N,), "qacc": (N, nv), "ctrl_out": (N, nu),
        "xpos": (N, nb * 3), "xquat": (N, nb * 4), "cvel": (N, nb * 6), "traj_ctrl": (N, nu),
        "traj_xpos": (N, nb * 3), "traj_xquat": (N, nb * 4), "solver_niter": (N,), "nefc": (N,),
        "dbg_M": (N, nv * nv), "dbg_bias": (N, nv), "dbg_qacc_smooth": (N, nv), "contact_dist": (N, ns),
        "cinert": (N, nb * 10), "cfrc_ext": (N, nb * 6), "armature_scale": (N, nv), "damping_scale": (N, nv), "env_order": (N,), "work": (N,),
        "frictionloss": (N, nv), "body_ipos": (N, nb * 3), "body_inertia": (N, nb * 3), "sph_pos": (N, ns * 3), "sph_radius": (N, ns),
    }


def _make_io(dm: DeviceModel, buffers: Mapping[str, torch.Tensor | None], substeps: int, actuator_period: int,
             actuator_type: int, action_scale: float) -> _lib_dyn.KsStepIO:
    """Checks every operand shape on the host against what the kernel's indexing assumes."""
    m = dm.model
    qpos = buffers.get("qpos")
    if qpos is None or qpos.dim() != 2:
        raise _lib.KsError("qpos (N, nq) is required")
    N = qpos.shape[0]
    shapes = _expected_shapes(m, N, max(substeps, 1), actuator_type)
    io = _lib_dyn.KsStepIO()
    io.N, io.substeps, io.actuator_period, io.actuator_type = N, substeps, actuator_period, actuator_type
    io.action_scale = action_scale
    for name, t in buffers.items():
        if name not in shapes:
            raise _lib.KsError(f"unknown step buffer {name!r}")
        if t is None:
            continue
        want = torch.uint8 if name in ("drop", "env_mask", "fresh") else (torch.int32 if name in _I32 else torch.float32)
        if name in ("drop", "env_mask", "fresh") and t.dtype == torch.bool:
            t = t.view(torch.uint8)
        _lib.require_cuda(t, dtype=want)
        if tuple(t.shape) != shapes[name] and not (t.numel() == 0 and 0 in shapes[name]):
            raise _lib.KsError(f"{name}: expected shape {shapes[name]}, got {tuple(t.shape)}")
        if t.numel():
            setattr(io, name, t.data_ptr())
    return io


def control_step(dm: DeviceModel, buffers: Mapping[str, torch.Tensor | None], *, substeps: int,
                 actuator_period: int = 1, actuator_type: int = _lib_dyn.KS_ACT_POSITION,
                 action_scale: float = 1.0, events=None) -> None:
    """One control step of every env, in place on ``qpos, qvel, qacc_warmstart, time, last_ctrl``.

    `events`: (descs, state (n_events, N), uniform (substeps, N, n_events, KS_EVENT_DRAWS) or None, KsRng[, force
    state (n_events, N, KS_EVENT_FORCE_STATE)]); the last entry is needed when a force push is among the events."""
    io = _make_io(dm, buffers, substeps, actuator_period, actuator_type, action_scale)
    if events is not None:
        descs, state, uniform, rng, *rest = events
        force = rest[0] if rest else None
        N, draws = int(io.N), _lib_dyn._T.KS_EVENT_DRAWS
        if len(descs) > _lib_dyn._T.KS_MAX_EVENTS:
            raise _lib.KsError(f"at most {_lib_dyn._T.KS_MAX_EVENTS} events")
        _lib.require_cuda(state, dtype=torch.float32)
        if tuple(state.shape) != (len(descs), N):
            raise _lib.KsError(f"event state: expected shape {(len(descs), N)}, got {tuple(state.shape)}")
        if uniform is not None:
            _lib.require_cuda(uniform, dtype=torch.float32)
            if tuple(uniform.shape) != (substeps, N, len(descs), draws):
                raise _lib.KsError(f"event draws: expected shape {(substeps, N, len(descs), draws)}, got {tuple(uniform.shape)}")
        if force is not None:
            _lib.require_cuda(force, dtype=torch.float32)
            if tuple(force.shape) != (len(descs), N, _lib_dyn._T.KS_EVENT_FORCE_STATE):
                raise _lib.KsError(f"force-push state: expected shape {(len(descs), N, _lib_dyn._T.KS_EVENT_FORCE_STATE)}")
            io.event_force = force.data_ptr()
        io.n_events = len(descs)
        for j, dsc in enumerate(descs):
            io.events[j] = dsc
        io.event_state, io.event_uniform = state.data_ptr(), _lib.ptr(uniform).value
        if rng is not None:
            io.event_rng = rng
    _lib.check(dm._lib.ks_step(dm.handle, _lib.current_stream(), ctypes.byref(io)))


def work_order(dm: DeviceModel, work: torch.Tensor, order: torch.Tensor) -> torch.Tensor:
    """`order` <- the envs sorted by `work` (the step kernel's cost estimate), heaviest first: the launch order of the
    next control step."""
    _lib.require_cuda(work, order, dtype=torch.int32)
    if work.dim() != 1 or tuple(order.shape) != tuple(work.shape):
        raise _lib.KsError("work and order must be (N,) int32")
    _lib.check(dm._lib.ks_work_order(_lib.current_stream(), work.shape[0], work.data_ptr(), order.data_ptr()))
    return order


def forward(dm: DeviceModel, buffers: Mapping[str, torch.Tensor | None]) -> None:
    """Derived quantities (and the warm start) for the given state, without integrating."""
    io = _make_io(dm, buffers, 0, 1, _lib_dyn.KS_ACT_TORQUE, 1.0)
    _lib.check(dm._lib.ks_forward(dm.handle, _lib.current_stream(), ctypes.byref(io)))
