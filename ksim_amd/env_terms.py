"""Compiled per-env terms: observations, terminations, resets -> one device spec + the fused kernels.

Covers get_observation (ksim/task/rl.py:153-186), get_terminations and the done/success combination
(rl.py:288-299,1049-1050), the reset-under-cond of _get_step_env_state (rl.py:1072-1080) and the NaN
scrub / clip of sampled actions (rl.py:998-1001).
"""
from __future__ import annotations

import ctypes
from typing import Mapping, Sequence

import numpy as np
import torch

from . import _lib
from . import _lib_terms as T
from .model import KinematicModel
from .observation import Observation
from .resets import Reset, compile_resets
from .terminations import Termination


def _rng(seed: int, step: int, step_base: torch.Tensor | None = None) -> T.KsRng:
    """Philox key; `step_base` (one int64 on the device) is added to `step` when the kernel runs."""
    if step_base is not None:
        _lib.require_cuda(step_base, dtype=torch.int64)
    return T.KsRng(int(seed) & (2**64 - 1), int(step) & (2**64 - 1), _lib.ptr(step_base).value)


# Sources an observation element reads besides its own `src`, per kind: the same list `ks_observe` checks for null
# pointers before it launches.  `Rollout` keeps a derived field of the live physics data up to date only when it is in
# the union of these sets, so a kind missing here would read the values of the last reset.
KIND_SOURCES = {
    T.OBS_JOINT_POS: (T.SRC_QPOS,),
    T.OBS_ROT_INV: (T.SRC_QPOS,),
    T.OBS_GRAVITY_EMA: (T.SRC_QPOS,),
    T.OBS_CONTACT_ANY: (T.SRC_CONTACT_DIST,),
    T.OBS_SITE_ROT6D: (T.SRC_XQUAT,),
    T.OBS_SITE_GYRO: (T.SRC_XQUAT, T.SRC_CVEL),
    T.OBS_SITE_ACCEL: (T.SRC_XQUAT, T.SRC_CVEL, T.SRC_QACC),
    T.OBS_SITE_POS: (T.SRC_XQUAT, T.SRC_XPOS),
    T.OBS_SITE_QUAT: (T.SRC_XQUAT,),
    T.OBS_SITE_MAGNETOMETER: (T.SRC_XQUAT,),
}


def compile_terms(model: KinematicModel, observations: Mapping[str, Observation],
                  terminations: Mapping[str, Termination], resets: Sequence[Reset], command_dim: int = 0,
                  terminate_on_nonfinite: bool = True, action_dim: int | None = None):
    """Host-side compilation of the task's terms into the flat tables of KsTermsDesc (no GPU involved).

    Returns (desc, obs_slices, sources_used, has_bias, reset_table); `desc.carry_dim` is the length of the per-env
    carry row of the stateful observations, laid out in dict order; `has_bias` says whether any observation carries a
    per-episode bias (then `observe` needs the bias-draw buffer)."""
    d = T.KsTermsDesc()
    d.nq, d.nv, d.nu, d.nb, d.command_dim = model.nq, model.nv, model.nu, model.nb, int(command_dim)
    d.ns = model.ns
    d.action_dim = model.nu if action_dim is None else int(action_dim)
    carry_at = 0
    obs_slices: dict[str, slice] = {}
    sources_used: set[int] = set()
    has_bias = False
    k = 0
    for name, obs in observations.items():
        elems = obs.elements(model, int(command_dim))
        noise, bias = obs._noise(), obs._bias()
        if k + len(elems) > T.KS_MAX_OBS:
            raise _lib.KsError(f"observation vector longer than {T.KS_MAX_OBS}")
        for el in elems:
            e = d.obs[k]
            e.kind, e.src, e.index, e.comp = el.kind, el.src, el.index, el.comp
            e.c0, e.c1, e.c2 = el.const
            e.carry, e.stride = carry_at + el.carry, el.stride
            e.q0, e.q1, e.q2 = el.q
            e.e0, e.e1, e.e2, e.e3 = el.e
            e.env_site = int(el.env_site)
            sources_used.add(el.src)
            sources_used.update(KIND_SOURCES.get(el.kind, ()))
            if noise is not None:
                stages = noise.stages()
                e.n_noise = len(stages)
                for j, st in enumerate(stages):
                    e.noise[j].kind, e.noise[j].mean, e.noise[j].scale, e.noise[j].scale2 = st.kind, st.mean, st.scale, st.scale2
            if bias is not None and bias.kind != T.NOISE_NONE:
                e.bias.kind, e.bias.mean, e.bias.scale, e.bias.scale2 = bias.kind, bias.mean, bias.scale, bias.scale2
                has_bias = True
            k += 1
        obs_slices[name] = slice(k - len(elems), k)
        carry_at += obs.carry_size(model)
    d.obs_dim, d.carry_dim = k, carry_at
    if len(terminations) > T.KS_MAX_TERMS:
        raise _lib.KsError("too many terminations")
    for j, term in enumerate(terminations.values()):
        t = d.terms[j]
        t.kind, t.value, t.p0, t.p1, t.p2, t.p3 = term.desc()
    d.n_terms = len(terminations)
    tab = compile_resets(resets, model)
    big = 3.0e38
    for i in range(model.nq):
        d.reset_base[i], d.reset_mag[i] = tab["base"][i], tab["mag"][i]
        d.reset_lo[i], d.reset_hi[i] = max(tab["lo"][i], -big), min(tab["hi"][i], big)
        d.reset_by_level[i] = int(tab["by_level"][i])
        d.reset_from_motion[i] = int(tab["motion"][i])
    d.random_heading = int(tab["heading"])
    d.reset_pitch_roll = int(tab["pitch_roll"])
    d.reset_pitch[0], d.reset_pitch[1] = (float(x) for x in tab["pitch"])
    d.reset_roll[0], d.reset_roll[1] = (float(x) for x in tab["roll"])
    if tab["hfield"] is not None:
        d.reset_hfield = 1
        d.hfield_bound[0], d.hfield_bound[1] = (float(x) for x in tab["hfield"]["bound"])
    d.nonfinite_terminates = int(terminate_on_nonfinite)
    return d, obs_slices, sources_used, has_bias, tab


class EnvTerms:
    def __init__(self, model: KinematicModel, observations: Mapping[str, Observation],
                 terminations: Mapping[str, Termination], resets: Sequence[Reset], command_dim: int = 0,
                 terminate_on_nonfinite: bool = True, action_dim: int | None = None):
        lib = _lib.load()
        torch.zeros(1, device="cuda")
        self.model, self._lib = model, lib
        self.observations, self.terminations, self.resets = dict(observations), dict(terminations), tuple(resets)
        self.command_dim = int(command_dim)
        d, self.obs_slices, self.sources_used, self.has_bias, self.reset_table = compile_terms(
            model, self.observations, self.terminations, self.resets, self.command_dim, terminate_on_nonfinite, action_dim)
        self.action_dim = int(d.action_dim)
        self._motion = self._hfield = None  # device copies of the reset tables' data, made on first use
        self.obs_dim, self.n_terms, self.carry_dim = int(d.obs_dim), int(d.n_terms), int(d.carry_dim)
        self._handle = ctypes.c_void_p()
        _lib.check(lib.ks_terms_create(ctypes.byref(d), ctypes.byref(self._handle)))

    # ------------------------------------------------------------------ observations
    def observe(self, sources: Mapping[int, torch.Tensor | None], N: int, *, level: float = 1.0,
                zero_offset=None, bias_draw=None, bias_redraw=None, noise_normal=None, noise_uniform=None, seed: int = 0,
                step: int = 0, step_base=None, carry=None, fresh=None, carry_uniform=None, site_pose=None,
                obs: torch.Tensor | None = None, noisy_obs: torch.Tensor | None = None, _io_only: bool = False):
        """`carry` (N, carry_dim) is advanced in place; `fresh` (N) uint8 marks the envs whose carries are initialised
        from the current state first (those that were just reset) and whose bias draws `bias_draw` (N, obs_dim, 2) are
        renewed (from `bias_redraw` when given, else from the Philox stream).  `site_pose` (N, 7): per-env orientation
        (wxyz) and position of the site that the observations built with `site_pose_per_env` read."""
        m = self.model
        dims = {T.SRC_QPOS: m.nq, T.SRC_QVEL: m.nv, T.SRC_QACC: m.nv, T.SRC_CTRL: m.nu, T.SRC_LAST_ACTION: self.action_dim,
                T.SRC_COMMAND: self.command_dim, T.SRC_TIME: 1, T.SRC_XPOS: m.nb * 3, T.SRC_XQUAT: m.nb * 4,
                T.SRC_CVEL: m.nb * 6, T.SRC_CONTACT_DIST: m.ns, T.SRC_CINERT: m.nb * 10, T.SRC_CFRC_EXT: m.nb * 6}
        io = T.KsObserveIO()
        io.N, io.level = N, level
        for s, t in sources.items():
            if t is None:
                continue
            _lib.require_cuda(t, dtype=torch.float32)
            if t.numel() != N * dims[s]:
                raise _lib.KsError(f"observation source {s}: expected {N}x{dims[s]} elements, got {tuple(t.shape)}")
            io.src[s] = t.data_ptr()
        for name, t, shape in (("zero_offset", zero_offset, (N, m.nu)), ("bias_draw", bias_draw, (N, self.obs_dim, 2)),
                               ("bias_redraw", bias_redraw, (N, self.obs_dim, 2)),
                               ("noise_normal", noise_normal, (N, self.obs_dim)),
                               ("noise_uniform", noise_uniform, (N, self.obs_dim)), ("obs", obs, (N, self.obs_dim)),
                               ("noisy_obs", noisy_obs, (N, self.obs_dim)), ("carry", carry, (N, self.carry_dim)),
                               ("carry_uniform", carry_uniform, (N, self.carry_dim)), ("site_pose", site_pose, (N, 7))):
            if t is None:
                continue
            _lib.require_cuda(t, dtype=torch.float32)
            if tuple(t.shape) != shape:
                raise _lib.KsError(f"{name}: expected {shape}, got {tuple(t.shape)}")
            setattr(io, name, t.data_ptr())
        if fresh is not None:
            _lib.require_cuda(fresh, dtype=torch.uint8)
            if tuple(fresh.shape) != (N,):
                raise _lib.KsError(f"fresh: expected ({N},), got {tuple(fresh.shape)}")
            io.fresh = fresh.data_ptr()
        io.rng = _rng(seed, step, step_base)
        if _io_only:
            return io
        _lib.check(self._lib.ks_observe(self._handle, _lib.current_stream(), ctypes.byref(io)))
        return obs, noisy_obs

    # ------------------------------------------------------------------ terminations + reset predication
    def terminate_reset(self, state: Mapping[str, torch.Tensor], *, level: float = 1.0, components=None, done=None,
                        success=None, traj_qpos=None, traj_qvel=None, traj_time=None, reset_mask=None,
                        episode_length=None, reset_uniform=None, seed: int = 0, step: int = 0, step_base=None,
                        event_state=None, event_intervals=(), event_reset_uniform=None, event_force=None,
                        contact_dist=None, apply_reset: bool = True, episode: Mapping | None = None, _io_only: bool = False):
        """`episode`: the per-episode quantities that the envs starting a fresh episode re-draw (engine.py:222-245), as
        `HipEngine.episode_args` builds them: buffers `action_latency`, `zero_offset`, `act_*`, the matching random
        variables, and optionally explicit draws `episode_uniform` / `episode_normal` (N, 3 nu + 4),
        `reset_pitch_roll_uniform` (N) in [0, 1) and `reset_frame` (N, int32) for the resets that draw them."""
        m = self.model
        qpos = state["qpos"]
        N = qpos.shape[0]
        io = T.KsTerminateIO()
        io.N, io.level, io.apply_reset = N, level, int(apply_reset)
        spec = [("qpos", state.get("qpos"), (N, m.nq), torch.float32), ("qvel", state.get("qvel"), (N, m.nv), torch.float32),
                ("qacc_warmstart", state.get("qacc_warmstart"), (N, m.nv), torch.float32),
                ("time", state.get("time"), (N,), torch.float32), ("last_ctrl", state.get("last_ctrl"), (N, self.action_dim), torch.float32),
                ("components", components, (self.n_terms, N), torch.int8), ("done", done, (N,), torch.uint8),
                ("success", success, (N,), torch.uint8), ("traj_qpos", traj_qpos, (N, m.nq), torch.float32),
                ("traj_qvel", traj_qvel, (N, m.nv), torch.float32), ("traj_time", traj_time, (N,), torch.float32),
                ("reset_mask", reset_mask, (N,), torch.uint8), ("episode_length", episode_length, (N,), torch.int32),
                ("reset_uniform", reset_uniform, (N, m.nq + 1), torch.float32)]
        for name, t, shape, dt in spec:
            if t is None:
                continue
            if t.dtype == torch.bool and dt == torch.uint8:
                t = t.view(torch.uint8)
            _lib.require_cuda(t, dtype=dt)
            if tuple(t.shape) != shape:
                raise _lib.KsError(f"{name}: expected {shape}, got {tuple(t.shape)}")
            setattr(io, name, t.data_ptr())
        io.rng = _rng(seed, step, step_base)
        if contact_dist is not None:  # for IllegalContactTermination
            _lib.require_cuda(contact_dist, dtype=torch.float32)
            if tuple(contact_dist.shape) != (N, m.ns):
                raise _lib.KsError(f"contact_dist must be ({N}, {m.ns})")
            io.contact_dist = contact_dist.data_ptr()
        if event_state is not None:  # timers of the events, re-drawn for the envs that start a fresh episode
            _lib.require_cuda(event_state, dtype=torch.float32)
            if tuple(event_state.shape) != (len(event_intervals), N):
                raise _lib.KsError("event state must be (n_events, N)")
            io.n_events, io.event_state = len(event_intervals), event_state.data_ptr()
            for j, (lo, hi) in enumerate(event_intervals):
                io.event_interval[j][0], io.event_interval[j][1] = float(lo), float(hi)
            if event_reset_uniform is not None:
                _lib.require_cuda(event_reset_uniform, dtype=torch.float32)
                if tuple(event_reset_uniform.shape) != (N, len(event_intervals)):
                    raise _lib.KsError("event reset draws must be (N, n_events)")
                io.event_reset_uniform = event_reset_uniform.data_ptr()
            if event_force is not None:
                _lib.require_cuda(event_force, dtype=torch.float32)
                if tuple(event_force.shape) != (len(event_intervals), N, T.KS_EVENT_FORCE_STATE):
                    raise _lib.KsError("force-push state must be (n_events, N, KS_EVENT_FORCE_STATE)")
                io.event_force = event_force.data_ptr()
        # tables of the resets that read data: the reference motion and the height field live on the device from first use
        tab = self.reset_table
        if apply_reset and tab["motion"].any():
            if self._motion is None:
                self._motion = torch.from_numpy(tab["motion_qpos"]).to(qpos.device)
            io.reset_motion_qpos, io.reset_motion_frames = self._motion.data_ptr(), self._motion.shape[0]
            io.reset_motion_dt = tab["motion_dt"]
        if apply_reset and tab["hfield"] is not None:
            if self._hfield is None:
                self._hfield = torch.from_numpy(tab["hfield"]["data"]).to(qpos.device)
            io.reset_hfield, io.hfield_nx, io.hfield_ny = self._hfield.data_ptr(), self._hfield.shape[0], self._hfield.shape[1]
        for name, dt in (("reset_pitch_roll_uniform", torch.float32), ("reset_frame", torch.int32)):
            t = (episode or {}).get(name)
            if t is not None:
                _lib.require_cuda(t, dtype=dt)
                if tuple(t.shape) != (N,):
                    raise _lib.KsError(f"{name}: expected ({N},), got {tuple(t.shape)}")
                setattr(io, name, t.data_ptr())
        if episode:
            nu, ned = m.nu, 3 * m.nu + 4
            shapes = dict(action_latency=(N,), zero_offset=(N, nu), act_action_bias=(N, nu), act_torque_bias=(N, nu),
                          act_kp_scale=(N,), act_kd_scale=(N,), act_torque_limit_scale=(N,), episode_uniform=(N, ned),
                          episode_normal=(N, ned))
            for name, shape in shapes.items():
                t = episode.get(name)
                if t is None:
                    continue
                _lib.require_cuda(t, dtype=torch.float32)
                if tuple(t.shape) != shape:
                    raise _lib.KsError(f"{name}: expected {shape}, got {tuple(t.shape)}")
                setattr(io, name, t.data_ptr())
            io.latency_lo, io.latency_hi = (float(x) for x in episode.get("latency_range", (0.0, 0.0)))
            for name in ("zero_offset_rv", "action_bias_rv", "torque_bias_rv", "kp_scale_rv", "kd_scale_rv", "torque_limit_scale_rv"):
                rv = episode.get(name)
                if rv is not None:
                    setattr(io, name, rv.desc())
        if _io_only:
            return io
        _lib.check(self._lib.ks_terminate_reset(self._handle, _lib.current_stream(), ctypes.byref(io)))

    def terminate_reset_observe(self, state: Mapping[str, torch.Tensor], terminate: Mapping, sources: Mapping[int, torch.Tensor | None],
                                observe: Mapping) -> None:
        """`terminate_reset(state, **terminate)` of one control step and `observe(sources, N, **observe)` of the next one in
        a single launch (`ks_terminate_reset_observe`): the observation sees the state the termination pass leaves, and
        its `fresh` flags must be that pass's `reset_mask`.  Same results as the two calls in a row."""
        tio = self.terminate_reset(state, _io_only=True, **terminate)
        oio = self.observe(sources, state["qpos"].shape[0], _io_only=True, **observe)
        _lib.check(self._lib.ks_terminate_reset_observe(self._handle, _lib.current_stream(), ctypes.byref(tio), ctypes.byref(oio)))

    def close(self) -> None:
        if self._handle:
            self._lib.ks_terms_destroy(self._handle)
            self._handle = ctypes.c_void_p()

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass


def sample_action(mean: torch.Tensor, log_std: torch.Tensor | None, *, noise: torch.Tensor | None = None,
                  seed: int = 0, step: int = 0, step_base=None, clip_max: float = 1e3,
                  out: torch.Tensor | None = None):
    """action = mean + exp(log_std) * N(0,1); NaN -> 0; clip to +-clip_max (ksim/task/rl.py:998-1001)."""
    lib = _lib.load()
    _lib.require_cuda(mean, log_std, noise, out, dtype=torch.float32)
    N, nu = mean.shape
    if log_std is not None and tuple(log_std.shape) != (nu,):
        raise _lib.KsError("log_std must have shape (nu,)")
    if noise is not None and noise.shape != mean.shape:
        raise _lib.KsError("noise must match the mean's shape")
    if out is None:
        out = torch.empty_like(mean)
    _lib.check(lib.ks_sample_action(_lib.current_stream(), N, nu, _lib.ptr(mean), _lib.ptr(log_std), _lib.ptr(noise),
                                    _rng(seed, step, step_base), float(clip_max), _lib.ptr(out)))
    return out


def sample_action_head(raw: torch.Tensor, *, min_std: float, max_std: float, var_scale: float = 1.0,
                       mean_bias: torch.Tensor | None = None, noise: torch.Tensor | None = None, deterministic: bool = False,
                       seed: int = 0, step: int = 0, step_base=None, clip_max: float = 1e3, out: torch.Tensor | None = None,
                       want_stats: bool = False):
    """Sampling tail for a network that emits means and raw deviations, `raw` (N, 2 nu) (examples/kbot/train.py:915-932):
    std = min((softplus(raw_std) + min_std) * var_scale, max_std); action = mean + std * N(0,1), scrubbed and clipped
    (ksim/task/rl.py:998-1001).  With `want_stats` also returns (mean, std, per-dimension log-probability)."""
    lib = _lib.load()
    _lib.require_cuda(raw, mean_bias, noise, out, dtype=torch.float32)
    if raw.dim() != 2 or raw.shape[1] % 2:
        raise _lib.KsError("raw must be (N, 2 nu)")
    N, nu = raw.shape[0], raw.shape[1] // 2
    if mean_bias is not None and tuple(mean_bias.shape) != (nu,):
        raise _lib.KsError("mean_bias must have shape (nu,)")
    if noise is not None and tuple(noise.shape) != (N, nu):
        raise _lib.KsError("noise must be (N, nu)")
    if out is None:
        out = torch.empty((N, nu), dtype=torch.float32, device=raw.device)
    elif tuple(out.shape) != (N, nu):
        raise _lib.KsError("out must be (N, nu)")
    stats = tuple(torch.empty((N, nu), dtype=torch.float32, device=raw.device) for _ in range(3)) if want_stats else (None,) * 3
    head = T.KsGaussianHead(float(min_std), float(max_std), float(var_scale), int(bool(deterministic)), _lib.ptr(mean_bias).value)
    _lib.check(lib.ks_sample_action_head(_lib.current_stream(), N, nu, _lib.ptr(raw), ctypes.byref(head), _lib.ptr(noise),
                                         _rng(seed, step, step_base), float(clip_max), _lib.ptr(out), *(_lib.ptr(t) for t in stats)))
    return (out, *stats) if want_stats else out


def sample_action_mixture(raw: torch.Tensor, num_mixtures: int, *, min_std: float, max_std: float, var_scale: float = 1.0,
                          mean_bias: torch.Tensor | None = None, clip_lo: torch.Tensor | None = None,
                          clip_hi: torch.Tensor | None = None, uniform: torch.Tensor | None = None,
                          noise: torch.Tensor | None = None, deterministic: bool = False, seed: int = 0, step: int = 0,
                          step_base=None, clip_max: float = 1e3, out: torch.Tensor | None = None, want_stats: bool = False):
    """Sampling tail of the walking example's actor (examples/walking.py:127-144): `raw` (N, 3 nu K) holds component means,
    raw deviations and logits, each (nu, K).  One component per action dimension is drawn from softmax(logits), the action
    from that component's Gaussian; scrub and clip as ksim/task/rl.py:998-1001.  With `want_stats` also returns the
    per-dimension log-probability of the sample under the mixture and the component drawn."""
    lib = _lib.load()
    _lib.require_cuda(raw, mean_bias, clip_lo, clip_hi, uniform, noise, out, dtype=torch.float32)
    K = int(num_mixtures)
    if raw.dim() != 2 or K < 1 or raw.shape[1] % (3 * K):
        raise _lib.KsError("raw must be (N, 3 nu K)")
    N, nu = raw.shape[0], raw.shape[1] // (3 * K)
    for name, t, shape in (("mean_bias", mean_bias, (nu,)), ("clip_lo", clip_lo, (nu,)), ("clip_hi", clip_hi, (nu,)),
                           ("uniform", uniform, (N, nu)), ("noise", noise, (N, nu))):
        if t is not None and tuple(t.shape) != shape:
            raise _lib.KsError(f"{name} must have shape {shape}")
    if out is None:
        out = torch.empty((N, nu), dtype=torch.float32, device=raw.device)
    elif tuple(out.shape) != (N, nu):
        raise _lib.KsError("out must be (N, nu)")
    logp = torch.empty((N, nu), dtype=torch.float32, device=raw.device) if want_stats else None
    comp = torch.empty((N, nu), dtype=torch.int32, device=raw.device) if want_stats else None
    head = T.KsMixtureHead(K, float(min_std), float(max_std), float(var_scale), int(bool(deterministic)),
                           _lib.ptr(mean_bias).value, _lib.ptr(clip_lo).value, _lib.ptr(clip_hi).value)
    _lib.check(lib.ks_sample_action_mixture(_lib.current_stream(), N, nu, _lib.ptr(raw), ctypes.byref(head), _lib.ptr(uniform),
                                            _lib.ptr(noise), _rng(seed, step, step_base), float(clip_max), _lib.ptr(out),
                                            _lib.ptr(logp), _lib.ptr(comp)))
    return (out, logp, comp) if want_stats else out
