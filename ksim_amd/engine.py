"""Physics engine behind the reference's PhysicsEngine interface (ksim/engine.py:48-523), batched.

``HipEngine`` is the MI355X counterpart of ``MjxEngine`` (engine.py:202-361): ``reset`` and ``step`` keep
the reference's argument meaning, but operate on all N envs at once (the reference vmaps the per-env call,
ksim/task/rl.py:1615) and update the PhysicsState in place (the reference donates it, engine.py:259-263).
"""
from __future__ import annotations

import logging
from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import Literal, Mapping, Sequence

import torch

from . import _lib, physics
from . import _lib_terms as T
from .actuators import Actuators, PositionActuators, TorqueActuators
from .env_terms import EnvTerms
from .noise import RandomVariable
from .resets import Reset
from .types import PhysicsData, PhysicsState

logger = logging.getLogger(__name__)
EngineType = Literal["hip"]
MISSING = None


# per-env replacements of model fields that randomisers may produce (ksim/randomization.py), passed to the kernels as they are
_RESIDENT_ENVS = 256 * 16  # wavefronts of the step kernel that an MI355X holds at a time: 256 CUs x 4 SIMDs x 4 waves
_MODEL_FIELD_OVERRIDES = ("frictionloss", "body_ipos", "body_inertia", "sph_pos", "sph_radius")

@dataclass
class EngineConfig:  # engine.py:48-139
    action_latency_range: tuple[float, float] = (0.0, 0.0)
    drop_action_prob: float = 0.0
    zero_offset_std: float | None = None
    zero_offset_mag: float | None = None
    actuator_update_dt: float | None = None
    ctrl_dt: float | None = MISSING
    dt: float | None = MISSING
    # not in the reference: launch the envs heaviest first, ordered by the previous step's cost (see KsStepIO.env_order)
    balance_launch_order: bool = True

    def __post_init__(self) -> None:
        if self.dt is MISSING:
            raise ValueError("`dt` is required")
        if self.ctrl_dt is MISSING:
            raise ValueError("`ctrl_dt` is required")
        lo, hi = self.action_latency_range
        if lo < 0:
            raise ValueError("`min_action_latency` must be non-negative")
        if lo > hi:
            raise ValueError("`min_action_latency` must be less than or equal to `max_action_latency`")
        if hi > self.ctrl_dt:
            logger.warning("`max_action_latency=%f` is greater than `ctrl_dt=%f`", hi, self.ctrl_dt)
        if (self.ctrl_dt - round(self.ctrl_dt / self.dt) * self.dt) > 1e-6:
            logger.warning("`ctrl_dt=%f` is not a multiple of `dt=%f`", self.ctrl_dt, self.dt)
        if self.drop_action_prob < 0 or self.drop_action_prob >= 1:
            raise ValueError("`drop_action_prob` must be between 0 and 1")

    @property
    def min_action_latency_step(self) -> float:
        return self.action_latency_range[0] / self.dt

    @property
    def max_action_latency_step(self) -> float:
        return self.action_latency_range[1] / self.dt

    @property
    def phys_steps_per_ctrl_steps(self) -> int:
        return round(self.ctrl_dt / self.dt)

    @property
    def phys_steps_per_actuator_step(self) -> int:
        if self.actuator_update_dt is not None:
            return max(1, round(self.actuator_update_dt / self.dt))
        return 1

    def zero_offset_random_variable(self) -> RandomVariable:  # engine.py:117-138
        both = self.zero_offset_std is not None and self.zero_offset_mag is not None  # then one key draws both parts
        return RandomVariable(mean=0.0, std=self.zero_offset_std or 0.0, mag=self.zero_offset_mag or 0.0, same_key=both)


@dataclass(frozen=True)
class EngineData:  # engine.py:141-168
    dt: float
    ctrl_dt: float
    drop_action_prob: float
    actuator_update_dt: float | None
    min_action_latency_step: float
    max_action_latency_step: float
    phys_steps_per_ctrl_steps: int
    phys_steps_per_actuator_step: int
    zero_offset: RandomVariable
    balance_launch_order: bool = True

    @classmethod
    def from_config(cls, config: EngineConfig) -> "EngineData":
        return cls(dt=config.dt, ctrl_dt=config.ctrl_dt, drop_action_prob=config.drop_action_prob,
                   actuator_update_dt=config.actuator_update_dt,
                   min_action_latency_step=config.min_action_latency_step,
                   max_action_latency_step=config.max_action_latency_step,
                   phys_steps_per_ctrl_steps=config.phys_steps_per_ctrl_steps,
                   phys_steps_per_actuator_step=config.phys_steps_per_actuator_step,
                   zero_offset=config.zero_offset_random_variable(), balance_launch_order=config.balance_launch_order)


class PhysicsEngine(ABC):  # engine.py:171-199
    actuators: Actuators
    resets: tuple
    events: Mapping
    data: EngineData

    @abstractmethod
    def reset(self, physics_model, curriculum_level, rng, num_envs: int, randomization=None) -> PhysicsState:
        """Reset the engine and return the physics state of `num_envs` fresh episodes."""

    @abstractmethod
    def step(self, action, physics_model, physics_state: PhysicsState, curriculum_level, rng,
             randomization=None) -> PhysicsState:
        """Step the engine and return the updated physics state."""


def _generator(rng, device) -> torch.Generator:
    if isinstance(rng, torch.Generator):
        return rng
    g = torch.Generator(device=device)
    g.manual_seed(int(rng))
    return g


class HipEngine(PhysicsEngine):
    """Engine for `physics.DeviceModel`s: every physics substep of a control step runs in one HIP kernel."""

    def __init__(self, actuators: Actuators, resets: Sequence[Reset], events: Mapping | None, data: EngineData):
        from .events import Event  # noqa: PLC0415
        events = dict(events or {})
        for name, ev in events.items():
            if not isinstance(ev, Event):
                raise NotImplementedError(f"event {name!r} ({type(ev).__name__}) is not one of the compiled events")
        if len(events) > T.KS_MAX_EVENTS:
            raise ValueError(f"at most {T.KS_MAX_EVENTS} events")
        self.actuators, self.resets, self.events, self.data = actuators, tuple(resets), events, data
        self._terms: dict[int, EnvTerms] = {}

    def __hash__(self) -> int:
        return id(self)

    def _reset_terms(self, physics_model: physics.DeviceModel) -> EnvTerms:
        key = id(physics_model)
        if key not in self._terms:
            self._terms[key] = EnvTerms(physics_model.model, {}, {}, self.resets,
                                        action_dim=self.actuators.action_dim(physics_model.model.nu))
        return self._terms[key]

    def _check(self, physics_model) -> None:
        m = physics_model.model
        if abs(m.dt - self.data.dt) > 1e-9:
            raise ValueError(f"model dt {m.dt} differs from the engine's dt {self.data.dt}")
        if isinstance(self.actuators, PositionActuators) and len(self.actuators.kps) != m.nu:
            raise ValueError("one kp / kd per actuator is required")

    # -------------------------------------------------------------------------------------- reset (engine.py:205-246)
    def reset(self, physics_model: physics.DeviceModel, curriculum_level, rng, num_envs: int,
              randomization: Mapping[str, torch.Tensor] | None = None, reset_uniform=None, episode_draws=None) -> PhysicsState:
        self._check(physics_model)
        m, N, dev = physics_model.model, int(num_envs), torch.device("cuda")
        gen = _generator(rng, dev)
        z = lambda *s: torch.zeros(*s, dtype=torch.float32, device=dev)  # noqa: E731
        data = PhysicsData(qpos=z(N, m.nq), qvel=z(N, m.nv), qacc=z(N, m.nv), qacc_warmstart=z(N, m.nv),
                           ctrl=z(N, m.nu), time=z(N), xpos=z(N, m.nb * 3), xquat=z(N, m.nb * 4), cvel=z(N, m.nb * 6),
                           contact_dist=z(N, m.ns) if m.ns else None, cinert=z(N, m.nb * 10), cfrc_ext=z(N, m.nb * 6))
        # latency, zero offset and actuator state are filled by the reset kernel below, the same code that re-draws them
        # for an env that is reset in the middle of a rollout (engine.py:222-245)
        act_state = None
        if isinstance(self.actuators, PositionActuators):
            act_state = {"action": z(N, m.nu), "torque": z(N, m.nu), "kp_scale": z(N), "kd_scale": z(N),
                         "torque_limit_scale": z(N)}
        state = PhysicsState(
            last_ctrl=z(N, self.actuators.action_dim(m.nu)), data=data, event_states=self._initial_event_states(N, gen, dev),
            actuator_state=act_state, action_latency=z(N), zero_offset=z(N, m.nu),
        )
        seed = int(torch.randint(0, 2**31 - 1, (1,), generator=gen, device=dev).item())
        self.reset_where(physics_model, state, None, curriculum_level, seed, 0, randomization, reset_uniform,
                         episode_draws=episode_draws)
        return state

    def episode_args(self, state: PhysicsState, draws: Mapping | None = None) -> dict:
        """What `EnvTerms.terminate_reset(episode=...)` takes: the per-episode buffers of `state`, the random variables
        behind them, and optionally explicit draws {"uniform", "normal"}, each (N, 3 nu + 4), and for the resets that
        use them {"pitch_roll_uniform"} (N) in [0, 1) and {"frame"} (N, int32)."""
        out = dict(action_latency=state.action_latency, zero_offset=state.zero_offset,
                   latency_range=(self.data.min_action_latency_step, self.data.max_action_latency_step),
                   zero_offset_rv=self.data.zero_offset)
        act = self.actuators
        if isinstance(act, PositionActuators) and state.actuator_state is not None:
            ast, rv = state.actuator_state, act._rv
            out.update(act_action_bias=ast["action"], act_torque_bias=ast["torque"], act_kp_scale=ast["kp_scale"],
                       act_kd_scale=ast["kd_scale"], act_torque_limit_scale=ast["torque_limit_scale"],
                       action_bias_rv=act.action_bias or RandomVariable(), torque_bias_rv=act.torque_bias or RandomVariable(),
                       kp_scale_rv=rv(act.kp_scale) or RandomVariable(mean=1.0), kd_scale_rv=rv(act.kd_scale) or RandomVariable(mean=1.0),
                       torque_limit_scale_rv=rv(act.torque_limit_scale) or RandomVariable(mean=1.0))
        if draws:
            out.update(episode_uniform=draws.get("uniform"), episode_normal=draws.get("normal"),
                       reset_pitch_roll_uniform=draws.get("pitch_roll_uniform"), reset_frame=draws.get("frame"))
        return out

    def _initial_event_states(self, N: int, gen, dev) -> dict:
        """One timer per event and env (engine.py:226-232); rows of one (n_events, N) buffer, which the kernels take."""
        if not self.events:
            return {}
        from .events import ForcePushEvent  # noqa: PLC0415
        buf = torch.stack([ev.get_initial_event_state(N, gen, dev) for ev in self.events.values()]).contiguous()
        out = {name: buf[j] for j, name in enumerate(self.events)}
        out["_buffer"] = buf
        if any(isinstance(ev, ForcePushEvent) for ev in self.events.values()):
            # force pushes also carry (duration left, force, torque) per env, zero at the start (events.py:360-365);
            # their state reads (time remaining, duration left, wrench) like the reference's tuple
            force = torch.zeros(len(self.events), N, T.KS_EVENT_FORCE_STATE, dtype=torch.float32, device=dev)
            out["_force_buffer"] = force
            for j, (name, ev) in enumerate(self.events.items()):
                if isinstance(ev, ForcePushEvent):
                    out[name] = (buf[j], force[j, :, 0], force[j, :, 1:7])
        return out

    def event_args(self, physics_state: PhysicsState, curriculum_level, seed: int, step: int, step_base=None, uniform=None):
        """(descs, state, draws, rng) for `physics.control_step`, or None when the engine has no events."""
        if not self.events:
            return None
        descs = [ev.desc(float(curriculum_level)) for ev in self.events.values()]
        rng = T.KsRng(int(seed) & (2**64 - 1), int(step) & (2**64 - 1), _lib.ptr(step_base).value)
        return descs, physics_state.event_states["_buffer"], uniform, rng, physics_state.event_states.get("_force_buffer")

    def reset_where(self, physics_model, state: PhysicsState, mask, curriculum_level, seed: int, step: int,
                    randomization=None, reset_uniform=None, episode_draws=None) -> None:
        """With `mask` None: fresh episodes for every env (resets, per-episode draws, then mjx.forward's counterpart).
        With a mask: only the forward pass of the masked envs, whose state `EnvTerms.terminate_reset` has already reset."""
        d = state.data
        terms = self._reset_terms(physics_model)
        st = dict(qpos=d.qpos, qvel=d.qvel, qacc_warmstart=d.qacc_warmstart, time=d.time, last_ctrl=state.last_ctrl)
        if mask is None:
            terms.terminate_reset(st, level=float(curriculum_level), seed=seed, step=step, apply_reset=2,
                                  reset_uniform=reset_uniform, episode=self.episode_args(state, episode_draws))
        self.forward(physics_model, state, mask, randomization)

    def forward(self, physics_model, state: PhysicsState, mask=None, randomization=None, live=None) -> None:
        """`live`: names of the derived fields of `state.data` to refresh (None = all of them); a rollout whose terms read
        none of a field leaves it out, and the field then holds stale values."""
        d = state.data
        rnd = randomization or {}
        keep = (lambda name, buf: buf) if live is None else (lambda name, buf: buf if name in live else None)
        physics.forward(physics_model, dict(qpos=d.qpos, qvel=d.qvel, qacc_warmstart=d.qacc_warmstart, env_mask=mask,
                                            friction=rnd.get("friction"), mass_scale=rnd.get("mass_scale"),
                                            armature_scale=rnd.get("armature_scale"), damping_scale=rnd.get("damping_scale"),
                                            **{k: rnd.get(k) for k in _MODEL_FIELD_OVERRIDES},
                                            xpos=keep("xpos", d.xpos), xquat=keep("xquat", d.xquat), cvel=keep("cvel", d.cvel),
                                            contact_dist=keep("contact_dist", d.contact_dist),
                                            cinert=keep("cinert", d.cinert), cfrc_ext=keep("cfrc_ext", d.cfrc_ext)))
        # engine.py:217-220: qvel and qacc are zeroed after the forward pass (qvel is already zero here)

    def prepare_state(self, state: PhysicsState):
        """The (order, work) buffers of the heaviest-first launch order, made on first use; call before capturing
        `step` into a HIP graph so that their initialisation is not part of the graph."""
        sched = getattr(state, "_schedule", None)
        # A launch of at most _RESIDENT_ENVS envs is resident all at once (one wavefront per env), so the order in which its
        # workgroups start changes nothing: no order is kept, and the kernel's own XCD-aware mapping applies.
        if sched is None and self.data.balance_launch_order and state.data.qpos.shape[0] > _RESIDENT_ENVS:
            n, dev = state.data.qpos.shape[0], state.data.qpos.device
            sched = (torch.arange(n, dtype=torch.int32, device=dev), torch.zeros(n, dtype=torch.int32, device=dev))
            state._schedule = sched
        return sched

    def prepare(self, device):
        """Uploads the actuator gain tables (once per device); call before capturing `step` into a HIP graph,
        where host-to-device copies are not allowed."""
        act = self.actuators
        if not isinstance(act, PositionActuators):
            return None
        cache = getattr(self, "_gain_cache", None)
        if cache is None or cache[0] is not act or cache[1].device != torch.device(device):
            t = lambda a: torch.tensor(a, dtype=torch.float32, device=device)  # noqa: E731
            cache = (act, t(act.kps), t(act.kds), t(act.clip_array()))
            object.__setattr__(self, "_gain_cache", cache)
        return cache

    # -------------------------------------------------------------------------------------- step (engine.py:259-361)
    def step(self, action: torch.Tensor, physics_model: physics.DeviceModel, physics_state: PhysicsState,
             curriculum_level, rng, randomization: Mapping[str, torch.Tensor] | None = None,
             noise: Mapping[str, torch.Tensor] | None = None,
             record: Mapping[str, torch.Tensor] | None = None, want_cvel: bool = True, want_cinert: bool = False,
             want_cfrc_ext: bool = False,
             step: int = 0, step_base=None, event_seed: int = 0, live=None, stats: Mapping[str, torch.Tensor] | None = None,
             fresh: torch.Tensor | None = None) -> PhysicsState:
        """`live`: names among qacc, ctrl, xpos, xquat, contact_dist of the derived fields of `physics_state.data` that
        the caller reads afterwards (None = all).  The rollout records ctrl / xpos / xquat into its own slot through
        `record`, so a task whose observations read none of them need not have them written twice.
        `stats`: optional int32 (N,) buffers `nefc` and `solver_niter` that receive the constraint rows and Newton iterations
        of the last substep (diagnostics; the reference exposes the same numbers as `data.nefc` / `data.solver_niter`), and
        `dbg_M` (N, nv * nv) float32, which the profiling build of the library fills with cycle counts per phase.
        `fresh`: (N,) uint8 mask of envs that were reset since their last step and have not had the forward pass of the
        reset (engine.py:213) yet: the step kernel runs it for them first, in the same launch, instead of a separate masked
        `forward` (the rollout's deferred mode; their derived fields at the reset state itself are then never written)."""
        m, d, s = physics_model.model, physics_state.data, physics_state
        rnd, noise, record = randomization or {}, noise or {}, record or {}
        keep = (lambda name, b: b) if live is None else (lambda name, b: b if name in live else None)
        drop = noise.get("drop")
        p_drop = self.data.drop_action_prob * float(curriculum_level)
        if drop is None and p_drop > 0:  # engine.py:277-278
            gen = _generator(rng, action.device)
            drop = (torch.rand(action.shape, generator=gen, device=action.device) < p_drop).to(torch.uint8)
        buf = dict(qpos=d.qpos, qvel=d.qvel, qacc_warmstart=d.qacc_warmstart, time=d.time, last_ctrl=s.last_ctrl,
                   action=action, latency=s.action_latency,
                   zero_offset=None if _constant(self.data.zero_offset, 0.0) else s.zero_offset, drop=drop,
                   friction=rnd.get("friction"), mass_scale=rnd.get("mass_scale"), armature_scale=rnd.get("armature_scale"),
                   damping_scale=rnd.get("damping_scale"), **{k: rnd.get(k) for k in _MODEL_FIELD_OVERRIDES},
                   qacc=keep("qacc", d.qacc), ctrl_out=keep("ctrl", d.ctrl),
                   xpos=keep("xpos", d.xpos), xquat=keep("xquat", d.xquat), cvel=d.cvel if want_cvel else None,
                   contact_dist=keep("contact_dist", d.contact_dist),
                   cinert=d.cinert if want_cinert else None, cfrc_ext=d.cfrc_ext if want_cfrc_ext else None,
                   action_noise=noise.get("action_noise"),
                   torque_noise=noise.get("torque_noise"), traj_ctrl=record.get("ctrl"),
                   traj_xpos=record.get("xpos"), traj_xquat=record.get("xquat"), fresh=fresh)
        if stats:
            buf.update({k: stats[k] for k in ("nefc", "solver_niter", "dbg_M") if k in stats})
        # heaviest-first launch order from the previous step's cost estimates (kept on the state object)
        sched = self.prepare_state(s)
        if sched is not None:
            buf.update(env_order=sched[0], work=sched[1])
        act = self.actuators
        ev = self.event_args(s, curriculum_level, event_seed, step, step_base, noise.get("event_uniform"))
        if isinstance(act, PositionActuators):
            cache = self.prepare(action.device)
            ast = s.actuator_state or {}
            # a per-episode quantity whose random variable is a constant 0 (offsets, biases) or 1 (scales) is the
            # kernel's default for a null pointer: its buffer holds that constant in every row and is not streamed
            live_ast = lambda name, rv, c: None if _constant(rv, c) else ast.get(name)  # noqa: E731
            buf.update(kp=cache[1], kd=cache[2], ctrl_clip=cache[3],
                       kp_scale=live_ast("kp_scale", act._rv(act.kp_scale), 1.0),
                       kd_scale=live_ast("kd_scale", act._rv(act.kd_scale), 1.0),
                       torque_limit_scale=live_ast("torque_limit_scale", act._rv(act.torque_limit_scale), 1.0),
                       action_bias=live_ast("action", act.action_bias, 0.0),
                       torque_bias=live_ast("torque", act.torque_bias, 0.0))
            physics.control_step(physics_model, buf, substeps=self.data.phys_steps_per_ctrl_steps,
                                 actuator_period=self.data.phys_steps_per_actuator_step,
                                 actuator_type=act.kind, action_scale=act.action_scale, events=ev)  # incl. position-velocity
        elif isinstance(act, TorqueActuators):
            physics.control_step(physics_model, buf, substeps=self.data.phys_steps_per_ctrl_steps,
                                 actuator_period=self.data.phys_steps_per_actuator_step, actuator_type=act.kind, events=ev)
        else:
            raise ValueError(f"Unsupported actuators: {type(act).__name__}")
        if sched is not None:
            physics.work_order(physics_model, sched[1], sched[0])
        return physics_state


def _constant(rv, value: float) -> bool:
    """True when the random variable (None = the default of its field) only ever takes `value`."""
    return rv is None or (rv.mean == value and rv.std == 0.0 and rv.mag == 0.0)


def get_physics_engine(engine_type: str, resets, events, actuators: Actuators, config: EngineConfig) -> PhysicsEngine:
    """Factory with the reference's signature (engine.py:488-515); the only engine type here is "hip"."""
    if engine_type != "hip":
        raise ValueError(f"Unsupported physics model type: {engine_type}")
    return HipEngine(actuators=actuators, resets=resets, events=events, data=EngineData.from_config(config))
