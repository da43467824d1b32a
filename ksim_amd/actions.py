"""Action filters with the reference's names (ksim/actions.py): small per-env recursions between the network output and
the target positions.  State tensors are batched (N, num_joints); every function returns new parameter objects like the
reference's, and takes an optional `fresh` (N,) uint8 mask of envs whose state restarts first (the reference re-creates
the parameters with the model carry when an episode starts, ksim/task/rl.py:1083-1123).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _lib
from . import _lib_terms as T

LOWPASS, CLIP_ACCELERATION, INTEGRATE_VELOCITY, INTEGRATE_ACCELERATION, CLIP_POSITIONS, TANH_POSITIONS = range(6)


def _run(kind, x, position=None, velocity=None, *, ctrl_dt=0.0, p0=0.0, lo=None, hi=None, fresh=None, init=None):
    _lib.require_cuda(x, position, velocity, lo, hi, init, dtype=torch.float32)
    if x.dim() != 2:
        raise _lib.KsError("expected (N, num_joints)")
    N, nu = x.shape
    state = None
    if position is not None:
        if tuple(position.shape) != (N, nu) or (velocity is not None and tuple(velocity.shape) != (N, nu)):
            raise _lib.KsError("the filter state must have the shape of the input")
        state = torch.cat([position, velocity if velocity is not None else torch.zeros_like(position)], dim=1).contiguous()
    if fresh is not None:
        _lib.require_cuda(fresh, dtype=torch.uint8)
        if tuple(fresh.shape) != (N,):
            raise _lib.KsError("fresh must be (N,) uint8")
    if init is not None and tuple(init.shape) != (N, nu):
        raise _lib.KsError("init must be (N, num_joints)")
    for r in (lo, hi):
        if r is not None and tuple(r.shape) != (nu,):
            raise _lib.KsError("ranges must be (num_joints,)")
    y = torch.empty_like(x)
    _lib.check(_lib.load().ks_action_filter(_lib.current_stream(), N, nu, kind, float(ctrl_dt), float(p0), _lib.ptr(lo), _lib.ptr(hi),
                                            _lib.ptr(x.contiguous()), _lib.ptr(state), _lib.ptr(fresh), _lib.ptr(init), _lib.ptr(y)))
    return y, (None if state is None else (state[:, :nu].contiguous(), state[:, nu:].contiguous()))


@dataclass(frozen=True)
class LowPass:
    """ksim.lowpass_one_pole on an actor's biased means (examples/kbot/train.py:917-929, ksim/actions.py:248-257), as a
    setting of the policy head: the rollout filters the means before sampling and the policy update differentiates through
    the filter, whose state `lpf_params` rides in the model carry.  `obs_bias` = (first observation column, first action,
    count): that many action means also take the named observation columns as a bias before the filter (the arm commands
    of train.py:920-921)."""
    ctrl_dt: float
    cutoff_frequency: float
    obs_bias: tuple | None = None


@dataclass(frozen=True)
class LowPassFilterParams:  # actions.py:236-245
    y_last: torch.Tensor

    @classmethod
    def initialize(cls, num_envs: int, num_joints: int, device="cuda"):
        return cls(torch.zeros(num_envs, num_joints, device=device))


def lowpass_one_pole(x, ctrl_dt: float, fc: float, params: LowPassFilterParams, fresh=None):
    """y = y_last + alpha (x - y_last) with alpha = dt / (1 / (2 pi fc) + dt) (actions.py:248-257)."""
    y, (pos, _) = _run(LOWPASS, x, params.y_last, ctrl_dt=ctrl_dt, p0=fc, fresh=fresh)
    return y, LowPassFilterParams(pos)


def lowpass_one_pole_scan(x, ctrl_dt: float, fc: float, params: LowPassFilterParams):
    """The filter along the leading (time) axis of x (T, N, num_joints) (actions.py:265-288)."""
    out = []
    for xt in x:
        y, params = lowpass_one_pole(xt, ctrl_dt, fc, params)
        out.append(y)
    return torch.stack(out), params


@dataclass(frozen=True)
class ClipAccelerationParams:  # actions.py:31-46
    position: torch.Tensor
    velocity: torch.Tensor

    @classmethod
    def initialize(cls, num_envs: int, num_joints: int, device="cuda"):
        z = torch.zeros(num_envs, num_joints, device=device)
        return cls(z, z.clone())

    @classmethod
    def initialize_from(cls, init_position: torch.Tensor):
        return cls(init_position, torch.zeros_like(init_position))


def clip_acceleration(target_position, params: ClipAccelerationParams, max_acceleration: float, ctrl_dt: float, fresh=None, init=None):
    """Follows the target with a bounded acceleration (actions.py:54-80)."""
    _, (pos, vel) = _run(CLIP_ACCELERATION, target_position, params.position, params.velocity, ctrl_dt=ctrl_dt, p0=max_acceleration,
                         fresh=fresh, init=init)
    return ClipAccelerationParams(pos, vel)


@dataclass(frozen=True)
class IntegrateVelocityParams:  # actions.py:85-100
    position: torch.Tensor

    @classmethod
    def initialize(cls, num_envs: int, num_joints: int, device="cuda"):
        return cls(torch.zeros(num_envs, num_joints, device=device))

    @classmethod
    def initialize_from(cls, init_position: torch.Tensor):
        return cls(init_position)


def integrate_velocity(velocity, params: IntegrateVelocityParams, ctrl_dt: float, fresh=None, init=None):
    """position += velocity dt (actions.py:108-133; `backprop` only matters to the gradient)."""
    _, (pos, _) = _run(INTEGRATE_VELOCITY, velocity, params.position, ctrl_dt=ctrl_dt, fresh=fresh, init=init)
    return IntegrateVelocityParams(pos)


@dataclass(frozen=True)
class IntegrateAccelerationParams:  # actions.py:136-154
    position: torch.Tensor
    velocity: torch.Tensor

    @classmethod
    def initialize(cls, num_envs: int, num_joints: int, device="cuda"):
        z = torch.zeros(num_envs, num_joints, device=device)
        return cls(z, z.clone())

    @classmethod
    def initialize_from(cls, init_position: torch.Tensor):
        return cls(init_position, torch.zeros_like(init_position))


def integrate_acceleration(acceleration, params: IntegrateAccelerationParams, ctrl_dt: float, max_velocity: float = 10.0,
                           fresh=None, init=None):
    """velocity = clip(velocity + a dt, +-max_velocity), position += velocity dt (actions.py:162-191)."""
    _, (pos, vel) = _run(INTEGRATE_ACCELERATION, acceleration, params.position, params.velocity, ctrl_dt=ctrl_dt, p0=max_velocity,
                         fresh=fresh, init=init)
    return IntegrateAccelerationParams(pos, vel)


class _Ranges:
    def __init__(self, ranges):
        lo, hi = zip(*ranges)
        self.min_ranges, self.max_ranges, self.num_joints = tuple(float(v) for v in lo), tuple(float(v) for v in hi), len(lo)
        self._dev: tuple | None = None

    @classmethod
    def from_physics_model(cls, model):
        """The ranges of every joint but the floating base (actions.py:205-209); `model` is a KinematicModel."""
        hinges = [b for b in range(1, model.nb) if model.body_jtype[b] != 1]
        return cls([tuple(model.jnt_range[b]) for b in hinges])

    def _tensors(self, device):
        if self._dev is None or self._dev[0].device != device:
            self._dev = (torch.tensor(self.min_ranges, device=device), torch.tensor(self.max_ranges, device=device))
        return self._dev


class ClipPositions(_Ranges):  # actions.py:194-214
    def clip(self, positions: torch.Tensor) -> torch.Tensor:
        lo, hi = self._tensors(positions.device)
        return _run(CLIP_POSITIONS, positions, lo=lo, hi=hi)[0]


class TanhPositions(_Ranges):  # actions.py:217-241
    def clip(self, positions: torch.Tensor) -> torch.Tensor:
        lo, hi = self._tensors(positions.device)
        return _run(TANH_POSITIONS, positions, lo=lo, hi=hi)[0]

    def get_bias(self, zeros: torch.Tensor) -> torch.Tensor:
        """The pre-activation whose tanh image is `zeros` (a constant of the network, computed on the host side)."""
        lo, hi = self._tensors(zeros.device)
        return torch.atanh((zeros - lo) / (hi - lo))
