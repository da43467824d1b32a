"""Actuators with the reference's names (ksim/actuators.py:27-238); the PD law runs inside the step kernel."""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from ._lib_dyn import KS_ACT_POSITION, KS_ACT_POSITION_VELOCITY, KS_ACT_TORQUE
from .noise import Noise, RandomVariable


@dataclass(frozen=True, eq=False)
class Actuators:
    kind: int = KS_ACT_TORQUE

    def action_dim(self, nu: int) -> int:
        """Width of the action vector (and of `PhysicsState.last_ctrl`) for a model with `nu` actuators."""
        return nu


@dataclass(frozen=True, eq=False)
class TorqueActuators(Actuators):  # actuators.py:70-87
    noise: Noise | None = None
    kind: int = KS_ACT_TORQUE


@dataclass(frozen=True, eq=False)
class PositionActuators(Actuators):  # actuators.py:98-238
    """MIT-style PD: tau = kp*s_kp*(a*scale + noise + bias - q) + kd*s_kd*(0 - qd), noise + bias, clipped."""
    kps: tuple = ()
    kds: tuple = ()
    ctrl_clip: tuple | None = None
    action_noise: Noise | None = None
    torque_noise: Noise | None = None
    action_scale: float = 1.0
    action_bias: RandomVariable | None = None
    torque_bias: RandomVariable | None = None
    kp_scale: float | RandomVariable | None = None
    kd_scale: float | RandomVariable | None = None
    torque_limit_scale: float | RandomVariable | None = None
    kind: int = KS_ACT_POSITION

    def __post_init__(self):
        kps, kds = np.asarray(self.kps, dtype=np.float64), np.asarray(self.kds, dtype=np.float64)
        if kps.shape != kds.shape or kps.ndim != 1:
            raise ValueError("kps and kds must be 1-D and of equal length")
        if (kps < 0).any() or (kds < 0).any():  # actuators.py:173-174
            raise ValueError("Some KPs or KDs are negative. Check the provided metadata.")
        if self.ctrl_clip is not None and (np.asarray(self.ctrl_clip) < 0).any():  # actuators.py:138-139
            raise ValueError("Soft torque limits must be non-negative")

    def clip_array(self) -> np.ndarray:
        n = len(self.kps)
        return np.full(n, np.inf) if self.ctrl_clip is None else np.asarray(self.ctrl_clip, dtype=np.float64)

    @staticmethod
    def _rv(x) -> RandomVariable | None:
        if x is None or isinstance(x, RandomVariable):
            return x
        return RandomVariable(mean=float(x))  # actuators.py:162-167

    def get_initial_state(self, num_envs: int, gen) -> dict:
        """ActuatorState (actuators.py:90-95,219-238) for a batch of fresh episodes."""
        import torch

        n = len(self.kps)
        dev = gen.device
        zeros = lambda *s: torch.zeros(*s, dtype=torch.float32, device=dev)  # noqa: E731
        ones = lambda *s: torch.ones(*s, dtype=torch.float32, device=dev)  # noqa: E731
        rv = self._rv
        return {
            "action": self.action_bias.sample((num_envs, n), gen) if self.action_bias else zeros(num_envs, n),
            "torque": self.torque_bias.sample((num_envs, n), gen) if self.torque_bias else zeros(num_envs, n),
            "kp_scale": rv(self.kp_scale).sample((num_envs,), gen) if self.kp_scale is not None else ones(num_envs),
            "kd_scale": rv(self.kd_scale).sample((num_envs,), gen) if self.kd_scale is not None else ones(num_envs),
            "torque_limit_scale": rv(self.torque_limit_scale).sample((num_envs,), gen)
            if self.torque_limit_scale is not None else ones(num_envs),
        }


@dataclass(frozen=True, eq=False)
class PositionVelocityActuator(PositionActuators):  # actuators.py:241-293
    """PD on position and velocity targets: the action is (position targets, velocity targets), 2 nu wide, and
    tau = kp (target_pos - q) + kd (target_vel - qd); `action_noise` acts on the position half, `vel_action_noise` on the
    velocity half."""
    vel_action_noise: Noise | None = None
    kind: int = KS_ACT_POSITION_VELOCITY

    def action_dim(self, nu: int) -> int:
        return 2 * nu
