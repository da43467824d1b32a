"""Observations with the reference's class names (ksim/observation.py:184-352,705-713).

Each class compiles to per-element descriptors that the fused observation kernel evaluates
(`ks_observe`); ``noise`` / ``bias`` follow ksim/observation.py:89-145 (a float noise is additive
Gaussian).  Stateful observations (delay buffers, the IMU-lag filter of ProjectedGravityObservation,
contact observations) are not compiled here.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from . import _lib_terms as T
from .model import KinematicModel
from .noise import Noise, convert_to_noise


@dataclass(frozen=True)
class ObsElem:
    kind: int
    src: int
    index: int = 0
    comp: int = 0
    const: tuple = (0.0, 0.0, 0.0)


@dataclass(frozen=True)
class Observation:
    noise: Noise | float | None = None
    bias: float | None = None  # std of the per-episode additive Gaussian bias (observation.py:79-86)

    def elements(self, model: KinematicModel, command_dim: int) -> list[ObsElem]:  # pragma: no cover
        raise NotImplementedError

    def get_name(self) -> str:
        name = type(self).__name__
        out = "".join("_" + c.lower() if c.isupper() else c for c in name).lstrip("_")
        return out

    @property
    def observation_name(self) -> str:
        return self.get_name()

    def _noise(self) -> Noise | None:
        return convert_to_noise(self.noise)


def _copy(src, start, n):
    return [ObsElem(T.OBS_COPY, src, start + i) for i in range(n)]


def _rot(src, start, const=(0.0, 0.0, 0.0)):
    return [ObsElem(T.OBS_ROT_INV, src, start, c, const) for c in range(3)]


@dataclass(frozen=True)
class BasePositionObservation(Observation):  # observation.py:185-188
    def elements(self, m, command_dim):
        return _copy(T.SRC_QPOS, 0, 3)


@dataclass(frozen=True)
class BaseOrientationObservation(Observation):  # observation.py:192-195
    def elements(self, m, command_dim):
        return _copy(T.SRC_QPOS, 3, 4)


@dataclass(frozen=True)
class BaseLinearVelocityObservation(Observation):  # observation.py:199-206
    in_robot_frame: bool = False

    def elements(self, m, command_dim):
        return _rot(T.SRC_QVEL, 0) if self.in_robot_frame else _copy(T.SRC_QVEL, 0, 3)


@dataclass(frozen=True)
class BaseAngularVelocityObservation(Observation):  # observation.py:210-217
    in_robot_frame: bool = False

    def elements(self, m, command_dim):
        return _rot(T.SRC_QVEL, 3) if self.in_robot_frame else _copy(T.SRC_QVEL, 3, 3)


@dataclass(frozen=True)
class JointPositionObservation(Observation):  # observation.py:221-225 (qpos[7:] - zero_offset)
    def elements(self, m, command_dim):
        return [ObsElem(T.OBS_JOINT_POS, T.SRC_QPOS, 7 + i) for i in range(m.nq - 7)]


@dataclass(frozen=True)
class JointVelocityObservation(Observation):  # observation.py:255-257
    def elements(self, m, command_dim):
        return _copy(T.SRC_QVEL, 6, m.nv - 6)


@dataclass(frozen=True)
class ActuatorForceObservation(Observation):  # observation.py:300-303 (unit-gear motors: force = ctrl)
    def elements(self, m, command_dim):
        return _copy(T.SRC_CTRL, 0, m.nu)


@dataclass(frozen=True)
class BaseLinearAccelerationObservation(Observation):  # observation.py:343-346
    def elements(self, m, command_dim):
        return _copy(T.SRC_QACC, 0, 3)


@dataclass(frozen=True)
class BaseAngularAccelerationObservation(Observation):  # observation.py:349-352
    def elements(self, m, command_dim):
        return _copy(T.SRC_QACC, 3, 3)


@dataclass(frozen=True)
class ActuatorAccelerationObservation(Observation):  # observation.py:445-448
    def elements(self, m, command_dim):
        return _copy(T.SRC_QACC, 6, m.nv - 6)


@dataclass(frozen=True)
class CenterOfMassVelocityObservation(Observation):  # observation.py:293-297 (cvel[1:].ravel())
    def elements(self, m, command_dim):
        return _copy(T.SRC_CVEL, 6, (m.nb - 1) * 6)


@dataclass(frozen=True)
class BodyPositionObservation(Observation):  # observation.py:524-559 (xpos of chosen bodies)
    body_ids: tuple = ()

    def elements(self, m, command_dim):
        return [e for b in self.body_ids for e in _copy(T.SRC_XPOS, 3 * b, 3)]


@dataclass(frozen=True)
class BodyOrientationObservation(Observation):  # observation.py:618-641
    body_ids: tuple = ()

    def elements(self, m, command_dim):
        return [e for b in self.body_ids for e in _copy(T.SRC_XQUAT, 4 * b, 4)]


@dataclass(frozen=True)
class TimestepObservation(Observation):  # observation.py:705-713
    def elements(self, m, command_dim):
        return _copy(T.SRC_TIME, 0, 1)


@dataclass(frozen=True)
class ProjectedGravityObservation(Observation):
    """Gravity in the base frame, rot(q_base)^-1 g: the stateless core of observation.py:355-442 (lag 0, no IMU bias)."""
    gravity: tuple = (0.0, 0.0, -9.81)

    def elements(self, m, command_dim):
        return _rot(T.SRC_CONST, 0, tuple(float(g) for g in self.gravity))


@dataclass(frozen=True)
class LastActionObservation(Observation):
    """The previous control step's action (PhysicsState.last_ctrl, ksim/types.py:33-43)."""

    def elements(self, m, command_dim):
        return _copy(T.SRC_LAST_ACTION, 0, m.nu)


@dataclass(frozen=True)
class CommandObservation(Observation):
    """The env's command vector (ksim/observation.py:61-66 ObservationInput.commands), passed through."""

    def elements(self, m, command_dim):
        return _copy(T.SRC_COMMAND, 0, command_dim)
