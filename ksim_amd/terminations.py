"""Terminations with the reference's class names and rules (ksim/terminations.py:60-192)."""
from __future__ import annotations

from dataclasses import dataclass

from . import _lib_terms as T


@dataclass(frozen=True)
class Termination:
    def desc(self) -> tuple:  # (kind, value, p0, p1, p2, p3)  # pragma: no cover
        raise NotImplementedError

    def get_name(self) -> str:
        name = type(self).__name__
        return "".join("_" + c.lower() if c.isupper() else c for c in name).lstrip("_")

    @property
    def termination_name(self) -> str:
        return self.get_name()


@dataclass(frozen=True)
class NotUprightTermination(Termination):  # terminations.py:60-70
    max_radians: float

    def __post_init__(self):
        if not self.max_radians > 0:
            raise ValueError("max_radians must be > 0")

    def desc(self):
        return (T.TERM_NOT_UPRIGHT, -1, self.max_radians, 0.0, 0.0, 0.0)


@dataclass(frozen=True)
class MinimumHeightTermination(Termination):  # terminations.py:73-80
    min_height: float

    def __post_init__(self):
        if not self.min_height > 0:
            raise ValueError("min_height must be > 0")

    def desc(self):
        return (T.TERM_MIN_HEIGHT, -1, self.min_height, 0.0, 0.0, 0.0)


@dataclass(frozen=True)
class BadZTermination(Termination):  # terminations.py:131-146
    min_z: float
    max_z: float
    final_min_z: float | None = None
    final_max_z: float | None = None

    def desc(self):
        fmin = self.min_z if self.final_min_z is None else self.final_min_z
        fmax = self.max_z if self.final_max_z is None else self.final_max_z
        return (T.TERM_BAD_Z, -1, self.min_z, self.max_z, fmin, fmax)


@dataclass(frozen=True)
class BadVelocityTermination(Termination):  # terminations.py:149-157
    max_vel: float

    def desc(self):
        return (T.TERM_BAD_VELOCITY, -1, self.max_vel, 0.0, 0.0, 0.0)


@dataclass(frozen=True)
class FarFromOriginTermination(Termination):  # terminations.py:160-172
    max_dist: float
    pos_termination: bool = True

    def desc(self):
        return (T.TERM_FAR_FROM_ORIGIN, 1 if self.pos_termination else -1, self.max_dist, 0.0, 0.0, 0.0)


@dataclass(frozen=True)
class EpisodeLengthTermination(Termination):  # terminations.py:175-192
    max_length_sec: float
    disable_at_curriculum_level: float | None = None
    pos_termination: bool = True

    def desc(self):
        lvl = -1.0 if self.disable_at_curriculum_level is None else float(self.disable_at_curriculum_level)
        return (T.TERM_EPISODE_LENGTH, 1 if self.pos_termination else -1, self.max_length_sec, lvl, 0.0, 0.0)
