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


@dataclass(frozen=True)
class IllegalContactTermination(Termination):
    """Fails the episode when one of the listed contact spheres is more than `-contact_eps` deep in the floor
    (terminations.py:84-99; every contact of this model pairs a sphere with the floor, so "a contact involving an illegal
    geom with dist < contact_eps" is a statement about the listed spheres)."""
    illegal_sphere_idxs: tuple = ()
    contact_eps: float = -0.001

    @classmethod
    def create(cls, physics_model, body_names, contact_eps: float = -1e-3) -> "IllegalContactTermination":
        """Spheres given by the names of the bodies they are attached to (terminations.py:104-127)."""
        names = set(body_names)
        idxs = []
        for s_, b in enumerate(physics_model.sph_body):
            n = physics_model.body_names[int(b)]
            if n in body_names:
                idxs.append(s_)
                names.discard(n)
        if names:
            raise ValueError(f"Bodies {names} carry no contact sphere. Choices are: {sorted(set(physics_model.body_names[int(b)] for b in physics_model.sph_body))}")
        return cls(illegal_sphere_idxs=tuple(idxs), contact_eps=contact_eps)

    def desc(self):
        mask = 0
        for s_ in self.illegal_sphere_idxs:
            if not 0 <= int(s_) < 24:
                raise ValueError("sphere index out of range")
            mask |= 1 << int(s_)
        return (T.TERM_ILLEGAL_CONTACT, -1, float(self.contact_eps), float(mask), 0.0, 0.0)
