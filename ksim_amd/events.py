"""Events applied inside the substep loop of the engine (ksim/events.py:25-237, engine.py:322-333).

The events are compiled into the fused step kernel: every physics substep their timers run down by dt and, when one
reaches zero, the velocity events (linear / angular push, jump) add an impulse to the root velocity and
`ForcePushEvent` draws a new force and torque, which one body then receives for a drawn duration; a new interval
is drawn as well.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _lib_terms as T
from .scales import convert_to_scale


def _scale(scale, level: float) -> float:
    """The event's magnitude multiplier at this curriculum level (events.py:96-97)."""
    return float(convert_to_scale(scale).get_scale(level))


@dataclass(frozen=True)
class Event:
    interval_range: tuple[float, float]

    def get_initial_event_state(self, num_envs: int, generator: torch.Generator, device) -> torch.Tensor:
        lo, hi = self.interval_range  # events.py:110-112
        return lo + (hi - lo) * torch.rand(num_envs, generator=generator, device=device)

    def desc(self, curriculum_level: float) -> T.KsEventDesc:
        raise NotImplementedError


@dataclass(frozen=True)
class LinearPushEvent(Event):  # events.py:115-171
    linvel: float = 0.0
    vel_range: tuple[float, float] = (0.0, 1.0)
    scale: object = 1.0

    def desc(self, curriculum_level: float) -> T.KsEventDesc:
        return T.KsEventDesc(T.EVENT_LINEAR_PUSH, self.linvel, self.vel_range[0], self.vel_range[1],
                             self.interval_range[0], self.interval_range[1], _scale(self.scale, curriculum_level))


@dataclass(frozen=True)
class AngularPushEvent(Event):  # events.py:58-112
    angvel: float = 0.0
    vel_range: tuple[float, float] = (0.0, 1.0)
    scale: object = 1.0

    def desc(self, curriculum_level: float) -> T.KsEventDesc:
        return T.KsEventDesc(T.EVENT_ANGULAR_PUSH, self.angvel, self.vel_range[0], self.vel_range[1],
                             self.interval_range[0], self.interval_range[1], _scale(self.scale, curriculum_level))


@dataclass(frozen=True)
class JumpEvent(Event):  # events.py:174-237
    jump_height_range: tuple[float, float] = (0.0, 0.0)
    scale: object = 1.0

    def desc(self, curriculum_level: float) -> T.KsEventDesc:
        return T.KsEventDesc(T.EVENT_JUMP, 0.0, self.jump_height_range[0], self.jump_height_range[1],
                             self.interval_range[0], self.interval_range[1], _scale(self.scale, curriculum_level))


@dataclass(frozen=True)
class ForcePushEvent(Event):  # events.py:240-365
    max_force: float = 0.0
    max_torque: float = 0.0
    duration_range: tuple[float, float] = (0.0, 0.0)
    body_id: int = 1
    force_range: tuple[float, float] = (0.0, 1.0)
    scale: object = 1.0

    @classmethod
    def from_body_name(cls, model, body_name: str, *, max_force: float, max_torque: float,
                       duration_range: tuple[float, float], interval_range: tuple[float, float],
                       force_range: tuple[float, float] = (0.0, 1.0), scale=1.0) -> "ForcePushEvent":
        names = list(model.body_names)  # events.py:252-277
        if body_name not in names:
            raise ValueError(f"Body name {body_name} not found in model")
        return cls(interval_range=interval_range, max_force=max_force, max_torque=max_torque,
                   duration_range=duration_range, body_id=names.index(body_name), force_range=force_range, scale=scale)

    def desc(self, curriculum_level: float) -> T.KsEventDesc:
        return T.KsEventDesc(T.EVENT_FORCE_PUSH, self.max_force, self.force_range[0], self.force_range[1],
                             self.interval_range[0], self.interval_range[1], _scale(self.scale, curriculum_level),
                             self.max_torque, self.duration_range[0], self.duration_range[1], int(self.body_id))
