"""Curricula with the reference's names (ksim/curriculum.py): the scalar level in [0, 1] that the engine, the resets, the
events, the noise and the reward scales read (`curriculum_level` at ksim/engine.py:179-192).  Host logic on a few
reductions of the recorded rollout; one call per training iteration (ksim/task/rl.py:2301-2310).

`Trajectory` arrays are time-major (T, N) here, so "per episode" reductions run over axis 0.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch


@dataclass(frozen=True)
class CurriculumState:  # curriculum.py:27-31
    level: float
    state: Any


class Curriculum:
    def __call__(self, trajectory, rewards, num_steps: int, prev_state: CurriculumState) -> CurriculumState:  # pragma: no cover
        raise NotImplementedError

    def get_initial_state(self) -> CurriculumState:  # pragma: no cover
        raise NotImplementedError


def _clip(x: float, lo: float, hi: float) -> float:
    return min(max(x, lo), hi)


@dataclass(frozen=True)
class ConstantCurriculum(Curriculum):  # curriculum.py:54-70
    level: float = 1.0

    def __call__(self, trajectory, rewards, num_steps, prev_state):
        return prev_state

    def get_initial_state(self):
        return CurriculumState(float(self.level), None)


@dataclass(frozen=True)
class LinearCurriculum(Curriculum):  # curriculum.py:73-96: a step every n epochs of training, after a delay
    step_size: float = 0.01
    step_every_n_epochs: int = 1
    min_level: float = 0.0
    delay_steps: int = 0

    def __call__(self, trajectory, rewards, num_steps, prev_state):
        level = (int(num_steps) - self.delay_steps) // self.step_every_n_epochs * self.step_size
        return CurriculumState(_clip(level, self.min_level, 1.0), None)

    def get_initial_state(self):
        return CurriculumState(float(self.min_level), None)


@dataclass(frozen=True)
class EpisodeLengthCurriculum(Curriculum):  # curriculum.py:105-159; state = (step counter, EMA of the episode length)
    num_levels: int = 100
    increase_threshold: float = 3.0
    decrease_threshold: float = 3.0
    min_level_steps: int = 1
    min_level: float = 0.0
    ema_decay: float = 0.9

    def __call__(self, trajectory, rewards, num_steps, prev_state):
        steps, ema_prev = prev_state.state
        ema = self.ema_decay * ema_prev + (1 - self.ema_decay) * float(trajectory.episode_length().mean())
        can_step = steps == 0
        inc, dec = ema > self.increase_threshold and can_step, ema < self.decrease_threshold and can_step
        level = prev_state.level + (1 / self.num_levels if inc else (-1 / self.num_levels if dec else 0.0))
        next_steps = self.min_level_steps if (inc or dec) else max(steps - 1, 0)
        return CurriculumState(_clip(level, self.min_level, 1.0), (next_steps, ema))

    def get_initial_state(self):
        return CurriculumState(float(self.min_level), (self.min_level_steps, 0.0))


@dataclass(frozen=True)
class DistanceFromOriginCurriculum(Curriculum):  # curriculum.py:168-225; state = (step counter, EMA of the distance)
    num_levels: int = 100
    increase_threshold: float = 3.0
    decrease_threshold: float = 3.0
    min_level_steps: int = 1
    min_level: float = 0.0
    ema_decay: float = 0.9

    def __call__(self, trajectory, rewards, num_steps, prev_state):
        steps, ema_prev = prev_state.state
        distance = float(torch.linalg.norm(trajectory.qpos[..., :3], dim=-1).max())
        ema = self.ema_decay * ema_prev + (1 - self.ema_decay) * distance
        cur, steps = prev_state.level, max(steps - 1, 0)
        if ema > self.increase_threshold:
            cand = min(cur + 1.0 / self.num_levels, 1.0)
        elif ema < self.decrease_threshold:
            cand = max(cur - 1.0 / self.num_levels, self.min_level)
        else:
            cand = cur
        new = cand if steps == 0 else cur
        if new != cur:
            steps = self.min_level_steps
        return CurriculumState(new, (steps, ema))

    def get_initial_state(self):
        return CurriculumState(float(self.min_level), (self.min_level_steps, 0.0))


@dataclass(frozen=True)
class StepWhenSaturated(Curriculum):  # curriculum.py:228-277; state = steps until the level may change again
    num_levels: int
    increase_threshold: float
    decrease_threshold: float
    min_level_steps: int
    min_level: float = 0.0

    def __call__(self, trajectory, rewards, num_steps, prev_state):
        level, steps = prev_state.level, prev_state.state
        if steps > 0:
            return CurriculumState(level, steps - 1)
        deaths = float(trajectory.done.float().sum(dim=0).mean())  # finished episodes per env in this rollout
        delta = 1.0 / self.num_levels
        if deaths < self.increase_threshold:
            level += delta
        elif deaths > self.decrease_threshold:
            level -= delta
        return CurriculumState(_clip(level, self.min_level, 1.0), self.min_level_steps)

    def get_initial_state(self):
        return CurriculumState(float(self.min_level), self.min_level_steps)
