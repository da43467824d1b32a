"""Data contracts of the rollout path, batched over envs (ksim/types.py:33-92).

Leaves are torch CUDA tensors: per-step state is (N, dim) env-major; trajectories are time-major
(T, N, dim).  Attribute names follow the reference's dataclasses and the mjx.Data fields its terms read.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping

import torch


@dataclass
class PhysicsData:
    """The fields of mjx.Data that the engine, observations and terminations touch."""
    qpos: torch.Tensor            # (N, nq)
    qvel: torch.Tensor            # (N, nv)
    qacc: torch.Tensor            # (N, nv)
    qacc_warmstart: torch.Tensor  # (N, nv)
    ctrl: torch.Tensor            # (N, nu) torques applied in the last physics step
    time: torch.Tensor            # (N,)
    xpos: torch.Tensor            # (N, nb*3)
    xquat: torch.Tensor           # (N, nb*4)
    cvel: torch.Tensor            # (N, nb*6)
    contact_dist: torch.Tensor | None = None  # (N, ns) sphere-floor distance of the last collision pass (contact.dist)
    cinert: torch.Tensor | None = None        # (N, nb*10) com-based body inertias (mjData.cinert)
    cfrc_ext: torch.Tensor | None = None      # (N, nb*6) contact force on each body, torque then force (mjData.cfrc_ext)


@dataclass
class PhysicsState:  # ksim/types.py:33-43
    last_ctrl: torch.Tensor
    data: PhysicsData
    event_states: Mapping[str, Any]
    actuator_state: Mapping[str, torch.Tensor] | None
    action_latency: torch.Tensor  # (N,) in physics steps
    zero_offset: torch.Tensor     # (N, nu)


@dataclass
class Trajectory:  # ksim/types.py:46-76
    qpos: torch.Tensor | None
    qvel: torch.Tensor | None
    xpos: torch.Tensor | None
    xquat: torch.Tensor | None
    ctrl: torch.Tensor | None
    obs: Mapping[str, torch.Tensor]
    command: Mapping[str, torch.Tensor]
    event_state: Mapping[str, Any]
    action: torch.Tensor | None
    done: torch.Tensor
    success: torch.Tensor | None
    timestep: torch.Tensor | None
    curriculum_level: torch.Tensor | None = None
    termination_components: Mapping[str, torch.Tensor] = field(default_factory=dict)
    aux_outputs: Mapping[str, Any] = field(default_factory=dict)

    def episode_length(self) -> torch.Tensor:
        """Per env, the mean of the recorded timestep over the steps that end an episode, the rollout's last step counted
        as one (ksim/types.py:72-76); arrays are time-major here, so the reference's last axis is axis 0."""
        done = self.done.bool().clone()
        done[-1] = True
        return (self.timestep * done).sum(dim=0) / done.sum(dim=0)


@dataclass
class RewardState:  # ksim/types.py:79-84
    total: torch.Tensor
    components: Mapping[str, torch.Tensor]
    carry: Mapping[str, Any]


@dataclass
class Action:  # ksim/types.py:87-92
    action: torch.Tensor
    carry: Any = None
    aux_outputs: Mapping[str, Any] = field(default_factory=dict)
