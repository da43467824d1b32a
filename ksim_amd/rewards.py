"""Rewards with the reference's class names (ksim/rewards.py) evaluated by the fused reward kernel.

``get_rewards`` mirrors ksim/task/rl.py:189-245: each term times ``scale`` (negated when the class name
ends in ``Penalty``, rewards.py:117-124), summed in dict order, optionally clipped.  Trajectory leaves are
time-major (T, N, ...) tensors.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Mapping

import torch

from . import _lib
from . import _lib_terms as T
from .types import RewardState, Trajectory


@dataclass(frozen=True)
class Reward:
    scale: float = 1.0

    def descs(self) -> list[tuple]:  # [(suffix | None, kind, norm, p0, p1, p2)]  # pragma: no cover
        raise NotImplementedError

    @property
    def is_penalty(self) -> bool:  # rewards.py:117-124
        name = type(self).__name__.lower()
        if name.endswith("reward"):
            return False
        if name.endswith("penalty"):
            return True
        raise ValueError(f"Reward function {type(self).__name__} does not end with 'Reward' or 'Penalty'")


@dataclass(frozen=True)
class StayAliveReward(Reward):  # rewards.py:166-188
    balance: float = 100.0
    success_reward: float | None = None

    def descs(self):
        has = self.success_reward is not None
        return [(None, T.REW_STAY_ALIVE, 0, self.balance, self.success_reward if has else 0.0, 1.0 if has else 0.0)]


@dataclass(frozen=True)
class BaseHeightReward(Reward):  # rewards.py:374-385
    height_target: float = 1.0
    kernel_scale: float = 0.25

    def descs(self):
        return [(None, T.REW_BASE_HEIGHT, 0, self.height_target, self.kernel_scale, 0.0)]


@dataclass(frozen=True)
class BaseHeightRangeReward(Reward):  # rewards.py:388-401
    z_lower: float = 0.0
    z_upper: float = 1.0
    dropoff: float = 1.0

    def descs(self):
        return [(None, T.REW_BASE_HEIGHT_RANGE, 0, self.z_lower, self.z_upper, self.dropoff)]


def _norm(n: str) -> int:
    if n not in ("l1", "l2"):
        raise ValueError(f"Invalid norm: {n}")
    return T.NORM_L1 if n == "l1" else T.NORM_L2


@dataclass(frozen=True)
class ActionVelocityPenalty(Reward):  # rewards.py:404-419
    norm: str = "l2"

    def descs(self):
        return [(None, T.REW_ACTION_VEL, _norm(self.norm), 0.0, 0.0, 0.0)]


@dataclass(frozen=True)
class ActionAccelerationPenalty(Reward):  # rewards.py:422-440
    norm: str = "l2"

    def descs(self):
        return [(None, T.REW_ACTION_ACC, _norm(self.norm), 0.0, 0.0, 0.0)]


@dataclass(frozen=True)
class ActionJerkPenalty(Reward):  # rewards.py:443-460
    norm: str = "l2"

    def descs(self):
        return [(None, T.REW_ACTION_JERK, _norm(self.norm), 0.0, 0.0, 0.0)]


@dataclass(frozen=True)
class UprightReward(Reward):  # rewards.py:746-777 — a mapping of three components
    angvel_scale: float = 0.25
    linvel_scale: float = 0.25
    pose_scale: float = 0.25
    angvel_sq_scale: float = 0.1
    angvel_abs_scale: float = 0.1
    linvel_sq_scale: float = 0.1
    linvel_abs_scale: float = 0.1
    pose_sq_scale: float = 0.1
    pose_abs_scale: float = 0.1

    def descs(self):
        return [("angvel", T.REW_UPRIGHT_ANGVEL, 0, self.angvel_scale, self.angvel_sq_scale, self.angvel_abs_scale),
                ("linvel", T.REW_UPRIGHT_LINVEL, 0, self.linvel_scale, self.linvel_sq_scale, self.linvel_abs_scale),
                ("pose", T.REW_UPRIGHT_POSE, 0, self.pose_scale, self.pose_sq_scale, self.pose_abs_scale)]


DISCRIMINATOR_OUTPUT_KEY = "_discriminator_output"  # ksim/task/amp.py:47


@dataclass(frozen=True)
class AMPReward(Reward):  # ksim/task/amp.py:99-112
    """max(0, 1 - 0.25 (logit - 1)^2) of the discriminator logits found in `trajectory.aux_outputs`."""

    def descs(self):
        return [(None, T.REW_AMP, 0, 0.0, 0.0, 0.0)]


def get_rewards(trajectory: Trajectory, rewards: Mapping[str, Reward], clip_min: float | None = None,
                clip_max: float | None = None, want_components: bool = True) -> RewardState:
    """Reward total and components over a (T, N) rollout (ksim/task/rl.py:189-245)."""
    lib = _lib.load()
    done = trajectory.done
    Tn, N = done.shape
    io = T.KsRewardIO()
    io.T, io.N = Tn, N
    names = []
    for name, rew in rewards.items():
        sign = -1.0 if rew.is_penalty else 1.0
        for suffix, kind, norm, p0, p1, p2 in rew.descs():
            j = len(names)
            if j >= T.KS_MAX_REWARD_TERMS:
                raise _lib.KsError("too many reward terms")
            d = io.rewards[j]
            d.kind, d.norm, d.scale, d.p0, d.p1, d.p2 = kind, norm, sign * float(rew.scale), p0, p1, p2
            names.append(name if suffix is None else f"{name}/{suffix}")  # rl.py:223-226
    io.n_rewards = len(names)
    if not names:
        raise _lib.KsError("at least one reward is required")

    def tensor(t, dt, last):
        if t is None:
            return None
        if t.dtype == torch.bool and dt == torch.uint8:
            t = t.view(torch.uint8)
        _lib.require_cuda(t, dtype=dt)
        want = (Tn, N) if last is None else (Tn, N, last)
        if tuple(t.shape) != want:
            raise _lib.KsError(f"trajectory leaf has shape {tuple(t.shape)}, expected {want}")
        return t

    qpos = tensor(trajectory.qpos, torch.float32, None if trajectory.qpos is None else trajectory.qpos.shape[-1])
    qvel = tensor(trajectory.qvel, torch.float32, None if trajectory.qvel is None else trajectory.qvel.shape[-1])
    action = tensor(trajectory.action, torch.float32, None if trajectory.action is None else trajectory.action.shape[-1])
    done_t = tensor(done, torch.uint8, None)
    succ_t = tensor(trajectory.success, torch.uint8, None)
    logits = None
    if any(io.rewards[j].kind == T.REW_AMP for j in range(len(names))):
        if DISCRIMINATOR_OUTPUT_KEY not in trajectory.aux_outputs:  # same failure as amp.py:103-107
            raise ValueError("AMPReward auxiliary output is missing! Make sure you are using it within the context of "
                             "an AMP task, which populates the auxiliary output for you.")
        logits = tensor(trajectory.aux_outputs[DISCRIMINATOR_OUTPUT_KEY], torch.float32, None)
    io.nq = 0 if qpos is None else qpos.shape[-1]
    io.nv = 0 if qvel is None else qvel.shape[-1]
    io.nu = 0 if action is None else action.shape[-1]
    io.use_clip_min, io.clip_min = int(clip_min is not None), float(clip_min or 0.0)
    io.use_clip_max, io.clip_max = int(clip_max is not None), float(clip_max or 0.0)
    total = torch.empty((Tn, N), dtype=torch.float32, device=done.device)
    comps = torch.empty((len(names), Tn, N), dtype=torch.float32, device=done.device) if want_components else None
    io.qpos, io.qvel, io.action = _lib.ptr(qpos).value, _lib.ptr(qvel).value, _lib.ptr(action).value
    io.done, io.success = _lib.ptr(done_t).value, _lib.ptr(succ_t).value
    io.disc_logits = _lib.ptr(logits).value
    io.components, io.total = _lib.ptr(comps).value, _lib.ptr(total).value
    _lib.check(lib.ks_rewards(_lib.current_stream(), ctypes.byref(io)))
    components = {} if comps is None else {n: comps[j] for j, n in enumerate(names)}
    return RewardState(total=total, components=components, carry={})
