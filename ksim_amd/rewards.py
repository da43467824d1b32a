"""Rewards with the reference's class names (ksim/rewards.py) evaluated by the fused reward kernel.

``get_rewards`` mirrors ksim/task/rl.py:189-245: each term times ``scale`` (negated when the class name
ends in ``Penalty``, rewards.py:117-124), summed in dict order, optionally clipped.  Trajectory leaves are
time-major (T, N, ...) tensors.
"""
from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass
from typing import Mapping

import numpy as np
import torch

from . import _lib
from . import _lib_terms as T
from .scales import convert_to_scale
from .types import RewardState, Trajectory


def _reward_scale(rew, level: float) -> float:
    """reward.scale.get_scale(curriculum_level) (rl.py:217): a float is a constant scale."""
    return float(convert_to_scale(rew.scale).get_scale(level))


@dataclass(frozen=True)
class Reward:
    scale: object = 1.0  # a float or a curriculum scale (ksim/scales.py)

    def descs(self) -> list[tuple]:  # [(suffix | None, kind, norm, p0, p1, p2[, p3, index])]  # pragma: no cover
        raise NotImplementedError

    def descs_in(self, obs_slices: Mapping[str, slice], command_slices: Mapping[str, slice]) -> list[tuple]:
        """Descriptors for rewards that read a named command or observation; the others ignore the maps."""
        return self.descs()

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


def _extra(**kw) -> dict:
    """The trailing entry of a descriptor for the kinds with a second index, a count or a table of constants."""
    return kw


@dataclass(frozen=True)
class SmallJointVelocityReward(Reward):  # rewards.py:463-476
    kernel_scale: float = 0.25
    _order = 1

    def descs(self):
        return [(None, T.REW_JOINT_SMOOTH, self._order, self.kernel_scale, 0.0, 0.0)]


@dataclass(frozen=True)
class SmallJointAccelerationReward(SmallJointVelocityReward):  # rewards.py:479-492
    _order = 2


@dataclass(frozen=True)
class SmallJointJerkReward(SmallJointVelocityReward):  # rewards.py:495-509
    _order = 3


@dataclass(frozen=True)
class AvoidLimitsPenalty(Reward):  # rewards.py:521-553
    joint_limits: tuple = ()  # ((lo, hi), ...) one pair per joint behind the floating base

    def __post_init__(self):
        arr = np.asarray(self.joint_limits, dtype=np.float32)
        if arr.ndim != 2 or arr.shape[1] != 2:
            raise ValueError(f"Joint range must have shape (n_joints, 2), got {arr.shape}")
        if not np.all(arr[:, 0] <= arr[:, 1]):
            raise ValueError(f"Joint range must be sorted, got {arr}")

    def descs(self):
        flat = [float(x) for pair in self.joint_limits for x in pair]
        return [(None, T.REW_AVOID_LIMITS, 0, 0.0, 0.0, 0.0, 0.0, 0, _extra(params=flat))]

    @classmethod
    def create(cls, model, factor: float = 0.05, scale=1.0) -> "AvoidLimitsPenalty":
        """Limits widened by factor x range on both sides, none where a joint is not limited (rewards.py:535-553); `model` is a
        `KinematicModel` with a floating base."""
        rng = np.asarray(model.jnt_range, dtype=np.float64)[2:model.nb]   # body 0 is the world, body 1 the base
        lim = np.asarray(model.jnt_limited)[2:model.nb].astype(bool)
        diff = (rng[:, 1] - rng[:, 0]) * factor
        lo = np.where(lim, rng[:, 0] - diff, -np.inf)
        hi = np.where(lim, rng[:, 1] + diff, np.inf)
        return cls(joint_limits=tuple((float(a), float(b)) for a, b in zip(lo, hi)), scale=scale)


@dataclass(frozen=True)
class TorquePenalty(Reward):  # rewards.py:556-581
    ctrl_scales: tuple = ()
    _kind = T.REW_TORQUE

    def descs(self):
        return [(None, self._kind, 0, 0.0, 0.0, 0.0, 0.0, 0, _extra(params=[float(x) for x in self.ctrl_scales]))]

    @classmethod
    def create(cls, model, scale=1.0):
        """Half the width of each actuator's control range (rewards.py:571-581)."""
        cr = np.asarray(model.arrays()["act_ctrlrange"], dtype=np.float64)[:model.nu]
        return cls(ctrl_scales=tuple(float(x) for x in (cr[:, 1] - cr[:, 0]) / 2.0), scale=scale)


@dataclass(frozen=True)
class EnergyPenalty(TorquePenalty):  # rewards.py:584-592
    _kind = T.REW_ENERGY


@dataclass(frozen=True)
class JointDeviationPenalty(Reward):  # rewards.py:595-662
    norm: str = "l2"
    joint_indices: tuple = ()
    joint_targets: tuple = ()
    joint_weights: tuple | None = None

    def descs(self):
        if len(self.joint_indices) != len(self.joint_targets):
            raise ValueError(f"Joint names and targets must match, got {len(self.joint_indices)} and {len(self.joint_targets)}")
        w = self.joint_weights if self.joint_weights is not None else (1.0,) * len(self.joint_indices)
        if len(w) != len(self.joint_indices):
            raise ValueError(f"Joint weights and names must match, got {len(w)} and {len(self.joint_indices)}")
        flat = [float(x) for trip in zip(self.joint_indices, self.joint_targets, w) for x in trip]
        return [(None, T.REW_JOINT_DEVIATION, _norm(self.norm), 0.0, 0.0, 0.0, 0.0, 0, _extra(count=len(self.joint_indices), params=flat))]

    @classmethod
    def create(cls, physics_model, joint_names, joint_targets, scale=1.0, joint_weights=None):
        """Joints are named after the body they move (a `KinematicModel` keeps body names); index = qpos address - 7."""
        names = list(physics_model.body_names)
        idx = tuple(int(physics_model.body_qadr[names.index(n)]) - 7 for n in joint_names)
        return cls(joint_indices=idx, joint_targets=tuple(float(x) for x in joint_targets),
                   joint_weights=None if joint_weights is None else tuple(float(x) for x in joint_weights), scale=scale)


@dataclass(frozen=True)
class FlatBodyReward(Reward):  # rewards.py:665-700
    body_indices: tuple = ()
    plane: tuple = (0.0, 0.0, 1.0)
    norm: str = "l2"

    def descs(self):
        _norm(self.norm)
        flat = [float(b) for b in self.body_indices] + [float(x) for x in self.plane]
        return [(None, T.REW_FLAT_BODY, 0, 0.0, 0.0, 0.0, 0.0, 0, _extra(count=len(self.body_indices), params=flat))]

    @classmethod
    def create(cls, physics_model, body_names, plane=(0.0, 0.0, 1.0), norm="l2", scale=1.0):
        names = list(physics_model.body_names)
        return cls(body_indices=tuple(names.index(n) for n in body_names), plane=tuple(plane), norm=norm, scale=scale)


@dataclass(frozen=True)
class PositionTrackingReward(Reward):  # rewards.py:703-743
    tracked_body_idx: int = 0
    base_body_idx: int = 0
    command_name: str = ""
    body_name: str = ""
    norm: str = "l1"
    kernel_scale: float = 0.25

    def descs(self):  # pragma: no cover
        raise ValueError("PositionTrackingReward reads a named command: pass command_slices to get_rewards")

    def descs_in(self, obs_slices, command_slices):
        sl = _named(command_slices, self.command_name, "command")
        return [(None, T.REW_POSITION_TRACKING, _norm(self.norm), self.kernel_scale, 0.0, 0.0, 0.0, sl.start,
                 _extra(index2=self.tracked_body_idx, count=self.base_body_idx))]

    @classmethod
    def create(cls, model, command_name, tracked_body_name, base_body_name, norm="l1", kernel_scale=0.25, scale=1.0):
        names = list(model.body_names)
        return cls(tracked_body_idx=names.index(tracked_body_name), base_body_idx=names.index(base_body_name), norm=norm,
                   command_name=command_name, body_name=tracked_body_name, scale=scale, kernel_scale=kernel_scale)


@dataclass(frozen=True)
class NoRollReward(Reward):  # rewards.py:778-804 — a mapping of two components
    angvel_scale: float = 0.25
    roll_scale: float = 0.25
    angvel_sq_scale: float = 0.1
    angvel_abs_scale: float = 0.1
    roll_sq_scale: float = 0.1
    roll_abs_scale: float = 0.1

    def descs(self):
        return [("angvel", T.REW_NO_ROLL_ANGVEL, 0, self.angvel_scale, self.angvel_sq_scale, self.angvel_abs_scale),
                ("pose", T.REW_NO_ROLL_POSE, 0, self.roll_scale, self.roll_sq_scale, self.roll_abs_scale)]


@dataclass(frozen=True)
class LinkAccelerationPenalty(Reward):  # rewards.py:807-821
    norm: str = "l2"
    _order = 2

    def descs(self):
        return [(None, T.REW_LINK_SMOOTH, _norm(self.norm), float(self._order), 0.0, 0.0)]


@dataclass(frozen=True)
class LinkJerkPenalty(LinkAccelerationPenalty):  # rewards.py:824-840
    _order = 3


@dataclass(frozen=True)
class FeetSlipPenalty(Reward):  # rewards.py:1088-1105
    contact_obs: str = ""
    velocity_obs: str = ""

    def descs(self):  # pragma: no cover
        raise ValueError("FeetSlipPenalty reads named observations: pass obs_slices to get_rewards")

    def descs_in(self, obs_slices, command_slices):
        c, v = _named(obs_slices, self.contact_obs, "observation"), _named(obs_slices, self.velocity_obs, "observation")
        nv_, nc_ = v.stop - v.start, c.stop - c.start
        if nv_ % 6 != 0 or nv_ == 0 or nc_ % (nv_ // 6) != 0:
            raise ValueError(f"velocity observation of {nv_} entries is not (n, 6) for the {nc_} contact flags")
        n = nv_ // 6
        return [(None, T.REW_FEET_SLIP, n, 0.0, 0.0, 0.0, 0.0, c.start, _extra(index2=v.start, count=nc_ // n))]


@dataclass(frozen=True)
class ReachabilityPenalty(Reward):  # rewards.py:1108-1129
    delta_max_j: tuple = ()
    squared: bool = True

    def descs(self):
        return [(None, T.REW_REACHABILITY, T.NORM_L2 if self.squared else T.NORM_L1, 0.0, 0.0, 0.0, 0.0, 0,
                 _extra(params=[float(x) for x in self.delta_max_j]))]


@dataclass(frozen=True)
class IntersectionPenalty(Reward):  # rewards.py:1417-1430
    position_obs: str = ""
    min_distance: float = 0.0

    def descs(self):  # pragma: no cover
        raise ValueError("IntersectionPenalty reads a named observation: pass obs_slices to get_rewards")

    def descs_in(self, obs_slices, command_slices):
        sl = _named(obs_slices, self.position_obs, "observation")
        if (sl.stop - sl.start) % 3 != 0:
            raise ValueError(f"position observation of {sl.stop - sl.start} entries is not (n, 3)")
        return [(None, T.REW_INTERSECTION, (sl.stop - sl.start) // 3, self.min_distance, 0.0, 0.0, 0.0, sl.start)]


@dataclass(frozen=True)
class SinusoidalGaitReward(Reward):  # rewards.py:1320-1335
    ctrl_dt: float = 0.02
    max_height: float = 0.1
    pos_obs: str = ""
    pos_cmd: str = ""
    num_feet: int = 2

    def descs(self):  # pragma: no cover
        raise ValueError("SinusoidalGaitReward reads a named observation and command: pass obs_slices and command_slices to get_rewards")

    def descs_in(self, obs_slices, command_slices):
        if self.pos_cmd not in command_slices:
            raise ValueError(f"Command {self.pos_cmd} not found! Ensure that it is in the task.")
        ob, cm = _named(obs_slices, self.pos_obs, "observation"), command_slices[self.pos_cmd]
        feet = cm.stop - cm.start - 2
        if ob.stop - ob.start != 3 * feet:
            raise ValueError(f"position observation of {ob.stop - ob.start} entries is not ({feet}, 3) for the command's {feet} feet")
        return [(None, T.REW_SINUSOIDAL_GAIT, feet, self.max_height, 0.0, 0.0, 0.0, ob.start, _extra(index2=cm.start + 2))]


@dataclass(frozen=True)
class JointPositionReward(Reward):  # rewards.py:1352-1380
    """Tracks a joint-position command: "pos" and "vel" are means over the joints of a kernel of (commanded - actual).
    The command named `command_name` is a JointPositionCommandValue (commands.py:795-818) laid out in the command vector as
    [start_position (n), target_position (n), total_time, num_steps, step_id]."""
    command_name: str = ""
    indices: tuple = ()
    pos_scale: float = 0.25
    vel_scale: float = 0.25
    sq_scale: float = 0.1
    abs_scale: float = 0.1

    def descs(self):  # pragma: no cover
        raise ValueError("JointPositionReward reads a named command: pass command_slices to get_rewards")

    def descs_in(self, obs_slices, command_slices):
        if self.command_name not in command_slices:
            raise ValueError(f"Command {self.command_name} not found! Ensure that it is in the task.")
        if not (self.sq_scale > 0.0 and self.abs_scale > 0.0):
            raise ValueError("sq_scale and abs_scale must be positive")
        cm, n = command_slices[self.command_name], len(self.indices)
        if cm.stop - cm.start != 2 * n + 3:
            raise ValueError(f"the command holds {cm.stop - cm.start} numbers, a joint-position command of {n} joints holds {2 * n + 3}")
        idx = [float(i) for i in self.indices]
        return [("pos", T.REW_JOINT_POSITION, 0, self.pos_scale, self.sq_scale, self.abs_scale, 0.0, cm.start, _extra(count=n, params=idx)),
                ("vel", T.REW_JOINT_VELOCITY_CMD, 0, self.vel_scale, self.sq_scale, self.abs_scale, 0.0, cm.start, _extra(count=n, params=idx))]

    @classmethod
    def create(cls, physics_model, joint_names, command_name, pos_scale=0.25, vel_scale=0.25, sq_scale=0.1, abs_scale=0.1, scale=1.0):
        names = list(physics_model.body_names)
        for n in joint_names:
            if n not in names:
                raise ValueError(f"Joint {n} not found in the model! Options are: {names[1:]}")
        idx = tuple(int(physics_model.body_qadr[names.index(n)]) - 7 for n in joint_names)
        return cls(command_name=command_name, indices=idx, pos_scale=pos_scale, vel_scale=vel_scale, sq_scale=sq_scale,
                   abs_scale=abs_scale, scale=scale)


DISCRIMINATOR_OUTPUT_KEY = "_discriminator_output"  # ksim/task/amp.py:47


@dataclass(frozen=True)
class AMPReward(Reward):  # ksim/task/amp.py:99-112
    """max(0, 1 - 0.25 (logit - 1)^2) of the discriminator logits found in `trajectory.aux_outputs`."""

    def descs(self):
        return [(None, T.REW_AMP, 0, 0.0, 0.0, 0.0)]


def _named(slices, name, what):
    if name not in slices:
        raise KeyError(f"{what} {name!r} is not among {sorted(slices)}")
    return slices[name]


@dataclass(frozen=True)
class LinearVelocityReward(Reward):
    """Tracks a planar velocity command in the robot frame (rewards.py:236-275): components vel, yaw, x, y.  The command is
    the LinearVelocityCommandValue laid out as (vel, yaw, xvel, yvel, ...) at `command_slices[cmd]`."""
    cmd: str = ""
    vel_length_scale: float = 0.25
    yaw_length_scale: float = 0.25
    zero_threshold: float = 0.01
    sq_scale: float = 0.1
    abs_scale: float = 0.1

    def __post_init__(self):
        if not (self.sq_scale > 0.0 and self.abs_scale > 0.0):
            raise ValueError("sq_scale and abs_scale must be positive")

    def descs_in(self, obs_slices, command_slices):
        sl = _named(command_slices, self.cmd, "command")
        if sl.stop - sl.start < 4:
            raise ValueError("a linear velocity command has at least (vel, yaw, xvel, yvel)")
        return [(name, T.REW_LINVEL_CMD, k, self.yaw_length_scale if k == 1 else self.vel_length_scale, self.sq_scale,
                 self.abs_scale, self.zero_threshold, sl.start) for k, name in enumerate(("vel", "yaw", "x", "y"))]


@dataclass(frozen=True)
class AngularVelocityReward(Reward):
    """Tracks a yaw-rate command (rewards.py:321-350): components mag and dir."""
    cmd: str = ""
    angvel_length_scale: float = 0.25
    sq_scale: float = 0.1
    abs_scale: float = 0.1
    zero_threshold: float = math.radians(5.0)

    def __post_init__(self):
        if not (self.sq_scale > 0.0 and self.abs_scale > 0.0):
            raise ValueError("sq_scale and abs_scale must be positive")

    def descs_in(self, obs_slices, command_slices):
        sl = _named(command_slices, self.cmd, "command")
        return [(name, T.REW_ANGVEL_CMD, k, self.angvel_length_scale, self.sq_scale, self.abs_scale, self.zero_threshold, sl.start)
                for k, name in enumerate(("mag", "dir"))]


@dataclass(frozen=True)
class OffAxisVelocityReward(Reward):  # rewards.py:353-372: components linz, angx, angy (qvel[2], qvel[4], qvel[5])
    lin_length_scale: float = 0.25
    ang_length_scale: float = 0.25

    def descs(self):
        return [("linz", T.REW_OFF_AXIS, 0, self.lin_length_scale, 0.0, 0.0), ("angx", T.REW_OFF_AXIS, 1, self.ang_length_scale, 0.0, 0.0),
                ("angy", T.REW_OFF_AXIS, 2, self.ang_length_scale, 0.0, 0.0)]


@dataclass(frozen=True)
class MotionlessAtRestPenalty(Reward):  # rewards.py:1206-1221: joint speed while the base is not moving
    linvel_moving_threshold: float = 0.5
    angvel_moving_threshold: float = math.radians(30)

    def descs(self):
        return [(None, T.REW_MOTIONLESS, 0, self.linvel_moving_threshold, self.angvel_moving_threshold, 0.0)]


@dataclass(frozen=True)
class ForcePenalty(Reward):
    """Squared contact force over the expected weight, worst body (rewards.py:1224-1240); `force_obs` names an (n, 3)
    observation such as FeetForceObservation."""
    force_obs: str = ""
    ctrl_dt: float = 0.02
    expected_weight: float = 1.0
    bias: float = 0.0

    def descs_in(self, obs_slices, command_slices):
        sl = _named(obs_slices, self.force_obs, "observation")
        if (sl.stop - sl.start) % 3:
            raise ValueError("the force observation must be (n, 3)")
        return [(None, T.REW_FORCE, (sl.stop - sl.start) // 3, self.expected_weight, self.bias, 0.0, 0.0, sl.start)]


@dataclass(frozen=True)
class StatefulReward(Reward):
    """Rewards that scan the rollout with a per-env carry (rewards.py:127-163); evaluated by `ks_reward_scan`."""

    def carry_size(self) -> int:  # pragma: no cover
        raise NotImplementedError

    def n_slots(self) -> int:  # pragma: no cover
        raise NotImplementedError

    def suffixes(self) -> tuple:
        return (None,)

    def initial_carry(self) -> tuple:
        """The carry an env starts with, and restarts with when its rollout ended on a done step (rl.py:206-214)."""
        return (0.0,) * self.carry_size()

    def scan_desc(self, obs_slices: Mapping[str, slice], command_slices: Mapping[str, slice], level: float) -> T.KsRewardScanDesc:
        raise NotImplementedError  # pragma: no cover


def _block(obs_slices, name, what):
    if name not in obs_slices:
        raise KeyError(f"{what} observation {name!r} is not among the observations: {sorted(obs_slices)}")
    return obs_slices[name]


@dataclass(frozen=True)
class FeetAirTimeReward(StatefulReward):  # rewards.py:992-1085
    gait_period: object = 1.0   # a float or a curriculum scale
    air_time_percent: float = 0.5
    ctrl_dt: float = 0.02
    contact_obs: str = ""
    num_feet: int = 2
    bias: float = 0.0
    alpha: float = 0.1
    ground_penalty: float = 0.1
    linvel_moving_threshold: float = 0.1
    angvel_moving_threshold: float = math.radians(10)
    linvel_cmd: str | None = None
    angvel_cmd: str | None = None

    def carry_size(self):
        return 3 * self.num_feet  # air, ground and stationary-ground step counters per foot

    def n_slots(self):
        return 3

    def suffixes(self):
        return ("air", "gnd", "stationary_gnd")

    def scan_desc(self, obs_slices, command_slices, level):
        sl = _block(obs_slices, self.contact_obs, "contact")
        width = sl.stop - sl.start
        if width % self.num_feet:
            raise ValueError(f"contact observation has {width} entries, not a multiple of {self.num_feet} feet")
        f32 = np.float32
        period = f32(convert_to_scale(self.gait_period).get_scale(level))
        d = T.KsRewardScanDesc()
        d.kind, d.n, d.n_contact, d.contact_index = T.SCAN_FEET_AIR_TIME, self.num_feet, width // self.num_feet, sl.start
        # rewards.py:1049-1050, in float32 like the reference; numpy rounds half to even like jnp.round
        d.air_steps = float(np.round(period * f32(self.air_time_percent) / f32(self.ctrl_dt)))
        d.gnd_steps = float(np.round(period * f32(1.0 - self.air_time_percent) / f32(self.ctrl_dt)))
        d.bias, d.ground_penalty = self.bias, self.ground_penalty
        d.linvel_threshold, d.angvel_threshold = self.linvel_moving_threshold, self.angvel_moving_threshold
        for field_, cmd in (("linvel_cmd_index", self.linvel_cmd), ("angvel_cmd_index", self.angvel_cmd)):
            if cmd is None:
                setattr(d, field_, -1)
            else:
                if cmd not in command_slices:
                    raise KeyError(f"command {cmd!r} is not among the commands: {sorted(command_slices)}")
                setattr(d, field_, command_slices[cmd].start)
        return d


@dataclass(frozen=True)
class SparseTargetHeightReward(StatefulReward):  # rewards.py:1148-1192
    contact_obs: str = ""
    position_obs: str = ""
    height: float = 0.0
    num_bodies: int = 2
    linvel_moving_threshold: float = 0.5
    angvel_moving_threshold: float = math.radians(30)

    def carry_size(self):
        return self.num_bodies  # highest point of each body since it last touched down

    def n_slots(self):
        return 1

    def scan_desc(self, obs_slices, command_slices, level):
        sl, ps = _block(obs_slices, self.contact_obs, "contact"), _block(obs_slices, self.position_obs, "position")
        width = sl.stop - sl.start
        if width % self.num_bodies or ps.stop - ps.start != 3 * self.num_bodies:
            raise ValueError("contact / position observations do not match num_bodies")
        d = T.KsRewardScanDesc()
        d.kind, d.n, d.n_contact = T.SCAN_SPARSE_TARGET_HEIGHT, self.num_bodies, width // self.num_bodies
        d.contact_index, d.position_index, d.height = sl.start, ps.start, self.height
        d.linvel_threshold, d.angvel_threshold = self.linvel_moving_threshold, self.angvel_moving_threshold
        d.linvel_cmd_index = d.angvel_cmd_index = -1
        return d


@dataclass(frozen=True)
class SymmetryReward(StatefulReward):  # rewards.py:843-896
    """With x = qpos[7 + joint] - target: the carry follows the rollout's mean x with rate alpha (once per rollout), and the
    reward is -sum_j x_j carry_j, which pushes each joint away from the side it has been leaning to."""
    joint_indices: tuple = ()
    joint_targets: tuple = ()
    alpha: float = 0.1

    def carry_size(self):
        return len(self.joint_indices)

    def n_slots(self):
        return 1

    def initial_carry(self):
        return tuple(float(x) for x in self.joint_targets)  # rewards.py:865-866

    def scan_desc(self, obs_slices, command_slices, level):
        n = len(self.joint_indices)
        if n != len(self.joint_targets):
            raise ValueError(f"Joint names and targets must match, got {n} and {len(self.joint_targets)}")
        if not 1 <= n <= T.KS_MAX_SCAN_JOINTS:
            raise ValueError(f"1..{T.KS_MAX_SCAN_JOINTS} joints, got {n}")
        d = T.KsRewardScanDesc()
        d.kind, d.n, d.alpha = T.SCAN_SYMMETRY, n, self.alpha
        for k, (j, t) in enumerate(zip(self.joint_indices, self.joint_targets)):
            d.joints[k], d.targets[k] = int(j), float(t)
        return d

    @classmethod
    def create(cls, physics_model, joint_names, joint_targets, alpha=0.1, scale=1.0):
        names = list(physics_model.body_names)
        idx = tuple(int(physics_model.body_qadr[names.index(n)]) - 7 for n in joint_names)
        if len(joint_names) != len(joint_targets):
            raise ValueError(f"Joint names and targets must match, got {len(joint_names)} and {len(joint_targets)}")
        return cls(joint_indices=idx, joint_targets=tuple(float(x) for x in joint_targets), alpha=alpha, scale=scale)


@dataclass(frozen=True)
class PairwiseSymmetryReward(StatefulReward):  # rewards.py:899-936
    """Two terms for a left / right pair of joints (each minus its zero, the right one negated when `flipped`): "lr", a
    kernel of their difference, and "self", the SymmetryReward of the pair."""
    left_joint_index: int = 0
    right_joint_index: int = 0
    left_zero: float = 0.0
    right_zero: float = 0.0
    flipped: bool = False
    alpha: float = 0.1
    kernel_scale: float = 0.25
    sq_scale: float = 0.1
    abs_scale: float = 0.1

    def carry_size(self):
        return 2

    def n_slots(self):
        return 2

    def suffixes(self):
        return ("lr", "self")

    def initial_carry(self):
        return (float(self.left_zero), float(self.right_zero))  # rewards.py:913-914

    def scan_desc(self, obs_slices, command_slices, level):
        if not (self.sq_scale > 0.0 and self.abs_scale > 0.0):
            raise ValueError("sq_scale and abs_scale must be positive")
        d = T.KsRewardScanDesc()
        d.kind, d.n, d.alpha, d.flipped = T.SCAN_PAIRWISE_SYMMETRY, 2, self.alpha, int(self.flipped)
        d.joints[0], d.joints[1] = int(self.left_joint_index), int(self.right_joint_index)
        d.targets[0], d.targets[1] = float(self.left_zero), float(self.right_zero)
        d.kernel_scale, d.sq_scale, d.abs_scale = self.kernel_scale, self.sq_scale, self.abs_scale
        return d

    @classmethod
    def create(cls, physics_model, left_joint_name, right_joint_name, left_zero=0.0, right_zero=0.0, flipped=False, alpha=0.1,
               kernel_scale=0.25, sq_scale=0.1, abs_scale=0.1, scale=1.0):
        names = list(physics_model.body_names)
        li, ri = (int(physics_model.body_qadr[names.index(n)]) - 7 for n in (left_joint_name, right_joint_name))
        return cls(left_joint_index=li, right_joint_index=ri, left_zero=left_zero, right_zero=right_zero, flipped=flipped,
                   alpha=alpha, kernel_scale=kernel_scale, sq_scale=sq_scale, abs_scale=abs_scale, scale=scale)


def reward_carry_size(rewards: Mapping[str, Reward]) -> int:
    return sum(r.carry_size() for r in rewards.values() if isinstance(r, StatefulReward))


def initial_reward_carry(rewards: Mapping[str, Reward], num_envs: int, device) -> torch.Tensor | None:
    """(N, reward_carry_size) filled with every stateful reward's initial carry, or None without stateful rewards."""
    row = [x for r in rewards.values() if isinstance(r, StatefulReward) for x in r.initial_carry()]
    if not row:
        return None
    return torch.tensor(row, dtype=torch.float32, device=device).repeat(int(num_envs), 1).contiguous()


def _scan_stateful(trajectory, rewards, rewards_carry, obs_slices, command_slices, obs_key, level, Tn, N):
    """Runs `ks_reward_scan` over the stateful terms; returns (values (n_slots, T, N), first slot per reward name)."""
    stateful = {n: r for n, r in rewards.items() if isinstance(r, StatefulReward)}
    if len(stateful) > T.KS_MAX_REWARD_SCANS:
        raise _lib.KsError(f"at most {T.KS_MAX_REWARD_SCANS} stateful rewards")
    reads_obs = any(not isinstance(r, (SymmetryReward, PairwiseSymmetryReward)) for r in stateful.values())
    io = T.KsRewardScanIO()
    io.T, io.N, io.nv = Tn, N, trajectory.qvel.shape[-1]
    obs = None
    if reads_obs:
        if obs_slices is None:
            raise _lib.KsError("stateful rewards read named observations: pass obs_slices (EnvTerms.obs_slices)")
        obs = trajectory.obs[obs_key]
        _lib.require_cuda(obs, dtype=torch.float32)
        if obs.dim() != 3 or tuple(obs.shape[:2]) != (Tn, N):
            raise _lib.KsError(f"observation leaf has shape {tuple(obs.shape)}, expected ({Tn}, {N}, obs_dim)")
        io.obs_dim, io.obs = obs.shape[-1], obs.data_ptr()
    _lib.require_cuda(trajectory.qpos, dtype=torch.float32)
    io.qpos, io.nq = trajectory.qpos.data_ptr(), trajectory.qpos.shape[-1]
    dev = trajectory.qpos.device
    slots, carry_at, first = 0, 0, {}
    for j, (name, r) in enumerate(stateful.items()):
        d = r.scan_desc(obs_slices, command_slices or {}, level)
        d.slot, d.carry_index = slots, carry_at
        io.scans[j] = d
        first[name] = slots
        slots += r.n_slots()
        carry_at += r.carry_size()
    io.n_scans, io.n_slots, io.carry_dim = len(stateful), slots, carry_at
    if rewards_carry is None:
        rewards_carry = initial_reward_carry(rewards, N, dev)
    _lib.require_cuda(rewards_carry, dtype=torch.float32)
    if tuple(rewards_carry.shape) != (N, carry_at):
        raise _lib.KsError(f"reward carry has shape {tuple(rewards_carry.shape)}, expected {(N, carry_at)}")
    cmd = trajectory.command.get("_buffer") if trajectory.command else None
    if cmd is not None:
        _lib.require_cuda(cmd, dtype=torch.float32)
        if cmd.dim() != 3 or tuple(cmd.shape[:2]) != (Tn, N):
            raise _lib.KsError(f"command leaf has shape {tuple(cmd.shape)}, expected ({Tn}, {N}, command_dim)")
        io.command_dim, io.command = cmd.shape[-1], cmd.data_ptr()
    out = torch.empty((slots, Tn, N), dtype=torch.float32, device=dev)
    done = trajectory.done.view(torch.uint8) if trajectory.done.dtype == torch.bool else trajectory.done
    io.qvel, io.done = trajectory.qvel.data_ptr(), done.data_ptr()
    io.carry, io.out = rewards_carry.data_ptr(), out.data_ptr()
    _lib.check(_lib.load().ks_reward_scan(_lib.current_stream(), ctypes.byref(io)))
    return out, first, rewards_carry


def get_rewards(trajectory: Trajectory, rewards: Mapping[str, Reward], clip_min: float | None = None,
                clip_max: float | None = None, want_components: bool = True, *, rewards_carry: torch.Tensor | None = None,
                obs_slices: Mapping[str, slice] | None = None, command_slices: Mapping[str, slice] | None = None,
                obs_key: str = "obs", level: float = 1.0) -> RewardState:
    """Reward total and components over a (T, N) rollout (ksim/task/rl.py:189-245).

    Stateful rewards read their observations by name out of the concatenated vector `trajectory.obs[obs_key]`
    (`obs_slices` maps names to columns) and advance `rewards_carry` (N, reward_carry_size(rewards)) in place; the
    returned state holds it under `carry["_buffer"]`.  Commands for them come as `trajectory.command["_buffer"]`
    (T, N, command_dim) with `command_slices`."""
    lib = _lib.load()
    done = trajectory.done
    Tn, N = done.shape
    io = T.KsRewardIO()
    io.T, io.N = Tn, N
    names = []
    n_params = 0
    scanned, first_slot = None, {}
    if any(isinstance(r, StatefulReward) for r in rewards.values()):
        scanned, first_slot, rewards_carry = _scan_stateful(trajectory, rewards, rewards_carry, obs_slices, command_slices,
                                                           obs_key, float(level), Tn, N)
        io.stateful = scanned.data_ptr()
    for name, rew in rewards.items():
        sign = -1.0 if rew.is_penalty else 1.0
        if isinstance(rew, StatefulReward):
            for k, suffix in enumerate(rew.suffixes()):
                j = len(names)
                if j >= T.KS_MAX_REWARD_TERMS:
                    raise _lib.KsError("too many reward terms")
                d = io.rewards[j]
                d.kind, d.norm, d.scale = T.REW_STATEFUL, first_slot[name] + k, sign * _reward_scale(rew, level)
                names.append(name if suffix is None else f"{name}/{suffix}")
            continue
        for suffix, kind, norm, p0, p1, p2, *more in rew.descs_in(obs_slices or {}, command_slices or {}):
            j = len(names)
            if j >= T.KS_MAX_REWARD_TERMS:
                raise _lib.KsError("too many reward terms")
            d = io.rewards[j]
            d.kind, d.norm, d.scale, d.p0, d.p1, d.p2 = kind, norm, sign * _reward_scale(rew, level), p0, p1, p2
            if more:
                d.p3, d.index = float(more[0]), int(more[1])
            if len(more) >= 3:
                ex = more[2]
                d.index2, d.count = int(ex.get("index2", 0)), int(ex.get("count", 0))
                pr = ex.get("params")
                if pr is not None:
                    if n_params + len(pr) > T.KS_MAX_REWARD_PARAMS:
                        raise _lib.KsError(f"the rewards' constants exceed the table of {T.KS_MAX_REWARD_PARAMS} entries")
                    d.param_offset = n_params
                    for x in pr:
                        io.params[n_params] = x
                        n_params += 1
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
    kinds = {io.rewards[j].kind for j in range(len(names))}
    io.n_params = n_params
    if kinds & {T.REW_TORQUE, T.REW_ENERGY}:
        if trajectory.ctrl is None:
            raise _lib.KsError("torque and energy penalties read trajectory.ctrl")
        ctrl = tensor(trajectory.ctrl, torch.float32, trajectory.ctrl.shape[-1])
        io.ctrl = ctrl.data_ptr()
        if action is not None and ctrl.shape[-1] != action.shape[-1]:
            raise _lib.KsError("trajectory.ctrl and trajectory.action differ in width")
        nu_ctrl = ctrl.shape[-1]
    else:
        nu_ctrl = None
    if kinds & {T.REW_FLAT_BODY, T.REW_POSITION_TRACKING, T.REW_LINK_SMOOTH}:
        for leaf, per, name in ((trajectory.xpos, 3, "xpos"), (trajectory.xquat, 4, "xquat")):
            if leaf is None:
                continue
            flat = leaf.reshape(Tn, N, -1) if leaf.dim() == 4 else leaf
            flat = tensor(flat, torch.float32, flat.shape[-1])
            if flat.shape[-1] % per != 0 or (io.nb and io.nb != flat.shape[-1] // per):
                raise _lib.KsError(f"trajectory.{name} has {flat.shape[-1]} entries per step: not (nb, {per}) for the other leaf's nb")
            io.nb = flat.shape[-1] // per
            setattr(io, name, flat.data_ptr())
    if kinds & {T.REW_LINVEL_CMD, T.REW_ANGVEL_CMD, T.REW_POSITION_TRACKING, T.REW_SINUSOIDAL_GAIT, T.REW_JOINT_POSITION,
                T.REW_JOINT_VELOCITY_CMD}:
        cmd = trajectory.command.get("_buffer") if trajectory.command else None
        if cmd is None:
            raise KeyError('command-tracking rewards read trajectory.command["_buffer"] (T, N, command_dim)')
        cmd = tensor(cmd, torch.float32, cmd.shape[-1])
        io.command, io.command_dim = cmd.data_ptr(), cmd.shape[-1]
    if kinds & {T.REW_FORCE, T.REW_FEET_SLIP, T.REW_INTERSECTION, T.REW_SINUSOIDAL_GAIT}:
        ob_ = trajectory.obs[obs_key]
        ob_ = tensor(ob_, torch.float32, ob_.shape[-1])
        io.obs, io.obs_dim = ob_.data_ptr(), ob_.shape[-1]
    io.nq = 0 if qpos is None else qpos.shape[-1]
    io.nv = 0 if qvel is None else qvel.shape[-1]
    io.nu = (nu_ctrl or 0) if action is None else action.shape[-1]
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
    return RewardState(total=total, components=components, carry={} if rewards_carry is None else {"_buffer": rewards_carry})
