"""Commands with the reference's class names (ksim/commands.py), advanced once per control step on the device.

`CommandSet` lays the commands' values out in one `(N, command_dim)` vector per env (`slices[name]` says where) and
replaces get_initial_commands / get_commands (ksim/task/rl.py:302-332): an env that starts an episode draws an initial
command from its reset state, the others are updated.  A velocity command's value is the reference's dataclass flattened:
`LinearVelocityCommandValue` = (vel, yaw, xvel, yvel, target_vel, target_yaw), `AngularVelocityCommandValue` = (vel, target_vel).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Mapping

import torch

from . import _lib
from . import _lib_terms as T
from .scales import convert_to_scale


@dataclass(frozen=True)
class Command:
    def dim(self) -> int:  # pragma: no cover
        raise NotImplementedError

    def desc(self, level: float) -> T.KsCommandDesc:  # pragma: no cover
        raise NotImplementedError


def _s(scale, level: float) -> float:
    return float(convert_to_scale(scale).get_scale(level))


@dataclass(frozen=True)
class LinearVelocityCommand(Command):  # commands.py:281-391
    min_vel: object = 0.0
    max_vel: object = 0.0
    ctrl_dt: float = 0.02
    linear_accel: float = 1.0
    angular_accel: float = 1.0
    max_yaw: object = 0.0
    zero_prob: object = 0.0
    backward_prob: object = 0.0
    switch_prob: object = 0.0

    def dim(self):
        return 6

    def desc(self, level):
        d = T.KsCommandDesc()
        d.kind, d.dim = T.CMD_LINEAR_VELOCITY, 6
        d.min_vel, d.max_vel, d.max_yaw = _s(self.min_vel, level), _s(self.max_vel, level), _s(self.max_yaw, level)
        d.zero_prob, d.backward_prob, d.switch_prob = _s(self.zero_prob, level), _s(self.backward_prob, level), _s(self.switch_prob, level)
        d.ctrl_dt, d.linear_accel, d.angular_accel = self.ctrl_dt, self.linear_accel, self.angular_accel
        return d


@dataclass(frozen=True)
class AngularVelocityCommand(Command):  # commands.py:451-507
    max_vel: object = 0.0
    ctrl_dt: float = 0.02
    angular_accel: float = 1.0
    min_vel: object = 0.0
    zero_prob: object = 0.0
    switch_prob: object = 0.0

    def dim(self):
        return 2

    def desc(self, level):
        d = T.KsCommandDesc()
        d.kind, d.dim = T.CMD_ANGULAR_VELOCITY, 2
        d.min_vel, d.max_vel = _s(self.min_vel, level), _s(self.max_vel, level)
        d.zero_prob, d.switch_prob = _s(self.zero_prob, level), _s(self.switch_prob, level)
        d.ctrl_dt, d.angular_accel = self.ctrl_dt, self.angular_accel
        return d


@dataclass(frozen=True)
class ConstantCommand(Command):
    """`size` floats that the task sets itself and that no step changes."""
    size: int = 1

    def dim(self):
        return int(self.size)

    def desc(self, level):
        d = T.KsCommandDesc()
        d.kind, d.dim = T.CMD_CONST, int(self.size)
        return d


@dataclass(frozen=True)
class FloatVectorCommand(Command):  # commands.py:97-133
    ranges: tuple = ()
    switch_prob: float = 0.0
    zero_prob: float = 0.0
    _kind = T.CMD_FLOAT_VECTOR

    def __post_init__(self):
        if not 1 <= len(self.ranges) <= T.KS_MAX_VECTOR_COMMAND:
            raise ValueError(f"a vector command has 1..{T.KS_MAX_VECTOR_COMMAND} scalars")

    def dim(self):
        return len(self.ranges)

    def desc(self, level):
        d = T.KsCommandDesc()
        d.kind, d.dim, d.switch_prob, d.zero_prob = self._kind, len(self.ranges), float(self.switch_prob), float(self.zero_prob)
        for j, (lo, hi) in enumerate(self.ranges):
            d.lo[j], d.hi[j] = float(lo), float(hi)
        return d


@dataclass(frozen=True)
class IntVectorCommand(FloatVectorCommand):  # commands.py:136-170: integers lo..hi inclusive, stored as floats
    _kind = T.CMD_INT_VECTOR


@dataclass(frozen=True)
class StartPositionCommand(Command):  # commands.py:173-192: where the episode started
    _kind, _dim = T.CMD_START_POSITION, 3

    def dim(self):
        return self._dim

    def desc(self, level):
        d = T.KsCommandDesc()
        d.kind, d.dim = self._kind, self._dim
        return d


@dataclass(frozen=True)
class StartQuaternionCommand(StartPositionCommand):  # commands.py:195-215: the orientation the episode started with
    _kind, _dim = T.CMD_START_QUATERNION, 4


@dataclass(frozen=True)
class BaseHeightCommand(Command):  # commands.py:773-796
    min_height: float = 0.0
    max_height: float = 1.0
    switch_prob: float = 0.005

    def dim(self):
        return 1

    def desc(self, level):
        d = T.KsCommandDesc()
        d.kind, d.dim, d.switch_prob = T.CMD_BASE_HEIGHT, 1, float(self.switch_prob)
        d.lo[0], d.hi[0] = float(self.min_height), float(self.max_height)
        return d


@dataclass(frozen=True)
class SinusoidalGaitCommand(Command):  # commands.py:696-770: layout moving_flag, phase, height per foot
    gait_period: float = 1.0
    ctrl_dt: float = 0.02
    max_height: float = 0.1
    height_offset: float = 0.0
    num_feet: int = 2
    stance_ratio: float = 0.6
    moving_threshold: float = 0.05

    def dim(self):
        return 2 + self.num_feet

    def desc(self, level):
        d = T.KsCommandDesc()
        d.kind, d.dim, d.ctrl_dt = T.CMD_SINUSOIDAL_GAIT, 2 + self.num_feet, float(self.ctrl_dt)
        for j, x in enumerate((self.gait_period, self.max_height, self.height_offset, self.stance_ratio, self.moving_threshold)):
            d.lo[j] = float(x)
        return d


@dataclass(frozen=True)
class JointPositionCommand(Command):  # commands.py:821-914; the value is JointPositionCommandValue flattened
    """start (n), target (n), total_time, num_steps, step_id: JointPositionReward reads this layout."""

    indices: tuple = ()   # actuated-joint indices (joint order without the floating base)
    ranges: tuple = ()    # (lo, hi) per joint
    ctrl_dt: float = 0.02
    min_time: float = 0.1
    max_time: float = 1.0

    def __post_init__(self):
        if not 1 <= len(self.indices) <= T.KS_MAX_VECTOR_COMMAND or len(self.ranges) != len(self.indices):
            raise ValueError(f"a joint position command takes 1..{T.KS_MAX_VECTOR_COMMAND} joints and one range for each")
        if not (self.min_time > 0.0 and self.max_time > 0.0):
            raise ValueError("min_time and max_time must be positive")

    @classmethod
    def create(cls, model, ctrl_dt: float, joint_names, min_time: float = 0.1, max_time: float = 1.0):
        """By name, with the joints' own ranges as the target ranges (commands.py:895-914).  A hinge is named after the body
        it moves (every body here carries at most one joint)."""
        names = list(model.body_names)
        idx, ranges = [], []
        for name in joint_names:
            if name not in names or int(model.body_qadr[names.index(name)]) < 7:
                raise ValueError(f"Joint {name} not found in the model! Options are: {[n for n in names if int(model.body_qadr[names.index(n)]) >= 7]}")
            b = names.index(name)
            idx.append(int(model.body_qadr[b]) - 7)
            ranges.append((float(model.jnt_range[b][0]), float(model.jnt_range[b][1])))
        return cls(indices=tuple(idx), ranges=tuple(ranges), ctrl_dt=ctrl_dt, min_time=min_time, max_time=max_time)

    def dim(self):
        return 2 * len(self.indices) + 3

    def desc(self, level):
        d = T.KsCommandDesc()
        d.kind, d.dim, d.ctrl_dt = T.CMD_JOINT_POSITION, self.dim(), float(self.ctrl_dt)
        d.min_time, d.max_time = float(self.min_time), float(self.max_time)
        for j, (i, (lo, hi)) in enumerate(zip(self.indices, self.ranges)):
            d.joints[j], d.lo[j], d.hi[j] = int(i), float(lo), float(hi)
        return d


@dataclass(frozen=True)
class CartesianCoordinateCommand(Command):  # commands.py:537-694; the value is current (3), target (3), speed
    box_min: tuple = (0.0, 0.0, 0.0)
    box_max: tuple = (0.0, 0.0, 0.0)
    dt: float = 0.02
    min_speed: float = 0.5
    max_speed: float = 3.0
    switch_prob: float = 0.0
    jump_prob: float = 0.0
    curriculum_scale: float = 0.1

    def dim(self):
        return 7

    def desc(self, level):
        d = T.KsCommandDesc()
        d.kind, d.dim, d.ctrl_dt = T.CMD_CARTESIAN_COORDINATE, 7, float(self.dt)
        d.min_vel, d.max_vel, d.switch_prob, d.jump_prob = float(self.min_speed), float(self.max_speed), float(self.switch_prob), float(self.jump_prob)
        grow = self.curriculum_scale * float(level) + 1.0  # the box grows about its centre with the level (commands.py:561-572)
        for j in range(3):
            centre, half = 0.5 * (self.box_min[j] + self.box_max[j]), 0.5 * (self.box_max[j] - self.box_min[j])
            d.lo[j], d.hi[j] = centre - half * grow, centre + half * grow
        return d


class CommandSet:
    def __init__(self, commands: Mapping[str, Command]):
        if len(commands) > T.KS_MAX_COMMANDS:
            raise ValueError(f"at most {T.KS_MAX_COMMANDS} commands")
        self.commands = dict(commands)
        self.slices: dict[str, slice] = {}
        at = 0
        for name, c in self.commands.items():
            self.slices[name] = slice(at, at + c.dim())
            at += c.dim()
        self.command_dim = at
        self._lib = _lib.load()

    def initial(self, num_envs: int, device="cuda") -> torch.Tensor:
        """A zeroed command vector; the first `update(..., all_fresh=True)` draws the initial commands."""
        return torch.zeros(num_envs, self.command_dim, dtype=torch.float32, device=device)

    def update(self, command: torch.Tensor, qpos: torch.Tensor, qvel: torch.Tensor, *, level: float = 1.0,
               fresh: torch.Tensor | None = None, all_fresh: bool = False, record: torch.Tensor | None = None,
               uniform: torch.Tensor | None = None, seed: int = 0, step: int = 0, step_base=None) -> torch.Tensor:
        """Advances every env's commands in place; `record` (N, command_dim) receives the incoming values."""
        N = command.shape[0]
        _lib.require_cuda(command, qpos, qvel, record, uniform, dtype=torch.float32)
        if qpos.dim() != 2 or qvel.dim() != 2 or tuple(command.shape) != (N, self.command_dim) or qpos.shape[0] != N or qvel.shape[0] != N:
            raise _lib.KsError(f"command must be (N, {self.command_dim}) and the state must have N rows")
        if record is not None and tuple(record.shape) != tuple(command.shape):
            raise _lib.KsError("record must have the command's shape")
        if uniform is not None and tuple(uniform.shape) != (N, len(self.commands), T.KS_COMMAND_DRAWS):
            raise _lib.KsError(f"uniform must be (N, {len(self.commands)}, {T.KS_COMMAND_DRAWS})")
        io = T.KsCommandIO()
        io.N, io.command_dim, io.n_commands, io.nq, io.nv = N, self.command_dim, len(self.commands), qpos.shape[1], qvel.shape[1]
        for k, (name, c) in enumerate(self.commands.items()):
            d = c.desc(float(level))
            d.index = self.slices[name].start
            io.commands[k] = d
        io.command, io.traj_command = command.data_ptr(), _lib.ptr(record).value
        io.qpos, io.qvel = qpos.data_ptr(), qvel.data_ptr()
        if fresh is not None:
            _lib.require_cuda(fresh, dtype=torch.uint8)
            if tuple(fresh.shape) != (N,):
                raise _lib.KsError("fresh must be (N,) uint8")
            io.fresh = fresh.data_ptr()
        io.all_fresh, io.uniform = int(bool(all_fresh)), _lib.ptr(uniform).value
        if step_base is not None:
            _lib.require_cuda(step_base, dtype=torch.int64)
        io.rng = T.KsRng(int(seed) & (2**64 - 1), int(step) & (2**64 - 1), _lib.ptr(step_base).value)
        _lib.check(self._lib.ks_commands(_lib.current_stream(), ctypes.byref(io)))
        return command
