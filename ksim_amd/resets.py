"""Resets with the reference's class names (ksim/resets.py:44-189,284-354), compiled to a per-qpos table.

Every reset becomes, per qpos element i: ``qpos[i] = clip(start[i] + u * mag[i] * (level?), lo[i], hi[i])``
with u ~ U(-1, 1) and start[i] = base[i], or the reference-motion frame drawn for the env plus base[i] where
`InitialMotionStateReset` governs the element.  The height-field reset looks z up from the new x, y; the heading and
pitch / roll resets multiply the base quaternion from the right, in list order.  The resets apply in list order
(ksim/engine.py:209-211): one that sets an element replaces what earlier ones did to it, one that adds keeps it.
Two orderings the table cannot express raise when the list is compiled: a height draw after a height-field reset, and a
whole-qpos motion frame after a heading or pitch / roll reset.
Velocity resets are accepted and ignored: the engine zeroes qvel after the reset's forward pass (engine.py:217-220).
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np


@dataclass(frozen=True)
class Reset:
    def apply(self, table: dict, model) -> None:  # pragma: no cover
        raise NotImplementedError


@dataclass(frozen=True)
class RandomJointPositionReset(Reset):  # resets.py:122-144
    scale: float = 0.01
    scale_by_curriculum: bool = True
    zeros: tuple | None = None
    mins: tuple | None = None
    maxs: tuple | None = None

    def apply(self, table, model):
        nj = model.nq - 7
        table["motion"][7:] = 0
        table["mag"][7:] = self.scale
        table["by_level"][7:] = int(self.scale_by_curriculum)
        table["base"][7:] = 0.0 if self.zeros is None else np.asarray(self.zeros, dtype=np.float64).reshape(nj)
        if self.mins is not None:
            table["lo"][7:] = np.asarray(self.mins).reshape(nj)
        if self.maxs is not None:
            table["hi"][7:] = np.asarray(self.maxs).reshape(nj)


@dataclass(frozen=True)
class RandomJointVelocityReset(Reset):  # resets.py:176-189 — wiped by engine.py:217-220
    scale: float = 0.01
    scale_by_curriculum: bool = True

    def apply(self, table, model):
        return None


@dataclass(frozen=True)
class RandomBaseVelocityXYReset(Reset):  # resets.py:192-207 — a no-op on the MJX path (result discarded)
    scale: float = 0.01

    def apply(self, table, model):
        return None


@dataclass(frozen=True)
class RandomHeightReset(Reset):  # resets.py:322-334: qpos[2] += U(range)
    range: tuple = (0.0, 0.0)

    def apply(self, table, model):
        lo, hi = self.range
        if table["hfield"] is not None and hi != lo:
            # the kernel's height-field path sets z = field height + base and has no draw of its own to add
            raise ValueError("a RandomHeightReset with a non-empty range cannot follow an HFieldXYPositionReset; list it first "
                             "or give it a single height")
        table["base"][2] += 0.5 * (lo + hi)
        table["mag"][2] = 0.5 * (hi - lo)
        table["by_level"][2] = 0


@dataclass(frozen=True)
class RandomHeadingReset(Reset):  # resets.py:308-319
    def apply(self, table, model):
        table["heading"] = 1
        if table["pitch_roll"]:
            table["pitch_roll"] = 2  # the pitch / roll reset came first


def _set_xy(table, x_range, y_range, padded_bounds) -> None:
    """x, y <- clip(U(-range, range), padded bounds) (resets.py:56-63, 105-112)."""
    lower_x, upper_x, lower_y, upper_y = padded_bounds
    table["base"][0:2] = 0.0
    table["motion"][0:2] = 0
    table["mag"][0], table["mag"][1] = x_range, y_range
    table["by_level"][0:2] = 0
    table["lo"][0], table["hi"][0], table["lo"][1], table["hi"][1] = lower_x, upper_x, lower_y, upper_y


@dataclass(frozen=True)
class PlaneXYPositionReset(Reset):  # resets.py:93-120
    """x, y uniform in +-range clipped to the padded bounds; z <- plane height + robot_base_height.
    `bounds` = (x_bound, y_bound, z_pos) of the floor plane."""
    bounds: tuple = (5.0, 5.0, 0.0)
    padded_bounds: tuple = (-np.inf, np.inf, -np.inf, np.inf)
    x_range: float = 5.0
    y_range: float = 5.0
    robot_base_height: float = 0.0

    def apply(self, table, model):
        _set_xy(table, self.x_range, self.y_range, self.padded_bounds)
        table["base"][2], table["mag"][2], table["motion"][2] = self.bounds[2] + self.robot_base_height, 0.0, 0
        table["hfield"] = None


@dataclass(frozen=True)
class HFieldXYPositionReset(Reset):  # resets.py:45-90
    """x, y as above; z <- hfield[ix, iy] + z_top + robot_base_height, the cell found by scaling x, y from
    [-bound, bound] to [0, n - 1] and truncating.  `bounds` = (x_bound, y_bound, z_top, z_bottom)."""
    bounds: tuple = (5.0, 5.0, 0.0, 0.0)
    padded_bounds: tuple = (-np.inf, np.inf, -np.inf, np.inf)
    x_range: float = 5.0
    y_range: float = 5.0
    hfield_data: np.ndarray | None = None
    robot_base_height: float = 0.0

    def apply(self, table, model):
        if self.hfield_data is None or np.asarray(self.hfield_data).ndim != 2:
            raise ValueError("hfield_data must be a (rows, columns) array of heights")
        _set_xy(table, self.x_range, self.y_range, self.padded_bounds)
        table["base"][2], table["mag"][2], table["motion"][2] = self.bounds[2] + self.robot_base_height, 0.0, 0
        table["hfield"] = dict(data=np.ascontiguousarray(self.hfield_data, dtype=np.float32), bound=(self.bounds[0], self.bounds[1]))

    def __hash__(self):  # the array field is not hashable
        return id(self)


@dataclass(frozen=True)
class RandomPitchRollReset(Reset):  # resets.py:338-354
    """quat <- quat * euler(roll, pitch, 0).  The reference draws pitch and roll from the same key, so one uniform
    number places both inside their ranges."""
    pitch_range: tuple = (-0.1, 0.1)
    roll_range: tuple = (-0.1, 0.1)

    def apply(self, table, model):
        table["pitch_roll"] = 2 if not table["heading"] else 1  # before or after the heading, as the list orders them
        table["pitch"], table["roll"] = tuple(self.pitch_range), tuple(self.roll_range)


@dataclass(frozen=True)
class InitialMotionStateReset(Reset):  # resets.py:284-306
    """qpos <- a frame of the reference motion drawn uniformly per env, time <- frame * ctrl_dt.  `freejoint`: the whole
    qpos, otherwise only the joints (qpos[7:]).  Its qvel is wiped by the engine like every reset's (engine.py:217-220).
    `reference_motion`: anything with `qpos` (frames, nq) and `ctrl_dt` (`priors.MotionReferenceData`)."""
    reference_motion: object = None
    freejoint: bool = False

    def apply(self, table, model):
        q = np.asarray(getattr(self.reference_motion.qpos, "array", self.reference_motion.qpos), dtype=np.float32)
        if q.ndim != 2 or q.shape[1] != model.nq:
            raise ValueError(f"the reference motion has frames of {q.shape[-1]} numbers, the model's qpos has {model.nq}")
        if self.freejoint and (table["heading"] or table["pitch_roll"]):
            # the kernel turns the base quaternion after the table pass, so it cannot replace a turn made earlier
            raise ValueError("an InitialMotionStateReset(freejoint=True) cannot follow a heading or pitch / roll reset: it "
                             "would have to replace the base orientation they set; list it before them")
        sl = slice(0, model.nq) if self.freejoint else slice(7, model.nq)
        table["motion"][sl] = 1
        table["base"][sl] = 0.0
        table["mag"][sl] = 0.0
        table["lo"][sl], table["hi"][sl] = -np.inf, np.inf
        table["motion_qpos"], table["motion_dt"] = np.ascontiguousarray(q), float(self.reference_motion.ctrl_dt)

    def __hash__(self):
        return id(self)


def compile_resets(resets, model) -> dict:
    """Applies the resets in list order (engine.py:209-211) to the make_data state qpos0."""
    nq = model.nq
    table = dict(base=np.array(model.qpos0, dtype=np.float64), mag=np.zeros(nq), lo=np.full(nq, -np.inf),
                 hi=np.full(nq, np.inf), by_level=np.zeros(nq, dtype=np.int32), heading=0,
                 motion=np.zeros(nq, dtype=np.int32), motion_qpos=None, motion_dt=0.0, pitch_roll=0, pitch=(0.0, 0.0),
                 roll=(0.0, 0.0), hfield=None)
    for r in resets:
        r.apply(table, model)
    return table


def get_xy_position_reset(physics_model=None, x_range: float = 5.0, y_range: float = 5.0, x_edge_padding: float = 5.0,
                          y_edge_padding: float = 5.0, robot_base_height: float = 0.0, hfield_data=None,
                          hfield_size=None, plane_height: float = 0.0) -> Reset:
    """The XY reset that fits the floor (resets.py:210-281): with a height field (`hfield_data` (rows, columns) and
    `hfield_size` = (x_bound, y_bound, z_top, z_bottom)) a `HFieldXYPositionReset`, otherwise a `PlaneXYPositionReset` on
    a plane of half extent 5 at `plane_height`.  The models built here have a plane floor at z = 0; the height-field
    arguments are for callers that bring the terrain themselves."""
    def padded(x_bound, y_bound):
        return (-x_bound + x_edge_padding, x_bound - x_edge_padding, -y_bound + y_edge_padding, y_bound - y_edge_padding)

    if hfield_data is not None:
        x_bound, y_bound, z_top, z_bottom = (float(v) for v in hfield_size)
        return HFieldXYPositionReset(bounds=(x_bound, y_bound, z_top, z_bottom), padded_bounds=padded(x_bound, y_bound),
                                     x_range=x_range, y_range=y_range, hfield_data=np.asarray(hfield_data), robot_base_height=robot_base_height)
    return PlaneXYPositionReset(bounds=(5.0, 5.0, float(plane_height)), padded_bounds=padded(5.0, 5.0), x_range=x_range,
                                y_range=y_range, robot_base_height=robot_base_height)
