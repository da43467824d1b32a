"""Resets with the reference's class names (ksim/resets.py:122-189,308-334), compiled to a per-qpos table.

Every reset becomes, per qpos element i: ``qpos[i] = clip(base[i] + u * mag[i] * (level?), lo[i], hi[i])``
with u ~ U(-1, 1); the heading reset multiplies the base quaternion by a uniform yaw.  Velocity resets are
accepted and ignored: the engine zeroes qvel after the reset's forward pass (ksim/engine.py:217-220).
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
        table["base"][2] += 0.5 * (lo + hi)
        table["mag"][2] = 0.5 * (hi - lo)
        table["by_level"][2] = 0


@dataclass(frozen=True)
class RandomHeadingReset(Reset):  # resets.py:308-319
    def apply(self, table, model):
        table["heading"] = 1


@dataclass(frozen=True)
class PlaneXYPositionReset(Reset):  # resets.py:44-72 without the plane lookup: uniform xy in +-range
    x_range: float = 0.0
    y_range: float = 0.0

    def apply(self, table, model):
        table["mag"][0], table["mag"][1] = self.x_range, self.y_range
        table["by_level"][0:2] = 0


def compile_resets(resets, model) -> dict:
    """Applies the resets in list order (engine.py:209-211) to the make_data state qpos0."""
    nq = model.nq
    table = dict(base=np.array(model.qpos0, dtype=np.float64), mag=np.zeros(nq), lo=np.full(nq, -np.inf),
                 hi=np.full(nq, np.inf), by_level=np.zeros(nq, dtype=np.int32), heading=0)
    for r in resets:
        r.apply(table, model)
    return table
