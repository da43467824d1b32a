"""Per-env physics randomisers with the reference's names (ksim/randomization.py:39-243).

Each returns ``{field: (N, ...) tensor}`` sampled once per env at initialisation (ksim/task/rl.py:2231-2243);
the step kernel reads ``friction`` (N), ``mass_scale`` (N, nb), ``armature_scale`` and ``damping_scale`` (N, nv)
every step (rl.py:1182).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class PhysicsRandomizer:
    def __call__(self, model, num_envs: int, gen) -> dict:  # pragma: no cover
        raise NotImplementedError


@dataclass(frozen=True)
class FloorFrictionRandomizer(PhysicsRandomizer):  # randomization.py:74-104: absolute value U(lo, hi)
    scale_lower: float = 0.4
    scale_upper: float = 1.0

    def __call__(self, model, num_envs, gen):
        u = torch.rand(num_envs, generator=gen, device=gen.device)
        return {"friction": self.scale_lower + (self.scale_upper - self.scale_lower) * u}


@dataclass(frozen=True)
class AllBodiesMassMultiplicationRandomizer(PhysicsRandomizer):  # randomization.py:207-222: body_mass *= U
    scale_lower: float = 0.95
    scale_upper: float = 1.05

    def __call__(self, model, num_envs, gen):
        u = torch.rand(num_envs, model.nb, generator=gen, device=gen.device)
        return {"mass_scale": self.scale_lower + (self.scale_upper - self.scale_lower) * u}


def _joint_scale(model, num_envs, gen, lo, hi):
    """A factor per dof: U(lo, hi) on the joints, 1 on the six dofs of the floating base (randomization.py:115-122)."""
    s = torch.ones(num_envs, model.nv, device=gen.device)
    first = 6 if model.has_free_root else 0
    s[:, first:] = lo + (hi - lo) * torch.rand(num_envs, model.nv - first, generator=gen, device=gen.device)
    return s


@dataclass(frozen=True)
class ArmatureRandomizer(PhysicsRandomizer):  # randomization.py:108-123: dof_armature[6:] *= U
    scale_lower: float = 0.95
    scale_upper: float = 1.05

    def __call__(self, model, num_envs, gen):
        return {"armature_scale": _joint_scale(model, num_envs, gen, self.scale_lower, self.scale_upper)}


@dataclass(frozen=True)
class JointDampingRandomizer(PhysicsRandomizer):  # randomization.py:226-243: dof_damping[6:] *= U
    scale_lower: float = 0.9
    scale_upper: float = 1.1

    def __call__(self, model, num_envs, gen):
        return {"damping_scale": _joint_scale(model, num_envs, gen, self.scale_lower, self.scale_upper)}


@dataclass(frozen=True)
class MassMultiplicationRandomizer(PhysicsRandomizer):  # randomization.py:166-204: one body's mass *= U
    body_id: int = 1
    scale_lower: float = 0.95
    scale_upper: float = 1.05

    @classmethod
    def from_body_name(cls, model, body_name: str, scale_lower: float = 0.0, scale_upper: float = 1.0):
        if body_name not in model.body_names:
            raise ValueError(f"Body name {body_name} not found in model")
        return cls(body_id=list(model.body_names).index(body_name), scale_lower=scale_lower, scale_upper=scale_upper)

    def __call__(self, model, num_envs, gen):
        s = torch.ones(num_envs, model.nb, device=gen.device)
        s[:, self.body_id] = self.scale_lower + (self.scale_upper - self.scale_lower) * torch.rand(num_envs, generator=gen, device=gen.device)
        return {"mass_scale": s}


@dataclass(frozen=True)
class MassAdditionRandomizer(PhysicsRandomizer):  # randomization.py:126-163: one body's mass += U(lo, hi), as a factor
    body_id: int = 1
    scale_lower: float = 0.0
    scale_upper: float = 1.0

    def __call__(self, model, num_envs, gen):
        s = torch.ones(num_envs, model.nb, device=gen.device)
        add = self.scale_lower + (self.scale_upper - self.scale_lower) * torch.rand(num_envs, generator=gen, device=gen.device)
        s[:, self.body_id] = (float(model.body_mass[self.body_id]) + add) / float(model.body_mass[self.body_id])
        return {"mass_scale": s}


def get_physics_randomizers(model, randomizers: dict, num_envs: int, gen) -> dict:
    """Merges the randomisers' fields; duplicate fields raise (ksim/task/rl.py:343-346)."""
    out: dict = {}
    for name, r in randomizers.items():
        for k, v in r(model, num_envs, gen).items():
            if k in out:
                raise ValueError(f"Found duplicate randomization keys: {k}")
            out[k] = v.contiguous()
    return out
