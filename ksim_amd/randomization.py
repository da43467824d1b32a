"""Per-env physics randomisers with the reference's names (ksim/randomization.py:39-243).

Each returns ``{field: (N, ...) tensor}`` sampled once per env at initialisation (ksim/task/rl.py:2231-2243);
the step kernel reads ``friction`` (N) and ``mass_scale`` (N, nb) every step (rl.py:1182).
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


def get_physics_randomizers(model, randomizers: dict, num_envs: int, gen) -> dict:
    """Merges the randomisers' fields; duplicate fields raise (ksim/task/rl.py:343-346)."""
    out: dict = {}
    for name, r in randomizers.items():
        for k, v in r(model, num_envs, gen).items():
            if k in out:
                raise ValueError(f"Found duplicate randomization keys: {k}")
            out[k] = v.contiguous()
    return out
