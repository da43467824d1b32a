"""Host side of the AMP discriminator update (ksim/task/amp.py:441-545): batches of reference and simulated motions, the
loss gradient (`ks_mlp_disc_loss_grad`), the optimiser step, `disc_num_passes` times per policy update.

The discriminator is an `MLP` with one output that scores each frame of a motion, so a motion (T, F) gets logits (T,) as
`AMPTask.call_discriminator` asks (amp.py:257-268).  The AMP reward from those logits is `ksim_amd.rewards.AMPReward`.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import _lib
from . import _lib_terms as T
from .mlp import MLP


@dataclass
class AMPConfig:  # the discriminator's part of ksim/task/amp.py:62-95
    amp_reference_batch_size: int = 32
    disc_num_passes: int = 1
    amp_grad_penalty_coef: float = 10.0
    learning_rate: float = 3e-4
    adam_b1: float = 0.9
    adam_b2: float = 0.999
    adam_eps: float = 1e-8
    weight_decay: float = 0.0
    max_grad_norm: float | None = None


def loop_slice(clip: torch.Tensor, start: int, window_t: int) -> torch.Tensor:
    """A window of `window_t` frames from `start`, wrapping round when the clip is shorter (amp.py:53-58)."""
    idx = (torch.arange(window_t, device=clip.device) + int(start)) % clip.shape[0]
    return clip[idx]


def make_real_batch(motions: torch.Tensor, window_t: int, batch_b: int, generator: torch.Generator) -> torch.Tensor:
    """`batch_b` windows from reference clips (N, T_clip, F): a clip drawn uniformly, then a uniform start in it
    (amp.py:570-625; the draws come from `generator`, not from jax's key splitting)."""
    clip_idx = torch.randint(0, motions.shape[0], (batch_b,), generator=generator)
    starts = torch.randint(0, motions.shape[1], (batch_b,), generator=generator)
    # every window of the batch in one gather: frame (start + t) mod T_clip of the drawn clip, as loop_slice takes them
    frames = (starts[:, None] + torch.arange(window_t)[None, :]) % motions.shape[1]
    return motions[clip_idx[:, None].to(motions.device), frames.to(motions.device)]


def make_sim_batch(sim_motions: torch.Tensor, batch_b: int, generator: torch.Generator) -> torch.Tensor:
    """`batch_b` distinct envs of the rollout's motions (num_envs, T, F) (amp.py:627-652)."""
    num_envs = sim_motions.shape[0]
    if num_envs % batch_b != 0:
        raise ValueError(f"amp_reference_batch_size ({batch_b}) must divide batch_size ({num_envs}).")
    return sim_motions[torch.randperm(num_envs, generator=generator)[:batch_b].to(sim_motions.device)]


class DiscriminatorUpdate:
    """Owns the discriminator's optimiser state; `step` is one pass of amp.py:486-527, `update` all of them."""

    def __init__(self, disc: MLP, cfg: AMPConfig):
        if disc.out_dim != 1:
            raise _lib.KsError(f"the discriminator scores a frame with one number, not {disc.out_dim}")
        self.disc, self.cfg, self.count = disc, cfg, 0
        disc.train_init()
        self._acc = torch.zeros(1, dtype=torch.float64, device="cuda")

    def loss_grad(self, real: torch.Tensor, sim: torch.Tensor) -> torch.Tensor:
        """Gradients into the discriminator's buffers; returns the (real, simulated, penalty) loss terms, on the device."""
        return self.disc.disc_loss_grad(real, sim, self.cfg.amp_grad_penalty_coef)

    def step(self, real: torch.Tensor, sim: torch.Tensor) -> dict[str, torch.Tensor]:
        losses = self.loss_grad(real, sim)
        sq = None
        if self.cfg.max_grad_norm is not None:
            self._acc.zero_()
            self.disc.grad_sqnorm(self._acc)
            sq = self._acc
        self.count += 1
        c = self.cfg
        self.disc.adam_step(T.KsAdamParams(c.learning_rate, c.adam_b1, c.adam_b2, c.adam_eps, c.weight_decay,
                                           0.0 if c.max_grad_norm is None else c.max_grad_norm, self.count), sq)
        return {"disc_loss": losses.sum(), "disc_real_loss": losses[0], "disc_sim_loss": losses[1], "disc_gp_loss": losses[2]}

    def update(self, motions: torch.Tensor, sim_motions: torch.Tensor, generator: torch.Generator) -> dict[str, torch.Tensor]:
        """`disc_num_passes` steps, each on fresh batches; the metrics are averaged over the passes (amp.py:529-536)."""
        window_t = sim_motions.shape[1]
        sums: dict[str, torch.Tensor] = {}
        for _ in range(self.cfg.disc_num_passes):
            real = make_real_batch(motions, window_t, self.cfg.amp_reference_batch_size, generator)
            sim = make_sim_batch(sim_motions, self.cfg.amp_reference_batch_size, generator)
            for k, v in self.step(real, sim).items():
                sums[k] = v if k not in sums else sums[k] + v
        return {k: v / self.cfg.disc_num_passes for k, v in sums.items()}
