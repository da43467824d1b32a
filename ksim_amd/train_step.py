"""One iteration of the training loop's device work (ksim/task/rl.py:1777-1816 `_rl_train_loop_step`): unroll, the
AMP task's discriminator scoring of the trajectory (ksim/task/amp.py:327-358), rewards, then the policy update with
the discriminator passes after every minibatch step (ksim/task/ppo.py:572-694, ksim/task/amp.py:455-545).

Only the composition lives here; every piece is a kernel behind the C ABI (`Rollout`, `MLP`, `get_rewards`,
`ppo_update.update_model`, `amp.DiscriminatorUpdate`).  Logging, curriculum stepping and checkpointing of the
reference's loop stay with the caller.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Mapping, Sequence

import torch

from . import _lib
from .amp import DiscriminatorUpdate, make_real_batch, make_sim_batch
from .ppo_update import GaussianMlpPolicy, PPOUpdateConfig, update_model
from .rewards import DISCRIMINATOR_OUTPUT_KEY, get_rewards
from .rollout import Rollout, RolloutEnvState
from .types import RewardState, Trajectory




def default_trajectory_to_motion(trajectory: Trajectory) -> torch.Tensor:
    """(T, N, F) motion frames of a trajectory (AMPTask.trajectory_to_motion is the task's to define, amp.py:270-283):
    base height and orientation, joint positions, all velocities and the applied torques."""
    return torch.cat([trajectory.qpos[..., 2:], trajectory.qvel, trajectory.ctrl], dim=-1).contiguous()


@dataclass
class AMPSetup:
    """The AMP task's additions to a PPO iteration: the discriminator's optimiser state, the reference motions
    (clips, frames, F) and how a trajectory becomes motion frames."""
    update: DiscriminatorUpdate
    real_motions: torch.Tensor
    trajectory_to_motion: Callable[[Trajectory], torch.Tensor] = default_trajectory_to_motion

    @property
    def disc(self):
        return self.update.disc


def postprocess_trajectory(trajectory: Trajectory, amp: AMPSetup) -> tuple[Trajectory, torch.Tensor]:
    """Discriminator logits of every (t, env) frame into `trajectory.aux_outputs` (amp.py:327-358); also returns the
    motion frames (T, N, F)."""
    motion = amp.trajectory_to_motion(trajectory)
    Tn, N, F = motion.shape
    if F != amp.disc.in_dim:
        raise _lib.KsError(f"the discriminator takes frames of {amp.disc.in_dim} numbers, the trajectory gives {F}")
    logits = amp.disc(motion.view(Tn * N, F)).view(Tn, N)
    aux = dict(trajectory.aux_outputs or {})
    aux[DISCRIMINATOR_OUTPUT_KEY] = logits
    trajectory.aux_outputs = aux
    return trajectory, motion


def rl_train_loop_step(rollout: Rollout, env: RolloutEnvState, policy: GaussianMlpPolicy, cfg: PPOUpdateConfig, *,
                       level: float = 1.0, amp: AMPSetup | None = None, noise: Sequence[Mapping | None] | None = None,
                       permutations: list[torch.Tensor] | None = None, generator: torch.Generator | None = None,
                       disc_batches: Callable[[int, torch.Tensor, torch.Tensor], tuple[torch.Tensor, torch.Tensor]] | None = None,
                       want_components: bool = False) -> dict:
    """Unroll T steps, score, reward, update.  `noise[t]` are explicit draws for step t (parity runs); `permutations`
    the minibatch orders of the passes; `disc_batches(k, idx, sim_motions)` returns the (real, sim) motion batches of the
    k-th discriminator step over the minibatch of envs `idx` of `sim_motions` (N, T, F) instead of sampling them
    (amp.py:486-497 samples with jax keys)."""
    c = rollout.c
    for t in range(rollout.T):
        rollout.step_engine(env, t, level, noise[t] if noise is not None else None)
    traj = rollout.trajectory()
    motion = None
    if amp is not None:
        traj, motion = postprocess_trajectory(traj, amp)
    rewards: RewardState = get_rewards(traj, c.rewards, c.reward_clip_min, c.reward_clip_max, want_components=want_components,
                                       rewards_carry=env.reward_carry, obs_slices=c.terms.obs_slices, level=level,
                                       command_slices=c.commands.slices if c.commands is not None else None)
    after = None
    disc_steps = [0]
    if amp is not None:
        gen = generator or torch.Generator().manual_seed(0)
        sim_motions = motion.transpose(0, 1)  # (N, T, F): one motion per env, like the reference's trajectories

        def after(idx: torch.Tensor):
            mets = []
            for _ in range(amp.update.cfg.disc_num_passes):
                if disc_batches is not None:
                    real, sim = disc_batches(disc_steps[0], idx, sim_motions)
                else:
                    real = make_real_batch(amp.real_motions, rollout.T, amp.update.cfg.amp_reference_batch_size, gen)
                    sim = make_sim_batch(sim_motions.index_select(0, idx), amp.update.cfg.amp_reference_batch_size, gen)
                mets.append(amp.update.step(real.contiguous(), sim.contiguous()))
                disc_steps[0] += 1
            return mets

    steps = update_model(policy, cfg, rollout.noisy_obs, rollout.obs, rollout.action, rewards.total, rollout.done,
                         rollout.success, permutations=permutations, after_step=after)
    return {"trajectory": traj, "rewards": rewards, "steps": steps, "motion": motion}
