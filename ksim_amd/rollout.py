"""Batched rollout of N envs for T control steps (ksim/task/rl.py:1164-1211 step_engine, 1604-1665 _single_unroll).

One control step launches, in order on the current stream: observation (+noise) -> actor MLP (and critic)
-> action sampling / scrub / clip -> fused physics control step -> terminations + transition record + reset
predication -> forward pass of the freshly reset envs.  Nothing synchronises the host inside the loop, so a
whole rollout (T steps and the reward pass) can be captured once as a HIP graph and replayed, which takes the
per-launch host cost out of the loop (`Rollout.unroll(..., graph=True)`).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Mapping, Sequence

import torch

from . import _lib
from . import _lib_terms as T
from . import ppo as ppo_mod
from .actions import LowPass
from .commands import CommandSet
from .engine import HipEngine
from .env_terms import EnvTerms, sample_action, sample_action_head, sample_action_mixture
from .mlp import MLP
from .physics import DeviceModel
from .recurrent import RecurrentNetwork
from .rewards import Reward, get_rewards, initial_reward_carry, reward_carry_size
from .types import PhysicsState, RewardState, Trajectory


@dataclass(frozen=True)
class GaussianHead:
    """The actor emits (means | raw deviations), 2 per action entry (examples/kbot/train.py:915-932)."""
    min_std: float
    max_std: float
    var_scale: float = 1.0
    mean_bias: torch.Tensor | None = None
    lowpass: LowPass | None = None  # the biased means pass a one-pole low-pass before sampling (train.py:923-929)

    def width(self, na: int) -> int:
        return 2 * na


@dataclass(frozen=True)
class MixtureHead:
    """The actor emits component means, raw deviations and logits, 3 K per action entry (examples/walking.py:127-144)."""
    num_mixtures: int
    min_std: float
    max_std: float
    var_scale: float = 1.0
    mean_bias: torch.Tensor | None = None
    clip_lo: torch.Tensor | None = None
    clip_hi: torch.Tensor | None = None

    def width(self, na: int) -> int:
        return 3 * na * self.num_mixtures


@dataclass
class RolloutConstants:  # the static pieces, ksim/task/rl.py:138-150
    physics_model: DeviceModel
    engine: HipEngine
    terms: EnvTerms
    rewards: Mapping[str, Reward]
    actor: MLP | RecurrentNetwork
    critic: MLP | RecurrentNetwork | None
    log_std: torch.Tensor | None
    action_clip_max: float = 1e3  # RLConfig.action_clip_max, rl.py:589-592
    reward_clip_min: float | None = None
    reward_clip_max: float | None = None
    commands: CommandSet | None = None  # commands advanced once per control step (rl.py:1082-1098); None: constant
    # The forward pass that a reset owes (engine.py:213) runs inside the next control step's physics launch instead of as a
    # masked launch of its own right after the termination pass: one launch less per control step, the same trajectories
    # bit for bit.  Between two steps the warm start of a freshly reset env is then not yet that of its new episode, and
    # the mode is only taken when no term of the task reads a derived field (xpos, xquat, cvel ...) of the live state.
    defer_reset_forward: bool = False
    # The observation of control step t + 1 is computed by the launch that ends step t (terminations, transition record,
    # resets): `ks_terminate_reset_observe`, one launch instead of two, the same numbers.  Taken when the task has no
    # command set to advance in between and its observations read no derived field of the live state.
    fuse_next_observation: bool = False
    head: GaussianHead | MixtureHead | None = None  # None: one mean per action entry and the log_std vector
    # A critic that does not share a launch with the actor (a recurrent one: a dozen short launches per control step) runs on a
    # side stream of its own, beside the actor, the sampling and the physics launch, and is joined before the termination pass
    # (which rewrites the reset mask the critic reads).  Nothing of a control step waits for the value, so the chain of launches
    # that a step has to wait for loses the critic's share.  Same numbers; off by default (a split rollout already has a stream
    # per group, and a process has four hardware queues).
    critic_on_side_stream: bool = False


class RolloutEnvState:  # ksim/task/rl.py:110-123, batched
    def __init__(self, physics_state: PhysicsState, randomization: Mapping[str, torch.Tensor], commands: torch.Tensor,
                 obs_bias: torch.Tensor | None, seed: int):
        self.physics_state = physics_state
        self.randomization_dict = dict(randomization)
        self.commands = commands
        self.obs_bias = obs_bias  # (N, obs_dim, 2) standard draws (z, w) behind the per-episode observation biases, or None
        self.seed = int(seed)
        self.step = 0
        self.obs_carry = None     # (N, carry_dim) carries of the stateful observations (rl.py:118), made on first use
        self.reward_carry = None  # (N, reward carry size) carries of the stateful rewards (rl.py:119)
        self.commands_drawn = False  # whether the command set has drawn this env state's initial commands
        self.actor_carry = None   # (depth, N, hidden) carries of recurrent networks (rl.py:117)
        self.critic_carry = None
        self.lpf_state = None     # (N, nu) state of the low-pass filter on the actor's means, part of the model carry
        N = physics_state.data.qpos.shape[0]
        self.episode_length = torch.zeros(N, dtype=torch.int32, device=physics_state.data.qpos.device)


class Rollout:
    """Owns the time-major trajectory buffers of one (T, N) rollout and runs it."""

    def __init__(self, constants: RolloutConstants, num_envs: int, rollout_length: int):
        c, m = constants, constants.physics_model.model
        self.c, self.N, self.T = c, int(num_envs), int(rollout_length)
        dev = torch.device("cuda")
        N, Tn = self.N, self.T
        f = lambda *s: torch.empty(*s, dtype=torch.float32, device=dev)  # noqa: E731
        b = lambda *s: torch.zeros(*s, dtype=torch.uint8, device=dev)  # noqa: E731
        self.obs, self.noisy_obs = f(Tn, N, c.terms.obs_dim), f(Tn, N, c.terms.obs_dim)
        na = c.engine.actuators.action_dim(m.nu)  # 2 nu for position-velocity actuators
        self.action, self.mean = f(Tn, N, na), f(N, na if c.head is None else c.head.width(na))
        self.qpos, self.qvel = f(Tn, N, m.nq), f(Tn, N, m.nv)
        self.xpos, self.xquat, self.ctrl = f(Tn, N, m.nb * 3), f(Tn, N, m.nb * 4), f(Tn, N, m.nu)
        self.done, self.success, self.timestep = b(Tn, N), b(Tn, N), f(Tn, N)
        self.components = torch.zeros(Tn, max(c.terms.n_terms, 1), N, dtype=torch.int8, device=dev)
        self.values = f(Tn, N, 1) if c.critic is not None else None
        self.reset_mask = b(N)
        # what a recurrent policy update replays the rollout from: the envs that started an episode at each step and the
        # carries the rollout began with (the model carry of the trajectory's first step, ksim/task/rl.py:117)
        self.fresh = b(Tn, N) if any(isinstance(n, RecurrentNetwork) for n in (c.actor, c.critic)) else None
        self.actor_carry0 = c.actor.initial_carry(N, dev) if isinstance(c.actor, RecurrentNetwork) else None
        self.critic_carry0 = c.critic.initial_carry(N, dev) if isinstance(c.critic, RecurrentNetwork) else None
        self._lowpass = c.head.lowpass if isinstance(c.head, GaussianHead) else None
        self.lpf_carry0 = f(N, na) if self._lowpass is not None else None  # the filter state at the rollout's first step
        if self._lowpass is not None and self.fresh is None:
            self.fresh = b(Tn, N)  # the update replays the filter from the same episode starts
        self.command = f(Tn, N, c.commands.command_dim) if c.commands is not None else None
        if c.commands is not None and c.commands.command_dim != c.terms.command_dim:
            raise _lib.KsError("the command set and the observation terms disagree about the width of the command vector")
        # Philox step counter of graph replays: kernels add it to the step baked into the captured launch
        self.step_base = torch.zeros(1, dtype=torch.int64, device=dev)
        self._graph = None
        # derived fields of the live physics data that the task's terms read: the others are recorded into the rollout
        # slot only (the step kernel would otherwise write xpos / xquat / ctrl twice per control step)
        used = c.terms.sources_used
        need = {T.SRC_QACC: "qacc", T.SRC_CTRL: "ctrl", T.SRC_XPOS: "xpos", T.SRC_XQUAT: "xquat", T.SRC_CVEL: "cvel",
                T.SRC_CONTACT_DIST: "contact_dist", T.SRC_CINERT: "cinert", T.SRC_CFRC_EXT: "cfrc_ext"}
        self._live = {name for src, name in need.items() if src in used}
        self._live.add("contact_dist")  # a few floats per env, also read by the illegal-contact termination
        reads_derived = any(src in used for src in need)
        self._defer = bool(c.defer_reset_forward) and not reads_derived
        self._fuse_obs = bool(c.fuse_next_observation) and not reads_derived and c.commands is None
        self._obs_done = None  # (env state, slot, step) whose observation the previous step's last launch has written
        self._side = None      # the critic's stream and its fork / join events (critic_on_side_stream), made on first use
        if c.actor.in_dim != c.terms.obs_dim or c.actor.out_dim != self.mean.shape[1]:
            raise _lib.KsError("actor must map the observation vector to one mean per action entry (or to what its head takes)")
        if c.critic is not None and (c.critic.in_dim != c.terms.obs_dim or c.critic.out_dim != 1):
            raise _lib.KsError("critic must map the observation vector to one value")

    def step_engine(self, env: RolloutEnvState, t: int, level: float = 1.0, noise: Mapping | None = None,
                    _relative_step: bool = False) -> None:
        """One control step of every env; the transition lands in slot t of the buffers."""
        c, ps = self.c, env.physics_state
        d, noise = ps.data, noise or {}
        # under graph capture the random-number step is (device counter + t) instead of the host counter
        step, step_base = (t, self.step_base) if _relative_step else (env.step, None)
        src = {T.SRC_QPOS: d.qpos, T.SRC_QVEL: d.qvel, T.SRC_QACC: d.qacc, T.SRC_CTRL: d.ctrl,
               T.SRC_LAST_ACTION: ps.last_ctrl, T.SRC_COMMAND: env.commands, T.SRC_TIME: d.time, T.SRC_XPOS: d.xpos,
               T.SRC_XQUAT: d.xquat, T.SRC_CVEL: d.cvel, T.SRC_CONTACT_DIST: d.contact_dist, T.SRC_CINERT: d.cinert,
               T.SRC_CFRC_EXT: d.cfrc_ext}
        self._prepare_env(env)

        def observe_args(slot: int, at_step: int) -> dict:
            # the reset mask holds the envs that the previous control step reset: their carries and biases start afresh
            return dict(level=level, zero_offset=ps.zero_offset, bias_draw=env.obs_bias, seed=env.seed, step=at_step,
                        step_base=step_base, obs=self.obs[slot], noisy_obs=self.noisy_obs[slot], carry=env.obs_carry,
                        fresh=self.reset_mask if (c.terms.carry_dim or c.terms.has_bias) else None,
                        site_pose=(env.randomization_dict or {}).get("site_pose"))

        if self._obs_done != (id(env), t, step, _relative_step):  # else the launch that ended the previous step wrote it
            c.terms.observe(src, self.N, bias_redraw=noise.get("obs_bias_redraw"), noise_normal=noise.get("obs_normal"),
                            noise_uniform=noise.get("obs_uniform"), carry_uniform=noise.get("obs_carry_uniform"),
                            **observe_args(t, step))
        self._obs_done = None
        # actor reads the noisy copy (walking.py:592-595), critic the clean one (walking.py:626-638); recurrent networks
        # advance their carries, which restart from zero for the envs the previous control step reset
        if self.fresh is not None:
            self.fresh[t].copy_(self.reset_mask)
            if t == 0:
                if self.actor_carry0 is not None:
                    self.actor_carry0.copy_(env.actor_carry)
                if self.critic_carry0 is not None:
                    self.critic_carry0.copy_(env.critic_carry)
        critic_joined = True
        if isinstance(c.actor, MLP) and isinstance(c.critic, MLP):
            # two plain MLPs over the same rows share one launch
            c.actor.forward_pair(self.noisy_obs[t], self.mean, c.critic, self.obs[t], self.values[t])
        else:
            def run_critic() -> None:
                if isinstance(c.critic, RecurrentNetwork):
                    c.critic(self.obs[t], env.critic_carry, fresh=self.reset_mask, out=self.values[t])
                elif c.critic is not None:
                    c.critic(self.obs[t], out=self.values[t])

            if c.critic is not None and c.critic_on_side_stream:
                if self._side is None:
                    self._side = (torch.cuda.Stream(), torch.cuda.Event(), torch.cuda.Event())
                side, forked, done_ev = self._side
                main = torch.cuda.current_stream()
                forked.record(main)  # the observation of this step and the previous step's reset mask are final
                side.wait_event(forked)
                with torch.cuda.stream(side):
                    run_critic()
                    done_ev.record(side)
                critic_joined = False
            else:
                run_critic()
            if isinstance(c.actor, RecurrentNetwork):
                c.actor(self.noisy_obs[t], env.actor_carry, fresh=self.reset_mask, out=self.mean)
            else:
                c.actor(self.noisy_obs[t], out=self.mean)
        if isinstance(c.head, GaussianHead):
            head_bias = c.head.mean_bias
            if self._lowpass is not None:
                # the filter's state belongs to the model carry: zero for the envs the previous step reset (rl.py:1072-1080)
                if t == 0:
                    self.lpf_carry0.copy_(env.lpf_state)
                lp, nu_ = self._lowpass, self.action.shape[-1]
                add, add_ld, a0, cnt = None, 0, 0, 0
                if lp.obs_bias is not None:
                    col0, a0, cnt = (int(v) for v in lp.obs_bias)
                    add, add_ld = _lib.c_void_p(self.noisy_obs[t].data_ptr() + 4 * col0), self.noisy_obs.shape[-1]
                _lib.check(_lib.load().ks_lowpass_scan(_lib.current_stream(), 1, self.N, nu_, 2 * nu_, float(lp.ctrl_dt),
                                                       float(lp.cutoff_frequency), _lib.ptr(self.mean), _lib.ptr(head_bias), add, add_ld,
                                                       a0, cnt, _lib.ptr(env.lpf_state), _lib.ptr(self.reset_mask), _lib.ptr(self.mean),
                                                       _lib.ptr(env.lpf_state)))
                head_bias = None  # now inside the filtered location
            sample_action_head(self.mean, min_std=c.head.min_std, max_std=c.head.max_std, var_scale=c.head.var_scale,
                               mean_bias=head_bias, noise=noise.get("action_normal"), seed=env.seed, step=step,
                               step_base=step_base, clip_max=c.action_clip_max, out=self.action[t])
        elif isinstance(c.head, MixtureHead):
            sample_action_mixture(self.mean, c.head.num_mixtures, min_std=c.head.min_std, max_std=c.head.max_std,
                                  var_scale=c.head.var_scale, mean_bias=c.head.mean_bias, clip_lo=c.head.clip_lo,
                                  clip_hi=c.head.clip_hi, uniform=noise.get("action_uniform"), noise=noise.get("action_normal"),
                                  seed=env.seed, step=step, step_base=step_base, clip_max=c.action_clip_max, out=self.action[t])
        else:
            sample_action(self.mean, c.log_std, noise=noise.get("action_normal"), seed=env.seed, step=step,
                          step_base=step_base, clip_max=c.action_clip_max, out=self.action[t])
        # the step kernel also writes ctrl / xpos / xquat of the post-step data into the transition slot
        c.engine.step(self.action[t], c.physics_model, ps, level, env.seed + env.step, env.randomization_dict,
                      noise=noise.get("engine"), record=dict(ctrl=self.ctrl[t], xpos=self.xpos[t], xquat=self.xquat[t]),
                      want_cvel=T.SRC_CVEL in c.terms.sources_used, want_cinert=T.SRC_CINERT in c.terms.sources_used,
                      want_cfrc_ext=T.SRC_CFRC_EXT in c.terms.sources_used, step=step, step_base=step_base, event_seed=env.seed,
                      live=self._live, fresh=self.reset_mask if self._defer else None)
        if not critic_joined:  # the termination pass rewrites the reset mask that the critic's launches read
            torch.cuda.current_stream().wait_event(self._side[2])
        ev_buf = ps.event_states.get("_buffer") if ps.event_states else None
        st = dict(qpos=d.qpos, qvel=d.qvel, qacc_warmstart=d.qacc_warmstart, time=d.time, last_ctrl=ps.last_ctrl)
        term_args = dict(level=level, components=self.components[t][: c.terms.n_terms] if c.terms.n_terms else None,
                         done=self.done[t], success=self.success[t], traj_qpos=self.qpos[t],
                         traj_qvel=self.qvel[t], traj_time=self.timestep[t], reset_mask=self.reset_mask,
                         episode_length=env.episode_length, reset_uniform=noise.get("reset_uniform"),
                         seed=env.seed, step=step, step_base=step_base, event_state=ev_buf,
                         event_intervals=[ev.interval_range for ev in c.engine.events.values()],
                         event_reset_uniform=noise.get("event_reset_uniform"),
                         event_force=ps.event_states.get("_force_buffer") if ps.event_states else None,
                         contact_dist=d.contact_dist if "contact_dist" in self._live else None, episode=c.engine.episode_args(ps, noise.get("episode")))
        if self._fuse_obs and t + 1 < self.T and not noise:
            # the next step's observation rides in this launch (its random numbers are those of step + 1)
            c.terms.terminate_reset_observe(st, term_args, src, observe_args(t + 1, step + 1))
            self._obs_done = (id(env), t + 1, step + 1, _relative_step)
        else:
            c.terms.terminate_reset(st, **term_args)
        # refresh the derived fields and the warm start of the reset envs (engine.py:213); in the deferred mode the next
        # step's physics launch does it for the envs still flagged in the reset mask
        if not self._defer:
            c.engine.forward(c.physics_model, ps, self.reset_mask, env.randomization_dict, live=self._live)
        if c.commands is not None:  # record the commands this step ran under, then advance them (rl.py:1082-1098)
            c.commands.update(env.commands, d.qpos, d.qvel, level=level, fresh=self.reset_mask, record=self.command[t],
                              uniform=noise.get("command_uniform"), seed=env.seed, step=step, step_base=step_base)
        if not _relative_step:
            env.step += 1

    def unroll(self, env: RolloutEnvState, level: float = 1.0, graph: bool = False) -> tuple[Trajectory, RewardState]:
        """T control steps and the reward pass.  With `graph=True` the launches are captured once as a HIP graph
        (per env state object and curriculum level) and replayed on later calls; the results are the same bits."""
        if graph:
            return self._unroll_graph(env, level)
        for t in range(self.T):
            self.step_engine(env, t, level)
        traj = self.trajectory()
        return traj, self._rewards(traj, env, level)

    def _unroll_graph(self, env: RolloutEnvState, level: float) -> tuple[Trajectory, RewardState]:
        if self.c.engine.data.drop_action_prob * float(level) > 0:
            raise _lib.KsError("graph replay needs drop_action_prob == 0 (the drop mask is sampled on the host side)")
        if not self._capture(env, level) and int(env.step) != self._graph_step:
            self.step_base.fill_(env.step)  # the eager path ran in between
        _, g, traj, rewards = self._graph
        g.replay()
        env.step += self.T
        self._graph_step = int(env.step)
        return traj, rewards

    def _capture(self, env: RolloutEnvState, level: float) -> bool:
        """Captures the rollout of `env` at `level` as a HIP graph unless that is the graph already held; True when it
        captured (which synchronises the device)."""
        key = (id(env), float(level))
        if self._graph is not None and self._graph[0] == key:
            return False
        self.step_base.fill_(env.step)
        self.c.engine.prepare(self.step_base.device)
        self._prepare_env(env)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for t in range(self.T):
                self.step_engine(env, t, level, _relative_step=True)
            traj = self.trajectory()
            rewards = self._rewards(traj, env, level)
            self.step_base += self.T
        self._graph = (key, g, traj, rewards)
        self._graph_step = int(env.step)
        return True

    def _prepare_env(self, env: RolloutEnvState) -> None:
        """Carry buffers of an env state seen for the first time (never inside a graph capture: `_unroll_graph`
        calls this before it starts capturing)."""
        self.c.engine.prepare_state(env.physics_state)
        if self.c.terms.carry_dim and env.obs_carry is None:
            env.obs_carry = torch.zeros(self.N, self.c.terms.carry_dim, dtype=torch.float32, device=self.done.device)
            self.reset_mask.fill_(1)  # every env starts an episode: the first observation initialises all carries
        if self.c.terms.has_bias and env.obs_bias is None:
            # the episode's standard draws behind the observation biases (rl.py:121,263-271 keeps keys instead)
            env.obs_bias = torch.zeros(self.N, self.c.terms.obs_dim, 2, dtype=torch.float32, device=self.done.device)
            self.reset_mask.fill_(1)  # every env starts an episode: the first observation draws all of them
        if self.c.commands is not None and not env.commands_drawn:  # get_initial_commands on the reset state (rl.py:319-332)
            d = env.physics_state.data
            self.c.commands.update(env.commands, d.qpos, d.qvel, all_fresh=True, seed=env.seed, step=(1 << 62) + env.step)
            env.commands_drawn = True
        if self._lowpass is not None and env.lpf_state is None:
            env.lpf_state = torch.zeros(self.N, self.action.shape[-1], dtype=torch.float32, device=self.done.device)
        for net, name in ((self.c.actor, "actor_carry"), (self.c.critic, "critic_carry")):
            if isinstance(net, RecurrentNetwork) and getattr(env, name) is None:
                setattr(env, name, net.initial_carry(self.N, self.done.device))
        n = reward_carry_size(self.c.rewards)
        if n and env.reward_carry is None:
            env.reward_carry = initial_reward_carry(self.c.rewards, self.N, self.done.device)

    def _rewards(self, traj: Trajectory, env: RolloutEnvState, level: float, want_components: bool = False) -> RewardState:
        """get_rewards over the recorded rollout; the carries of stateful rewards live in the env state (rl.py:1640-1650)."""
        self._prepare_env(env)
        return get_rewards(traj, self.c.rewards, self.c.reward_clip_min, self.c.reward_clip_max,
                           want_components=want_components, rewards_carry=env.reward_carry,
                           obs_slices=self.c.terms.obs_slices, level=level,
                           command_slices=self.c.commands.slices if self.c.commands is not None else None)

    def _command_leaves(self) -> dict:
        if self.command is None:
            return {}
        out = {name: self.command[..., sl] for name, sl in self.c.commands.slices.items()}
        out["_buffer"] = self.command
        return out

    def trajectory(self) -> Trajectory:
        names = list(self.c.terms.terminations)
        return Trajectory(qpos=self.qpos, qvel=self.qvel, xpos=self.xpos, xquat=self.xquat, ctrl=self.ctrl,
                          obs={"obs": self.obs, "noisy_obs": self.noisy_obs}, command=self._command_leaves(), event_state={},
                          action=self.action, done=self.done, success=self.success, timestep=self.timestep,
                          termination_components={n: self.components[:, j] for j, n in enumerate(names)})

    def ppo_inputs(self, rewards: RewardState, gamma: float, lam: float, normalize_advantages: bool = True):
        """GAE / returns over the rollout in its own (T, N) layout (ksim/task/ppo.py:54-121)."""
        if self.values is None:
            raise _lib.KsError("a critic is required for GAE")
        return ppo_mod.compute_ppo_inputs(self.values.view(self.T, self.N), rewards.total, self.done, self.success,
                                          gamma, lam, normalize_advantages=normalize_advantages, time_major=True)


_STREAMS: list = []


def _group_streams(n: int) -> list:
    """One pool of side streams for every SplitRollout of the process: a process has few hardware queues (4 by default),
    and streams beyond them share a queue, which serialises launches that were meant to overlap."""
    while len(_STREAMS) < n:
        _STREAMS.append(torch.cuda.Stream())
    return _STREAMS[:n]


class SplitRollout:
    """The same rollout with the N envs cut into `splits` independent groups, each on its own HIP stream.

    No counterpart in the reference, whose vmapped step runs all envs in lock step.  Here a control step is a chain of
    launches whose longest one, the fused physics step, ends with its slowest env, and the short launches around it
    (observation, networks, termination, reset pass) cannot fill the GPU on their own.  With two groups in flight the tail
    of one group's physics launch and its short launches overlap the other group's physics launch.  Envs never interact
    inside a rollout, so every env's trajectory is what the single-stream `Rollout` gives it for the same draws; only
    advantage normalisation spans the groups (`ppo_inputs`).  Streams are created at the default priority.
    """

    def __init__(self, constants: RolloutConstants, num_envs: int, rollout_length: int, splits: int = 2):
        if splits < 1 or num_envs % splits:
            raise _lib.KsError("the env count must be a multiple of the number of groups")
        if any(isinstance(n, RecurrentNetwork) for n in (constants.actor, constants.critic)):
            raise _lib.KsError("recurrent networks keep one workspace per cell: roll them out on a single stream")
        self.c, self.N, self.T, self.splits = constants, int(num_envs), int(rollout_length), int(splits)
        self.parts = [Rollout(constants, num_envs // splits, rollout_length) for _ in range(splits)]
        self.streams = _group_streams(splits)
        dev = torch.device("cuda")
        n = self.N // splits
        # GAE outputs of all groups side by side, so that advantage normalisation can run over their union
        self._gae = torch.empty(splits, self.T, n, dtype=torch.float32, device=dev)
        self._ret = torch.empty_like(self._gae)
        self._tgt = torch.empty_like(self._gae)
        self._adv = torch.empty_like(self._gae)
        self._ws = torch.empty(_lib.KS_REDUCE_WORKSPACE_BYTES, dtype=torch.uint8, device=dev)

    def fork(self) -> None:
        """The groups' streams wait for what the current stream has queued so far."""
        cur = torch.cuda.current_stream()
        for st in self.streams:
            st.wait_stream(cur)

    def join(self) -> None:
        """The current stream waits for the groups."""
        cur = torch.cuda.current_stream()
        for st in self.streams:
            cur.wait_stream(st)

    def step_engine(self, envs: Sequence[RolloutEnvState], t: int, level: float = 1.0,
                    noise: Sequence[Mapping | None] | None = None) -> None:
        """One control step of every group (no synchronisation: bracket a run of steps with `fork` and `join`)."""
        for g, (ro, env, st) in enumerate(zip(self.parts, envs, self.streams)):
            with torch.cuda.stream(st):
                ro.step_engine(env, t, level, noise[g] if noise is not None else None)

    def unroll(self, envs: Sequence[RolloutEnvState], level: float = 1.0, graph: bool = False) -> list[tuple[Trajectory, RewardState]]:
        """T control steps and the reward pass of every group; returns one (trajectory, rewards) per group.  With
        `graph=True` each group's launches are captured once as a HIP graph of its own and the graphs are replayed side by
        side on the groups' streams (`Rollout.unroll(graph=True)` per group): the same bits, without the per-launch host
        cost, which with two chains of launches to feed is what the eager path spends most of a step on."""
        if graph and any(ro._graph is None for ro in self.parts):
            for ro, env in zip(self.parts, envs):  # captures synchronise the device: do them before the groups fork
                ro._capture(env, level)
        self.fork()
        out = []
        if graph:
            for ro, env, st in zip(self.parts, envs, self.streams):
                with torch.cuda.stream(st):
                    out.append(ro.unroll(env, level, graph=True))
        else:
            for t in range(self.T):
                self.step_engine(envs, t, level)
            for ro, env, st in zip(self.parts, envs, self.streams):
                with torch.cuda.stream(st):
                    traj = ro.trajectory()
                    out.append((traj, ro._rewards(traj, env, level)))
        self.join()
        return out

    def ppo_inputs(self, rewards: Sequence[RewardState], gamma: float, lam: float, normalize_advantages: bool = True):
        """GAE / returns per group (ksim/task/ppo.py:54-121) with the advantages normalised over ALL envs, as one
        rollout of N envs has them (ppo.py:116-119).  Returns one PPOInputs per group (views of shared buffers)."""
        lib = _lib.load()
        self.fork()
        for g, (ro, rew, st) in enumerate(zip(self.parts, rewards, self.streams)):
            if ro.values is None:
                raise _lib.KsError("a critic is required for GAE")
            with torch.cuda.stream(st):
                _lib.check(lib.ks_gae_tn(_lib.current_stream(), ro.T, ro.N, _lib.ptr(ro.values), _lib.ptr(rew.total),
                                         _lib.ptr(ro.done), _lib.ptr(ro.success), float(gamma), float(lam), 0,
                                         _lib.ptr(self._gae[g]), _lib.ptr(self._ret[g]), _lib.ptr(self._tgt[g])))
        self.join()
        adv = self._gae
        if normalize_advantages:
            _lib.check(lib.ks_normalize_advantages(_lib.current_stream(), self._gae.numel(), _lib.ptr(self._gae),
                                                   _lib.ptr(self._adv), _lib.ptr(self._ws)))
            adv = self._adv
        return [ppo_mod.PPOInputs(advantages_bt=adv[g], value_targets_bt=self._tgt[g], gae_bt=self._gae[g],
                                  returns_bt=self._ret[g]) for g in range(self.splits)]
