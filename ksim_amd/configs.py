"""The benchmark workloads as ready-to-run rollouts (seeded, synthetic, random-init networks)."""
from __future__ import annotations

import numpy as np
import torch

from . import actuators, engine, model as km, observation as ob, physics, randomization as rnd, resets as rs
from . import rewards as rw, terminations as tm
from .env_terms import EnvTerms
from .mlp import MLP
from .rollout import Rollout, RolloutConstants, RolloutEnvState, SplitRollout

# soft torque limits by joint class (N m): legs (hip pitch/roll/yaw, knee, ankle), arms (shoulder x3, elbow, wrist)
KBOT_TORQUE_LIMITS = np.array([60.0, 40.0, 40.0, 60.0, 17.0] * 2 + [17.0, 17.0, 14.0, 14.0, 5.0] * 2)


def _net(dims, rng, last_scale=1.0, dtype="bf16"):
    ws = [rng.normal(scale=1.0 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])]
    ws[-1] *= last_scale
    bs = [np.zeros(o, dtype=np.float32) for o in dims[1:]]
    return MLP(ws, bs, activation="elu", dtype=dtype)


def integrator_name(model) -> str:
    """What a workload description must say about the velocity update of `model` (read off the model's own flag)."""
    return "implicitfast (damping-implicit)" if model.eulerdamp else "semi-implicit Euler"


def _kbot_constants(seed: int, hidden: int, dtype: str, min_height: float, integrator: str):
    m = km.kbot_scale_model(seed=seed, integrator=integrator)
    rng = np.random.default_rng(seed)
    kps = rng.uniform(20.0, 150.0, m.nu)
    kds = rng.uniform(0.5, 1.5, m.nu)
    act = actuators.PositionActuators(kps=tuple(kps), kds=tuple(kds), ctrl_clip=tuple(KBOT_TORQUE_LIMITS))
    resets = [rs.RandomJointPositionReset(scale=0.1, scale_by_curriculum=False)]
    eng = engine.get_physics_engine("hip", resets, {}, act, engine.EngineConfig(dt=0.005, ctrl_dt=0.02))
    noise = 0.01
    observations = {
        "joint_position": ob.JointPositionObservation(noise=noise),
        "joint_velocity": ob.JointVelocityObservation(noise=noise),
        "projected_gravity": ob.ProjectedGravityObservation(noise=noise),
        "base_angular_velocity": ob.BaseAngularVelocityObservation(in_robot_frame=True, noise=noise),
        "last_action": ob.LastActionObservation(),
        "command": ob.CommandObservation(),
    }
    terms = EnvTerms(m, observations, {"minimum_height": tm.MinimumHeightTermination(min_height)}, resets,
                     command_dim=2)
    dm = physics.DeviceModel(m)
    dev = torch.device("cuda")
    actor = _net((terms.obs_dim, hidden, hidden, hidden, m.nu), rng, last_scale=0.1, dtype=dtype)
    critic = _net((terms.obs_dim, hidden, hidden, hidden, 1), rng, dtype=dtype)
    rewards = {"stay_alive": rw.StayAliveReward(scale=1.0), "base_height": rw.BaseHeightReward(scale=0.5, height_target=0.87),
               "upright": rw.UprightReward(scale=0.2), "action_velocity": rw.ActionVelocityPenalty(scale=0.01)}
    consts = RolloutConstants(physics_model=dm, engine=eng, terms=terms, rewards=rewards, actor=actor, critic=critic,
                              log_std=torch.full((m.nu,), -2.0, device=dev), defer_reset_forward=True)
    return m, consts, dict(kps=kps, kds=kds, clip=KBOT_TORQUE_LIMITS)


def _kbot_env_state(m, consts, num_envs: int, seed: int) -> RolloutEnvState:
    dev = torch.device("cuda")
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    randomization = rnd.get_physics_randomizers(
        m, {"floor_friction": rnd.FloorFrictionRandomizer(0.4, 1.2),
            "mass": rnd.AllBodiesMassMultiplicationRandomizer(0.9, 1.1)}, num_envs, gen)
    ps = consts.engine.reset(consts.physics_model, 1.0, gen, num_envs, randomization)
    return RolloutEnvState(ps, randomization, torch.zeros(num_envs, 2, device=dev), None, seed=seed)


def kbot_rollout(num_envs: int = 8192, rollout_length: int = 32, seed: int = 1004, hidden: int = 512,
                 dtype: str = "bf16", min_height: float = 0.5, integrator: str = "euler"):
    """K-Bot-scale biped rollout: free root + 20 hinges, 8 foot spheres, per-env friction ~U(0.4,1.2) and
    mass scale ~U(0.9,1.1), observation noise N(0,0.01), reset on base height < `min_height`, actor and critic
    3 x `hidden` MLPs, dt 0.005 with 4 physics substeps per control step.  `integrator`: "euler" (semi-implicit
    Euler, what the benchmark configs name) or "implicitfast" (what ksim's RLConfig selects, ksim/task/rl.py:555-578)."""
    m, consts, gains = _kbot_constants(seed, hidden, dtype, min_height, integrator)
    # one chain of launches: the next step's observation rides in the launch that ends a step (measured +0.6 % here; with
    # two groups on two streams the longer launch costs more than the saved one gains, so the split rollout leaves it off)
    consts.fuse_next_observation = True
    env = _kbot_env_state(m, consts, num_envs, seed)
    return consts, env, Rollout(consts, num_envs, rollout_length), gains


def kbot_split_rollout(num_envs: int = 8192, rollout_length: int = 32, splits: int = 2, seed: int = 1004, hidden: int = 512,
                       dtype: str = "bf16", min_height: float = 0.5, integrator: str = "euler"):
    """The same workload with the envs in `splits` groups on separate streams (`SplitRollout`): returns the constants,
    one env state per group (seeded seed, seed + 1, ...) and the split rollout."""
    m, consts, _ = _kbot_constants(seed, hidden, dtype, min_height, integrator)
    envs = [_kbot_env_state(m, consts, num_envs // splits, seed + g) for g in range(splits)]
    return consts, envs, SplitRollout(consts, num_envs, rollout_length, splits)


def kbot_lstm_rollout(num_envs: int = 4096, rollout_length: int = 100, seed: int = 1006, integrator: str = "euler"):
    """The K-Bot-scale rollout with the K-Bot example's policy instead of the benchmark's MLPs (examples/kbot/train.py:80-95,
    837-995, 1754-1757): LSTM actor and critic, projection -> 2 x 128 -> linear head in fp32, the actor's head means |
    deviations with a mean bias and the one-pole low-pass (10 Hz) whose state rides in the model carry; 4096 envs, 2 s of
    control steps per rollout.  The critic runs on a side stream (RolloutConstants.critic_on_side_stream)."""
    import dataclasses

    from .actions import LowPass
    from .recurrent import LSTMCell, RecurrentNetwork
    from .rollout import GaussianHead

    m, consts, gains = _kbot_constants(seed, 512, "bf16", 0.5, integrator)
    rng = np.random.default_rng(seed)
    H, I, nu = 128, consts.terms.obs_dim, m.nu

    def net(out_dim: int, last_scale: float) -> RecurrentNetwork:
        proj = (rng.normal(size=(H, I)) / np.sqrt(I), np.zeros(H))
        cells = [LSTMCell(rng.normal(size=(4 * H, H)) / np.sqrt(H), rng.normal(size=(4 * H, H)) / np.sqrt(H), np.zeros(4 * H), dtype="f32")
                 for _ in range(2)]
        out = MLP([last_scale * rng.normal(size=(out_dim, H)) / np.sqrt(H)], [np.zeros(out_dim)], activation="none", dtype="f32")
        return RecurrentNetwork(proj, cells, out, dtype="f32")

    head = GaussianHead(min_std=0.01, max_std=1.0, var_scale=0.5, mean_bias=torch.zeros(nu, device="cuda"),
                        lowpass=LowPass(ctrl_dt=0.02, cutoff_frequency=10.0))
    consts = dataclasses.replace(consts, actor=net(2 * nu, 0.1), critic=net(1, 1.0), log_std=None, head=head,
                                 critic_on_side_stream=True)
    env = _kbot_env_state(m, consts, num_envs, seed)
    return consts, env, Rollout(consts, num_envs, rollout_length), gains


def humanoid_rollout(num_envs: int = 4096, rollout_length: int = 16, seed: int = 1003, min_height: float = 0.6):
    """Benchmark config 3: free root + 21 hinges in a 5-limb tree, 4 foot spheres, friction 1.0, 21 PD actuators, root height
    1.3 m, joints ~U(-0.1, 0.1), dt 0.005 with 4 substeps, fp32 actor 71 -> 3 x 256 (ELU) -> 21 means."""
    m = km.humanoid_model(seed=seed)
    rng = np.random.default_rng(seed)
    act = actuators.PositionActuators(kps=tuple(rng.uniform(20.0, 150.0, m.nu)), kds=tuple(rng.uniform(0.5, 1.5, m.nu)))
    resets = [rs.RandomJointPositionReset(scale=0.1, scale_by_curriculum=False)]
    eng = engine.get_physics_engine("hip", resets, {}, act, engine.EngineConfig(dt=0.005, ctrl_dt=0.02))
    observations = {
        "joint_position": ob.JointPositionObservation(), "joint_velocity": ob.JointVelocityObservation(),
        "projected_gravity": ob.ProjectedGravityObservation(),
        "base_angular_velocity": ob.BaseAngularVelocityObservation(in_robot_frame=True),
        "last_action": ob.LastActionObservation(), "command": ob.CommandObservation(),
    }
    terms = EnvTerms(m, observations, {"minimum_height": tm.MinimumHeightTermination(min_height)}, resets, command_dim=2)
    assert terms.obs_dim == 71
    dm = physics.DeviceModel(m)
    dev = torch.device("cuda")
    actor = _net((71, 256, 256, 256, m.nu), rng, last_scale=0.1, dtype="f32")
    critic = _net((71, 256, 256, 256, 1), rng, dtype="f32")
    rewards = {"stay_alive": rw.StayAliveReward(scale=1.0), "upright": rw.UprightReward(scale=0.2)}
    consts = RolloutConstants(physics_model=dm, engine=eng, terms=terms, rewards=rewards, actor=actor, critic=critic,
                              log_std=torch.full((m.nu,), -2.0, device=dev))
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    ps = eng.reset(dm, 1.0, gen, num_envs, {})
    ps.data.qpos[:, 2] = 1.3
    eng.forward(dm, ps)
    env = RolloutEnvState(ps, {}, torch.zeros(num_envs, 2, device=dev), None, seed=seed)
    return consts, env, Rollout(consts, num_envs, rollout_length)


def kbot_ppo_iteration(num_envs: int = 16384, rollout_length: int = 32, seed: int = 1005, batch_size: int = 2048,
                       num_passes: int = 4, integrator: str = "euler"):
    """Benchmark config 5: the K-Bot-scale rollout with T = 32, then `num_passes` epochs of minibatch steps of the bf16 actor
    and critic, and an AMP-style discriminator 71 -> 2 x 256 -> 1 scoring the trajectory's motion frames against seeded
    reference-motion frames ~N(0, 1).  Returns what `train_step.rl_train_loop_step` takes."""
    from .amp import AMPConfig, DiscriminatorUpdate
    from .ppo_update import GaussianMlpPolicy, PPOUpdateConfig
    from .train_step import AMPSetup

    m, consts, _ = _kbot_constants(seed, 512, "bf16", 0.5, integrator)
    consts.rewards = dict(consts.rewards, amp=rw.AMPReward(scale=0.5))
    env = _kbot_env_state(m, consts, num_envs, seed)
    rng = np.random.default_rng(seed)
    frame = (m.nq - 2) + m.nv + m.nu
    disc = _net((frame, 256, 256, 1), rng, dtype="bf16")
    real = torch.from_numpy(rng.normal(size=(64, rollout_length, frame)).astype(np.float32)).cuda()
    setup = AMPSetup(update=DiscriminatorUpdate(disc, AMPConfig(amp_reference_batch_size=32, disc_num_passes=1)), real_motions=real)
    policy = GaussianMlpPolicy(actor=consts.actor, critic=consts.critic, log_std=consts.log_std)
    cfg = PPOUpdateConfig(num_passes=num_passes, batch_size=batch_size)
    return consts, env, Rollout(consts, num_envs, rollout_length), policy, cfg, setup


def step_algorithmic_bytes(m, obs_dim: int, per_env_params: int) -> int:
    """Bytes one fused control step is obliged to move per env: state in/out, transition record, observation."""
    return 4 * (2 * m.nq + 4 * m.nv + 3 * m.nu + 1 + 7 * m.nb + obs_dim + per_env_params) + 2
