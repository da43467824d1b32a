"""End-to-end rollout (obs -> MLP -> action -> fused physics -> termination -> reset -> record) vs the oracle."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from dyn_common import rel_err
from oracle import ppo as oppo
from oracle import terms as ot
from oracle.dyn import Oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def t32(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32, device=DEV).contiguous()


# per-episode sim2real quantities of the `sim2real` builds, as the oracle's engine_reset_draws takes them
SIM2REAL = dict(latency_range=(1.0, 3.0), zero_offset=dict(mean=0.0, mag=0.0, std=0.01),
                action_bias=dict(mean=0.0, mag=0.02, std=0.0), torque_bias=dict(mean=0.0, mag=0.0, std=0.3),
                kp_scale=dict(mean=1.0, mag=0.1, std=0.0), kd_scale=dict(mean=1.0, mag=0.0, std=0.05),
                torque_limit_scale=dict(mean=0.95, mag=0.05, std=0.0))


def build(N, T, seed=0, min_height=0.9, events=None, gait=False, recurrent=False, head=None, sim2real=False):
    from ksim_amd import actuators, engine, model as km, observation as ob, physics, randomization as rnd, resets as rs
    from ksim_amd import rewards as rw, terminations as tm
    from ksim_amd.env_terms import EnvTerms
    from ksim_amd.mlp import MLP
    from ksim_amd.rollout import Rollout, RolloutConstants, RolloutEnvState

    m = km.kbot_scale_model()
    rng = np.random.default_rng(seed)
    # kd * dt / (armature + link inertia) must stay below 1 for the explicit damping term to be stable
    kps, kds = rng.uniform(20, 150, m.nu), rng.uniform(0.5, 1.5, m.nu)
    clip = np.tile([60.0, 40.0, 40.0, 60.0, 17.0], 4); clip[10:] = [17.0, 17.0, 14.0, 14.0, 5.0] * 2
    act = actuators.PositionActuators(kps=tuple(kps), kds=tuple(kds), ctrl_clip=tuple(clip))
    resets = [rs.RandomJointPositionReset(scale=0.1, scale_by_curriculum=False)]
    cfg = engine.EngineConfig(dt=0.005, ctrl_dt=0.02)
    if sim2real:  # what ksim's sim2real knobs add: every one of these is drawn afresh for each episode
        from ksim_amd import noise as kn
        act = actuators.PositionActuators(kps=tuple(kps), kds=tuple(kds), ctrl_clip=tuple(clip),
                                          action_bias=kn.UniformRandomVariable(0.0, 0.02), torque_bias=kn.GaussianRandomVariable(0.0, 0.3),
                                          kp_scale=kn.UniformRandomVariable(1.0, 0.1), kd_scale=kn.GaussianRandomVariable(1.0, 0.05),
                                          torque_limit_scale=kn.UniformRandomVariable(0.95, 0.05))
        cfg = engine.EngineConfig(dt=0.005, ctrl_dt=0.02, action_latency_range=(0.005, 0.015), zero_offset_std=0.01)
    eng = engine.get_physics_engine("hip", resets, events or {}, act, cfg)
    observations = {"jp": ob.JointPositionObservation(noise=0.01),
                    "jv": ob.JointVelocityObservation(noise=0.01, bias=0.02 if sim2real else None),
                    "g": ob.ProjectedGravityObservation(noise=0.01),
                    "w": ob.BaseAngularVelocityObservation(in_robot_frame=True, noise=0.01),
                    "a": ob.LastActionObservation(), "c": ob.CommandObservation()}
    if gait:  # what a walking task adds: contact flags, foot positions, sensor lag, and the gait rewards over them
        feet = [b for b in range(m.nb) if any(int(sb) == b for sb in m.sph_body)]
        left = tuple(i for i, sb in enumerate(m.sph_body) if int(sb) == feet[0])
        right = tuple(i for i, sb in enumerate(m.sph_body) if int(sb) == feet[1])
        observations.update({"contact": ob.FeetContactObservation(foot_left=left, foot_right=right),
                             "feet_pos": ob.BodyPositionObservation(body_ids=tuple(feet)),
                             "old_jp": ob.DelayedJointPositionObservation(delay_steps=2),
                             "imu_g": ob.ProjectedGravityObservation(min_lag=0.2, max_lag=0.6, imu_bias=0.02)})
    commands = None
    if gait:  # the walking tasks' commands: 6 + 2 floats instead of the two constants
        from ksim_amd.commands import AngularVelocityCommand, CommandSet, LinearVelocityCommand
        commands = CommandSet({"lin": LinearVelocityCommand(min_vel=0.2, max_vel=1.0, max_yaw=0.3, zero_prob=0.1, backward_prob=0.2,
                                                            switch_prob=0.05, ctrl_dt=0.02, linear_accel=1.0, angular_accel=1.0),
                               "ang": AngularVelocityCommand(max_vel=0.5, zero_prob=0.2, switch_prob=0.05, ctrl_dt=0.02, angular_accel=1.0)})
        observations["feet_force"] = ob.FeetTorqueObservation(foot_left=feet[0], foot_right=feet[1])
    terms = EnvTerms(m, observations, {"min_height": tm.MinimumHeightTermination(min_height)}, resets,
                     command_dim=commands.command_dim if commands else 2)
    dims = (terms.obs_dim, 64, 64, m.nu)
    ws = [rng.normal(scale=1 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])]
    ws[-1] *= 0.1  # small final layer: actions stay near the PD set point
    bs = [np.zeros(o, np.float32) for o in dims[1:]]
    cdims = (terms.obs_dim, 64, 1)
    cws = [rng.normal(scale=1 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(cdims[:-1], cdims[1:])]
    cbs = [np.zeros(o, np.float32) for o in cdims[1:]]
    dm = physics.DeviceModel(m)
    log_std = np.full(m.nu, -2.0, np.float32)
    rewards = {"stay_alive": rw.StayAliveReward(scale=1.0), "height": rw.BaseHeightReward(scale=0.5, height_target=1.0),
               "vel": rw.ActionVelocityPenalty(scale=0.01)}
    if gait:
        rewards.update({"air_time": rw.FeetAirTimeReward(scale=1.0, gait_period=0.2, air_time_percent=0.5, ctrl_dt=0.02,
                                                         contact_obs="contact", linvel_moving_threshold=0.05),
                        "step_height": rw.SparseTargetHeightReward(scale=2.0, contact_obs="contact", position_obs="feet_pos",
                                                                   height=0.1, linvel_moving_threshold=0.02),
                        "track_lin": rw.LinearVelocityReward(scale=0.5, cmd="lin"),
                        "track_ang": rw.AngularVelocityReward(scale=0.25, cmd="ang"),
                        "rest": rw.MotionlessAtRestPenalty(scale=0.01),
                        "force": rw.ForcePenalty(scale=0.01, force_obs="feet_force", expected_weight=200.0)})
    actor, critic = MLP(ws, bs, dtype="f32"), MLP(cws, cbs, dtype="f32")
    if recurrent:  # the shape of the shipped examples' networks: projection, GRU stack, GELU / ELU output MLP
        from ksim_amd.recurrent import GRUCell, RecurrentNetwork
        H = 32
        def cell():
            s_ = 1 / np.sqrt(H)
            return (rng.uniform(-s_, s_, (3 * H, H)), rng.uniform(-s_, s_, (3 * H, H)), rng.uniform(-s_, s_, 3 * H), rng.uniform(-s_, s_, H))
        def net(out, act):
            proj = (rng.normal(size=(H, terms.obs_dim)) / np.sqrt(terms.obs_dim), np.zeros(H))
            cells = [cell() for _ in range(2)]
            ow, ob_ = [rng.normal(size=(H, H)) / np.sqrt(H), 0.1 * rng.normal(size=(out, H)) / np.sqrt(H)], [np.zeros(H), np.zeros(out)]
            n = RecurrentNetwork(proj, [GRUCell(*c_, dtype="f32") for c_ in cells], MLP(ow, ob_, activation=act, dtype="f32"), dtype="f32")
            n.params = (proj, cells, ow, ob_)
            return n
        head_bias = t32(rng.normal(size=m.nu) * 0.05)
        if head == "gaussian":   # means | raw deviations, deviations squeezed to ~0 so that the sample shows the mean
            from ksim_amd.rollout import GaussianHead
            head = GaussianHead(min_std=0.0, max_std=1e-6, mean_bias=head_bias)
        elif head in ("gaussian-lowpass", "kbot"):
            # the K-Bot actor: the biased means (bias vector + two observation columns on the last two joints) pass a
            # one-pole low-pass whose state rides in the model carry (examples/kbot/train.py:917-929)
            from ksim_amd.actions import LowPass
            from ksim_amd.rollout import GaussianHead
            lp = LowPass(ctrl_dt=0.02, cutoff_frequency=4.0, obs_bias=(0, m.nu - 2, 2))
            head = (GaussianHead(min_std=0.0, max_std=1e-6, mean_bias=head_bias, lowpass=lp) if head == "gaussian-lowpass"
                    else GaussianHead(min_std=0.05, max_std=0.5, var_scale=0.5, mean_bias=head_bias, lowpass=lp))
        elif head == "gaussian-wide":   # deviations a policy update can work with
            from ksim_amd.rollout import GaussianHead
            head = GaussianHead(min_std=0.05, max_std=0.5, var_scale=0.5, mean_bias=head_bias)
        elif head == "mixture":
            from ksim_amd.rollout import MixtureHead
            head = MixtureHead(num_mixtures=2, min_std=0.0, max_std=1e-6, mean_bias=head_bias,
                               clip_lo=t32(np.full(m.nu, -0.3)), clip_hi=t32(np.full(m.nu, 0.3)))
        elif head == "mixture-wide":
            from ksim_amd.rollout import MixtureHead
            head = MixtureHead(num_mixtures=3, min_std=0.05, max_std=0.5, var_scale=0.5, mean_bias=head_bias,
                               clip_lo=t32(np.full(m.nu, -0.6)), clip_hi=t32(np.full(m.nu, 0.6)))
        actor, critic = net(m.nu if head is None else head.width(m.nu), "gelu"), net(1, "elu")
    consts = RolloutConstants(physics_model=dm, engine=eng, terms=terms, rewards=rewards,
                              actor=actor, critic=critic, log_std=t32(log_std), commands=commands, head=head)
    gen = torch.Generator(device=DEV); gen.manual_seed(seed)
    randomization = rnd.get_physics_randomizers(m, {"f": rnd.FloorFrictionRandomizer(0.4, 1.2),
                                                    "m": rnd.AllBodiesMassMultiplicationRandomizer(0.9, 1.1)}, N, gen)
    return m, consts, randomization, (ws, bs, cws, cbs, log_std, kps, kds, clip), Rollout(consts, N, T), RolloutEnvState


def test_critic_on_a_side_stream_gives_the_same_rollout():
    """A recurrent critic on a stream of its own, beside the actor and the physics launch and joined before the termination
    pass: actions, values, carries and flags bit for bit those of the single chain, eagerly and under graph replay, over
    rollouts in which episodes end (so the critic reads reset masks that the next termination pass rewrites)."""
    import dataclasses
    from ksim_amd.rollout import Rollout

    N, T = 24, 8
    runs = {}
    for side, use_graph in ((False, False), (True, False), (True, True)):
        m, c, rnd_, _, ro, EnvState = build(N, T, seed=13, min_height=0.95, recurrent=True, head="kbot")
        if side:
            c = dataclasses.replace(c, critic_on_side_stream=True)
            ro = Rollout(c, N, T)
        ps = c.engine.reset(c.physics_model, 1.0, 3, N, rnd_)
        env = EnvState(ps, rnd_, torch.zeros(N, 2, device=DEV), None, seed=21)
        snaps, finished = [], 0
        for it in range(4):
            traj, rew = ro.unroll(env, graph=use_graph)
            torch.cuda.synchronize()
            finished += int(traj.done.sum().item())
            snaps.append((traj.action.clone(), ro.values.clone(), env.actor_carry.clone(), env.critic_carry.clone(), traj.done.clone(),
                          rew.total.clone()))
        assert finished > 0
        runs[(side, use_graph)] = snaps
    for key in ((True, False), (True, True)):
        for a, b in zip(runs[(False, False)], runs[key]):
            assert all(torch.equal(x, y) for x, y in zip(a, b)), key


def _mlp64(x, ws, bs):
    h = torch.from_numpy(np.asarray(x, dtype=np.float64))
    for i, (w, b) in enumerate(zip(ws, bs)):
        h = F.linear(h, torch.from_numpy(w).double(), torch.from_numpy(b).double())
        if i + 1 < len(ws):
            h = F.elu(h)
    return h.numpy()


@pytest.mark.parametrize("sim2real", [False, True])
def test_rollout_matches_oracle_composition(sim2real):
    """`sim2real`: action latency, zero offset, actuator gain / bias randomisation and an observation bias, all of which the
    reference draws per episode (ksim/engine.py:222-245, ksim/actuators.py:219-238, ksim/task/rl.py:1110-1117): an env that
    is reset during the rollout must continue with the oracle's re-draw, the others with what they had."""
    N, T = 12, 3
    m, c, rnd_, (ws, bs, cws, cbs, log_std, kps, kds, clip), ro, EnvState = build(N, T, seed=5, sim2real=sim2real)
    rng = np.random.default_rng(6)
    K, nu, ned = c.terms.obs_dim, m.nu, 3 * m.nu + 4
    u0 = rng.uniform(-1, 1, (N, m.nq + 1))
    eu, ez = rng.uniform(-1, 1, (N, ned)), rng.normal(size=(N, ned))
    ps = c.engine.reset(c.physics_model, 1.0, 0, N, rnd_, reset_uniform=t32(u0), episode_draws=dict(uniform=t32(eu), normal=t32(ez)))
    spec = SIM2REAL if sim2real else dict(latency_range=(0.0, 0.0), zero_offset=None)
    epi = [ot.engine_reset_draws(nu, 1.0, eu[e], ez[e], **spec) for e in range(N)]  # the oracle's per-episode quantities
    bias_zw = np.zeros((N, K, 2))
    # a third of the envs start just below the termination height (feet touching), so they finish on the first step
    low = np.arange(N) % 3 == 0
    ps.data.qpos[torch.from_numpy(low).to(DEV), 2] = 0.87
    cmd = rng.normal(size=(N, 2))
    env = EnvState(ps, rnd_, t32(cmd), None, seed=1)
    fr, ms = rnd_["friction"].cpu().numpy().astype(np.float64), rnd_["mass_scale"].cpu().numpy().astype(np.float64)
    # ---- oracle side state
    orc = Oracle(m.arrays())
    q0 = ps.data.qpos.cpu().numpy().astype(np.float64)
    want_q0 = np.tile(m.qpos0, (N, 1)); want_q0[:, 7:] += 0.1 * u0[:, 7:m.nq]
    np.testing.assert_allclose(q0[~low], want_q0[~low], atol=1e-6)  # engine.reset applied the reset table
    datas = [orc.data(q0[e], friction=fr[e], mass_scale=ms[e]) for e in range(N)]
    for d in datas:
        orc.forward(d)  # engine.py:213 — warm start of the fresh episode
        d.qvel = 0.0
    last = np.zeros((N, m.nu))
    fresh = np.ones(N, bool)  # every env starts an episode at the first step
    for t in range(T):
        noise = dict(obs_normal=rng.normal(size=(N, K)), obs_uniform=rng.random((N, K)),
                     action_normal=rng.normal(size=(N, m.nu)), reset_uniform=rng.uniform(-1, 1, (N, m.nq + 1)),
                     obs_bias_redraw=np.stack([rng.normal(size=(N, K)), rng.uniform(-1, 1, (N, K))], -1),
                     episode=dict(uniform=rng.uniform(-1, 1, (N, ned)), normal=rng.normal(size=(N, ned))))
        ro.step_engine(env, t, 1.0, {k: ({kk: t32(vv) for kk, vv in v.items()} if isinstance(v, dict) else t32(v))
                                     for k, v in noise.items()})
        # oracle: observation; the envs that start an episode take new bias draws first (rl.py:1110-1117)
        bias_zw[fresh] = noise["obs_bias_redraw"][fresh]
        zo = np.array([ep["zero_offset"] for ep in epi])
        q = np.array([np.array(d.qpos) for d in datas]); v = np.array([np.array(d.qvel) for d in datas])
        g = ot.rotate_vector_by_quat(np.broadcast_to([0, 0, -9.81], (N, 3)), q[:, 3:7], inverse=True)
        w = ot.rotate_vector_by_quat(v[:, 3:6], q[:, 3:7], inverse=True)
        obs = np.concatenate([q[:, 7:] - zo, v[:, 6:], g, w, last, cmd], axis=1)
        noisy = obs.copy(); noisy[:, : 2 * m.nu + 6] += 0.01 * noise["obs_normal"][:, : 2 * m.nu + 6]
        if sim2real:
            noisy[:, nu:2 * nu] += 0.02 * bias_zw[:, nu:2 * nu, 0]
            np.testing.assert_allclose(ro.noisy_obs[t].cpu().numpy(), noisy, rtol=1e-4, atol=2e-4)
        np.testing.assert_allclose(ro.obs[t].cpu().numpy(), obs, rtol=1e-4, atol=2e-4)
        mean = _mlp64(noisy, ws, bs)
        action = ot.scrub_action(mean + np.exp(log_std.astype(np.float64)) * noise["action_normal"])
        np.testing.assert_allclose(ro.action[t].cpu().numpy(), action, rtol=1e-3, atol=2e-3)
        value = _mlp64(obs, cws, cbs)
        np.testing.assert_allclose(ro.values[t].cpu().numpy(), value, rtol=1e-3, atol=2e-3)
        # oracle: physics (4 substeps, blend + PD), termination, reset
        for e, d in enumerate(datas):
            tau = np.zeros(m.nu)
            ep = epi[e]
            for s in range(4):
                ctl = ot.latency_blend(float(s), ep["action_latency"], last[e], action[e], np.zeros(m.nu, bool))
                tau = ot.position_actuator_torque(ctl, np.array(d.qpos[7:]) - ep["zero_offset"], np.array(d.qvel[6:]), kps, kds, clip,
                                                  action_bias=ep["action"], torque_bias=ep["torque"], kp_scale=ep["kp_scale"],
                                                  kd_scale=ep["kd_scale"], torque_limit_scale=ep["torque_limit_scale"])
                d.ctrl = tau
                orc.step(d)
        last = action.copy()
        q = np.array([np.array(d.qpos) for d in datas]); v = np.array([np.array(d.qvel) for d in datas])
        term = ot.minimum_height_termination(q, 0.9)
        done, succ = ot.combine_terminations([term])
        assert np.array_equal(ro.done[t].cpu().numpy().astype(bool), done), f"done mask differs at step {t}"
        assert np.array_equal(ro.success[t].cpu().numpy().astype(bool), succ)
        assert np.array_equal(ro.components[t][0].cpu().numpy(), term)
        tol = 1e-4 if t == 0 else 1e-3
        assert rel_err(ro.qpos[t].cpu().numpy(), q).max() <= tol, rel_err(ro.qpos[t].cpu().numpy(), q).max()
        assert rel_err(ro.qvel[t].cpu().numpy(), v, floor=1e-2).max() <= tol
        xp = np.array([np.array(d.xpos).reshape(-1) for d in datas])
        assert rel_err(ro.xpos[t].cpu().numpy(), xp).max() <= tol
        np.testing.assert_allclose(ro.timestep[t].cpu().numpy(), [d.time for d in datas], rtol=1e-5)
        for e in np.where(done)[0]:
            nq = m.qpos0.copy(); nq[7:] += 0.1 * noise["reset_uniform"][e, 7:m.nq]
            datas[e] = orc.data(nq, friction=fr[e], mass_scale=ms[e])
            orc.forward(datas[e])
            last[e] = 0.0
            epi[e] = ot.engine_reset_draws(nu, 1.0, noise["episode"]["uniform"][e], noise["episode"]["normal"][e], **spec)
        fresh = done.copy()
        if sim2real:  # the live per-episode state: re-drawn where an episode ended, untouched elsewhere
            got = dict(action_latency=ps.action_latency, zero_offset=ps.zero_offset, **ps.actuator_state)
            for k, buf in got.items():
                np.testing.assert_allclose(buf.cpu().numpy(), np.array([ep[k] for ep in epi]), rtol=2e-6, atol=2e-7, err_msg=k)
        if t == 0:
            assert done.sum() == low.sum()
        # sphere-floor distances of the last collision pass (data.contact.dist): of the last substep for the envs that go
        # on, of the forward pass over the fresh state for the envs that were reset
        cd = np.array([np.array(d.con_dist) for d in datas])
        np.testing.assert_allclose(ps.data.contact_dist.cpu().numpy(), cd, rtol=0, atol=2e-5)
    # live state after the rollout: reset envs restarted, others continued
    q = np.array([np.array(d.qpos) for d in datas])
    assert rel_err(ps.data.qpos.cpu().numpy(), q).max() <= 1e-3
    # rewards + GAE over the recorded rollout, against the oracle on the recorded arrays
    traj = ro.trajectory()
    from ksim_amd.rewards import get_rewards
    rew = get_rewards(traj, c.rewards)
    a_, dn, sc, qq = (x.cpu().numpy() for x in (ro.action, ro.done, ro.success, ro.qpos))
    tot = np.stack([ot.stay_alive_reward(dn[:, e].astype(bool), sc[:, e].astype(bool)) + 0.5 * ot.base_height_reward(qq[:, e], 1.0)
                    - 0.01 * ot.action_velocity_penalty(a_[:, e], dn[:, e].astype(bool)) for e in range(N)], axis=1)
    np.testing.assert_allclose(rew.total.cpu().numpy(), tot, rtol=1e-5, atol=1e-5)
    inp = ro.ppo_inputs(rew, 0.99, 0.95, normalize_advantages=False)
    vals = ro.values.view(T, N).cpu().numpy()
    want = oppo.compute_ppo_inputs(vals.T, rew.total.cpu().numpy().T, dn.T, sc.T, 0.99, 0.95)
    np.testing.assert_allclose(inp.gae_bt.cpu().numpy(), want["gae"].T, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(inp.returns_bt.cpu().numpy(), want["returns"].T, rtol=1e-5, atol=1e-5)


def test_long_rollout_with_resets_stays_finite_and_reproducible():
    """Philox mode: 200 control steps with resets; two runs with one seed are bit-identical."""
    N, T = 256, 8
    outs = []
    for _ in range(2):
        m, c, rnd_, _, ro, EnvState = build(N, T, seed=11, min_height=0.7)
        ps = c.engine.reset(c.physics_model, 1.0, 3, N, rnd_)
        env = EnvState(ps, rnd_, torch.zeros(N, 2, device=DEV), None, seed=77)
        ndone = 0
        for _ in range(25):
            traj, rew = ro.unroll(env)
            ndone += int(traj.done.sum().item())
            assert torch.isfinite(traj.qpos).all() and torch.isfinite(rew.total).all()
        outs.append((ps.data.qpos.clone(), ndone, env.episode_length.clone()))
    assert outs[0][1] > 0, "no env ever terminated: the reset path was not exercised"
    assert torch.equal(outs[0][0], outs[1][0]) and outs[0][1] == outs[1][1]
    assert torch.equal(outs[0][2], outs[1][2])
    assert (outs[0][0][:, 2] > 0.5).all()  # every env sits above the termination height after its reset


def _push_events(force=False):
    from ksim_amd import events as kev
    evs = {"push": kev.LinearPushEvent(linvel=0.5, interval_range=(0.05, 0.3)),
           "spin": kev.AngularPushEvent(angvel=0.5, interval_range=(0.1, 0.4)),
           "jump": kev.JumpEvent(jump_height_range=(0.01, 0.05), interval_range=(0.2, 0.6))}
    if force:
        evs["shove"] = kev.ForcePushEvent(max_force=60.0, max_torque=5.0, duration_range=(0.05, 0.2),
                                          interval_range=(0.1, 0.5), body_id=1)
    return evs


@pytest.mark.parametrize("with_events,sim2real", [(False, False), (True, False), (False, True)])
def test_graph_replay_equals_eager_rollout(with_events, sim2real):
    """A captured rollout graph, replayed several times with eager work and synchronisations in between, gives
    the same bits as the eager loop on every replay (same Philox keys: device step counter + baked step)."""
    N, T, iters = 192, 8, 10
    runs = []
    for use_graph in (False, True):
        m, c, rnd_, _, ro, EnvState = build(N, T, seed=5, min_height=0.8, events=_push_events(force=True) if with_events else None,
                                            sim2real=sim2real)
        ps = c.engine.reset(c.physics_model, 1.0, 3, N, rnd_)
        env = EnvState(ps, rnd_, torch.zeros(N, 2, device=DEV), None, seed=123)
        snaps, pushed = [], False
        lat0 = ps.action_latency.clone()
        for it in range(iters):
            traj, rew = ro.unroll(env, graph=use_graph)
            torch.cuda.synchronize()
            snaps.append((traj.qpos.clone(), traj.action.clone(), traj.done.clone(), rew.total.clone(),
                          ps.data.qpos.clone(), env.episode_length.clone()))
            if sim2real:  # the per-episode draws are part of what a replay must reproduce
                snaps[-1] += (ps.action_latency.clone(), ps.zero_offset.clone(), ps.actuator_state["kp_scale"].clone(),
                              ps.actuator_state["torque"].clone(), env.obs_bias.clone())
            if with_events:
                shove = ps.event_states["shove"]  # (time remaining, duration left, wrench) like the reference's tuple
                snaps[-1] += (ps.event_states["_buffer"].clone(), shove[1].clone(), shove[2].clone())
                pushed |= bool((shove[2].abs().amax(dim=1) > 0).any())
            junk = torch.randn(512, 512, device=DEV)  # unrelated eager work between replays
            (junk @ junk).sum().item()
        assert env.step == iters * T
        assert pushed or not with_events, "no force push was ever drawn"
        if sim2real:
            changed = (ps.action_latency != lat0).float().mean().item()
            assert 0.02 < changed < 1.0, f"latency re-drawn for {changed:.2f} of the envs: expected only those that were reset"
        runs.append(snaps)
    assert sum(int(s[2].sum().item()) for s in runs[0]) > 0, "no resets happened: the reset path was not replayed"
    for it, (a, b) in enumerate(zip(*runs)):
        names = ("qpos", "action", "done", "reward", "state", "episode_length") + (
            ("latency", "zero offset", "kp scale", "torque bias", "observation bias draws") if sim2real else
            ("event timers", "force duration", "held wrench"))
        for x, y, name in zip(a, b, names):
            assert torch.equal(x, y), f"replay {it}: {name} differs from the eager rollout"


def test_events_in_the_rollout_fire_and_restart_with_the_episode():
    """Event timers through the environment loop: explicit draws, one control step; envs that continue carry
    the kernel's timers (fired ones re-armed from the draw), envs that finish get fresh timers from the reset draw
    (ksim/engine.py:226-232), and the pushes change the state relative to a run without events."""
    N, T = 12, 2
    evs = _push_events()
    m, c, rnd_, _, ro, EnvState = build(N, T, seed=5, events=evs)
    _, c0, rnd0, _, ro0, _ = build(N, T, seed=5)
    rng = np.random.default_rng(8)
    u0 = t32(rng.uniform(-1, 1, (N, m.nq + 1)))
    ps = c.engine.reset(c.physics_model, 1.0, 0, N, rnd_, reset_uniform=u0)
    ps0 = c0.engine.reset(c0.physics_model, 1.0, 0, N, rnd0, reset_uniform=u0)
    names = list(evs)
    assert set(ps.event_states) == set(names) | {"_buffer"}
    for j, n in enumerate(names):  # initial timers inside the interval range (events.py get_initial_event_state)
        lo, hi = evs[n].interval_range
        assert ((ps.event_states[n] >= lo) & (ps.event_states[n] <= hi)).all()
    low = np.arange(N) % 3 == 0
    for p in (ps, ps0):
        p.data.qpos[torch.from_numpy(low).to(DEV), 2] = 0.87
    left0 = rng.uniform(0.0, 0.05, (len(names), N)).astype(np.float32)  # some timers run out within the 4 substeps
    ps.event_states["_buffer"].copy_(t32(left0))
    K = c.terms.obs_dim
    noise = dict(obs_normal=rng.normal(size=(N, K)), obs_uniform=rng.random((N, K)), action_normal=rng.normal(size=(N, m.nu)),
                 reset_uniform=rng.uniform(-1, 1, (N, m.nq + 1)), event_reset_uniform=rng.random((N, len(names))))
    ev_u = rng.random((4, N, len(names), 12)).astype(np.float32)
    noise_t = {k: t32(v) for k, v in noise.items()}
    env = EnvState(ps, rnd_, torch.zeros(N, 2, device=DEV), None, seed=1)
    env0 = EnvState(ps0, rnd0, torch.zeros(N, 2, device=DEV), None, seed=1)
    ro.step_engine(env, 0, 1.0, dict(noise_t, engine=dict(event_uniform=t32(ev_u))))
    ro0.step_engine(env0, 0, 1.0, {k: v for k, v in noise_t.items() if k != "event_reset_uniform"})
    done = ro.done[0].cpu().numpy().astype(bool)
    assert np.array_equal(done, low)
    kinds = {"push": ("linear", dict(linvel=0.5, vel_range=(0.0, 1.0), interval_range=(0.05, 0.3))),
             "spin": ("angular", dict(angvel=0.5, vel_range=(0.0, 1.0), interval_range=(0.1, 0.4))),
             "jump": ("jump", dict(jump_height_range=(0.01, 0.05), interval_range=(0.2, 0.6)))}
    want = left0.astype(np.float64).copy()
    fired = np.zeros(N, bool)
    for j, n in enumerate(names):
        for e in range(N):
            for s in range(4):
                imp, want[j, e] = ot.velocity_event(kinds[n][0], kinds[n][1], want[j, e], m.dt, ev_u[s, e, j], 1.0)
                want[j, e] = float(np.float32(want[j, e]))
                fired[e] |= bool(imp.any())
        lo, hi = evs[n].interval_range
        want[j, done] = lo + noise["event_reset_uniform"][done, j] * (hi - lo)
    np.testing.assert_allclose(ps.event_states["_buffer"].cpu().numpy(), want, rtol=0, atol=1e-6)
    assert torch.equal(ps.event_states["push"], ps.event_states["_buffer"][0])  # named views of the one buffer
    moved = (ro.qvel[0] - ro0.qvel[0]).abs().amax(dim=1).cpu().numpy() > 1e-4
    assert fired.any() and np.array_equal(moved, fired), "exactly the envs whose events fired differ from the run without events"


def test_gait_terms_in_the_rollout_and_under_graph_replay():
    """Contact flags, delayed and lagged observations and the stateful gait rewards inside the environment loop: the
    rewards recomputed by the oracle from the recorded rollout, carried over three rollouts, and the graph replay
    equal to the eager loop bit for bit."""
    N, T = 64, 8
    runs = []
    for use_graph in (False, True):
        m, c, rnd_, _, ro, EnvState = build(N, T, seed=7, min_height=0.8, gait=True)
        ps = c.engine.reset(c.physics_model, 1.0, 3, N, rnd_)
        env = EnvState(ps, rnd_, c.commands.initial(N, DEV), None, seed=9)
        sl = c.terms.obs_slices
        carries = [((np.zeros(2, int),) * 3, np.zeros(2)) for _ in range(N)]
        snaps = []
        for it in range(4):
            traj, rew = ro.unroll(env, graph=use_graph)
            torch.cuda.synchronize()
            snaps.append((traj.obs["obs"].clone(), rew.total.clone(), env.obs_carry.clone(), env.reward_carry.clone()))
            snaps[-1] += (traj.command["_buffer"].clone(), env.commands.clone())
            if use_graph:
                continue
            cm = traj.command["_buffer"].cpu().numpy()
            # recorded commands: step t+1 shows the update of step t; a finished env drew a fresh command instead
            lin, ang = cm[..., c.commands.slices["lin"]], cm[..., c.commands.slices["ang"]]
            np.testing.assert_allclose(lin[..., 2], lin[..., 0] * np.cos(lin[..., 1]), atol=1e-6)
            assert (np.abs(lin[..., 4]) <= 1.0).all() and (np.abs(ang[..., 1]) <= 0.5).all() and np.abs(lin[..., 4]).max() > 0.2
            obs, qvel, done = traj.obs["obs"].cpu().numpy(), traj.qvel.cpu().numpy(), traj.done.cpu().numpy().astype(bool)
            from ksim_amd.rewards import get_rewards
            full = get_rewards(traj, c.rewards, want_components=True, obs_slices=sl, command_slices=c.commands.slices) if it == 0 else None  # zero carry
            xpos = traj.xpos.cpu().numpy().reshape(T, N, m.nb, 3)
            feet = [b for b in range(m.nb) if any(int(sb) == b for sb in m.sph_body)]
            # the recorded observation is taken before the step, the recorded xpos after it: row t+1 of the former
            # shows the bodies of row t of the latter, unless the env was reset in between
            for t in range(T - 1):
                keep = ~done[t]
                np.testing.assert_allclose(obs[t + 1][keep][:, sl["feet_pos"]].reshape(-1, 2, 3), xpos[t][keep][:, feet], atol=1e-6)
            assert set(np.unique(obs[..., sl["contact"]])) <= {0.0, 1.0}
            touched = obs[..., sl["contact"]].mean() if it == 0 else max(touched, obs[..., sl["contact"]].mean())
            want = np.zeros((T, N))
            for e in range(N):
                a0, h0 = carries[e] if not done[-1, e] else ((np.zeros(2, int),) * 3, np.zeros(2))
                con = obs[:, e, sl["contact"]].reshape(T, -1, 2)
                a, a1 = ot.feet_air_time_reward(con, qvel[:, e], done[:, e], a0, air_steps=5.0, gnd_steps=5.0, linvel_threshold=0.05)
                h, h1 = ot.sparse_target_height_reward(con, obs[:, e, sl["feet_pos"]].reshape(T, 2, 3), qvel[:, e], done[:, e], h0,
                                                       height=0.1, linvel_threshold=0.02)
                carries[e] = (a1, h1)
                want[:, e] = a["air"] + a["gnd"] + a["stationary_gnd"] + 2.0 * h
            if full is not None:
                got = sum(v for k, v in full.components.items() if k.startswith(("air_time", "step_height"))).cpu().numpy()
                np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
            else:  # later rollouts: the carried counters enter; check through the carry buffer
                cr = env.reward_carry.cpu().numpy()
                np.testing.assert_allclose(cr[:, :6], [np.concatenate(cv[0]) for cv in carries])
                np.testing.assert_allclose(cr[:, 6:8], [cv[1] for cv in carries], rtol=1e-6, atol=1e-7)
        assert use_graph or 0.05 < touched < 1.0, "the feet never touched the floor: the contact terms were not exercised"
        runs.append(snaps)
    for it, (a, b) in enumerate(zip(*runs)):
        for x, y, name in zip(a, b, ("observations", "reward", "observation carry", "reward carry", "recorded commands", "commands")):
            assert torch.equal(x, y), f"replay {it}: {name} differs from the eager rollout"


def test_rollout_written_to_the_dataset_format_and_read_back(tmp_path):
    """collect_dataset's data path (ksim/task/rl.py:2315-2411): a device rollout goes to the float32 memory map one env per
    sample and comes back equal."""
    from ksim_amd.dataset import TrajectoryDataset

    N, T = 16, 8
    m, c, rnd_, _, ro, EnvState = build(N, T, seed=3)
    ps = c.engine.reset(c.physics_model, 1.0, 3, N, rnd_)
    env = EnvState(ps, rnd_, torch.zeros(N, 2, device=DEV), None, seed=4)
    traj, _ = ro.unroll(env)
    rew = ro._rewards(traj, env, 1.0, want_components=True)
    path = tmp_path / "rollouts.bin"
    with TrajectoryDataset.writer(path, num_samples=N) as w:
        assert w.write_batch(traj, rew) == N
    ds = TrajectoryDataset(path, device=DEV)
    for e in (0, 7, 15):
        t, r = ds.get(e)
        assert torch.equal(t.qpos, traj.qpos[:, e]) and torch.equal(t.obs["noisy_obs"], traj.obs["noisy_obs"][:, e])
        assert torch.equal(t.xquat, traj.xquat[:, e]) and torch.equal(t.done, traj.done[:, e].float())
        assert torch.equal(r.total, rew.total[:, e]) and torch.equal(r.components["height"], rew.components["height"][:, e])


@pytest.mark.parametrize("head", [None, "gaussian", "mixture", "gaussian-lowpass"])
def test_recurrent_actor_and_critic_in_the_rollout(head):
    """GRU actor and critic inside the environment loop: the carries replayed by the oracle from the recorded
    observations and done flags (a finished env continues from a zero carry), and the graph replay equal to eager.  With a
    head, the actor's output goes through the deviation head or the mixture head; their deviations are squeezed to 1e-6
    here, so the recorded action must be the (biased, clipped) mean, of one of the components for the mixture."""
    from oracle import recurrent as orec

    N, T = 24, 8
    runs = []
    for use_graph in (False, True):
        m, c, rnd_, _, ro, EnvState = build(N, T, seed=13, min_height=0.95, recurrent=True, head=head)
        ps = c.engine.reset(c.physics_model, 1.0, 3, N, rnd_)
        env = EnvState(ps, rnd_, torch.zeros(N, 2, device=DEV), None, seed=21)
        want = {"actor": np.zeros((2, N, 32)), "critic": np.zeros((2, N, 32)), "lpf": np.zeros((N, m.nu))}
        fresh = np.zeros(N, bool)
        snaps, finished = [], 0
        for it in range(5):
            traj, rew = ro.unroll(env, graph=use_graph)
            torch.cuda.synchronize()
            finished += int(traj.done.sum().item())
            snaps.append((traj.action.clone(), ro.values.clone(), env.actor_carry.clone(), env.critic_carry.clone()))
            if use_graph:
                continue
            obs, noisy, done = (x.cpu().numpy() for x in (traj.obs["obs"], traj.obs["noisy_obs"], traj.done))
            for t in range(T):
                proj, cells, ow, ob_ = c.critic.params
                v, want["critic"] = orec.recurrent_network(obs[t], want["critic"], fresh, proj, cells, ow, ob_, act=lambda x: np.where(x > 0, x, np.expm1(x)))
                proj, cells, ow, ob_ = c.actor.params
                y, want["actor"] = orec.recurrent_network(noisy[t], want["actor"], fresh, proj, cells, ow, ob_)
                np.testing.assert_allclose(ro.values[t].cpu().numpy(), v, rtol=2e-4, atol=2e-4)
                if head is not None:
                    act_t, nu = traj.action[t].cpu().numpy(), m.nu
                    bias = c.head.mean_bias.cpu().numpy()
                    if head == "gaussian":
                        np.testing.assert_allclose(act_t, y[:, :nu] + bias, rtol=2e-4, atol=2e-4)
                    elif head == "gaussian-lowpass":  # the filter state restarts with the episode, like the carries
                        x_in = y[:, :nu] + bias
                        x_in[:, nu - 2:] += noisy[t][:, 0:2]
                        want["lpf"] = ot.lowpass_one_pole(x_in, np.where(fresh[:, None], 0.0, want["lpf"]), 0.02, 4.0)
                        np.testing.assert_allclose(act_t, want["lpf"], rtol=2e-4, atol=2e-4)
                    else:
                        means = np.clip(y[:, :2 * nu].reshape(N, nu, 2) + bias[None, :, None], -0.3, 0.3)
                        assert np.abs(means - act_t[..., None]).min(-1).max() < 2e-4
                fresh = done[t].astype(bool)
            np.testing.assert_allclose(env.actor_carry.cpu().numpy(), want["actor"], rtol=2e-4, atol=2e-4)
            if head == "gaussian-lowpass":
                np.testing.assert_allclose(env.lpf_state.cpu().numpy(), want["lpf"], rtol=2e-4, atol=2e-4)
        runs.append(snaps)
        assert use_graph or finished > 0, "no env finished: the carry restart was not exercised"
    for it, (a, b) in enumerate(zip(*runs)):
        for x, y, name in zip(a, b, ("action", "values", "actor carry", "critic carry")):
            assert torch.equal(x, y), f"replay {it}: {name} differs from the eager rollout"


@pytest.mark.parametrize("head", ["gaussian-wide", "mixture-wide"])
def test_recurrent_policy_update_from_a_rollout(head):
    """A rollout with a GRU actor (deviation head) and a GRU critic, then the recurrent policy update on its buffers: the
    on-policy pass, replayed from the recorded first-step carries and episode starts, reproduces the values the rollout
    computed bit for bit; the minibatch steps run through time, move every parameter and keep everything finite."""
    from ksim_amd import ppo_update as pu

    N, T = 32, 8
    m, c, rnd_, _, ro, EnvState = build(N, T, seed=17, min_height=0.95, recurrent=True, head=head)
    ps = c.engine.reset(c.physics_model, 1.0, 3, N, rnd_)
    env = EnvState(ps, rnd_, torch.zeros(N, 2, device=DEV), None, seed=23)
    for _ in range(3):  # the third rollout starts from carries that are not zero
        traj, rew = ro.unroll(env)
    assert ro.fresh.sum().item() > 0 and ro.actor_carry0.abs().max().item() > 0
    assert torch.equal(ro.fresh[1:], traj.done[:-1])  # an env starts an episode at the step after it finished
    policy = pu.RecurrentHeadPolicy(c.actor, c.critic, c.head.min_std, c.head.max_std, c.head.var_scale, c.head.mean_bias)
    if head == "mixture-wide":
        policy.num_mixtures, policy.clip_lo, policy.clip_hi = c.head.num_mixtures, c.head.clip_lo, c.head.clip_hi
    policy.train_init()
    args = (traj.obs["noisy_obs"], traj.obs["obs"], traj.action, rew.total, traj.done, traj.success, ro.actor_carry0, ro.critic_carry0, ro.fresh)
    on_lp, on_v = pu.recurrent_on_policy(policy, args[0], args[1], args[2], *args[6:])
    assert torch.equal(on_v, ro.values[..., 0])
    assert torch.isfinite(on_lp).all()
    before = [p.clone() for cell in c.actor.cells for p in cell.parameters().values()]
    cfg = pu.PPOUpdateConfig(batch_size=16, num_passes=2, learning_rate=1e-3)
    out = pu.update_model_recurrent(policy, cfg, *args, seed=1)
    assert len(out) == 4 and all(torch.isfinite(o["grad_norm"]).all() and o["grad_norm"].item() > 0 for o in out)
    after = [p for cell in c.actor.cells for p in cell.parameters().values()]
    assert all(torch.isfinite(a).all() and not torch.equal(a, b) for a, b in zip(after, before))
    # the rollout goes on with the updated networks
    traj2, _ = ro.unroll(env)
    assert torch.isfinite(traj2.action).all() and torch.isfinite(ro.values).all()
    # adaptive KL (ppo.py:546-563): after every minibatch step the coefficient follows the host rule on that step's log-probabilities
    cfg = pu.PPOUpdateConfig(batch_size=N, num_passes=1, learning_rate=3e-3, adaptive_kl=True, desired_kl=1e-3)
    on_lp, _ = pu.recurrent_on_policy(policy, args[0], args[1], args[2], *args[6:])
    coef, moved = cfg.kl_coef, 0
    for _ in range(4):
        met = pu.update_model_recurrent(policy, cfg, *args, seed=2)[0]
        kl_mean = float((on_lp.reshape(-1, on_lp.shape[-1]).double() - met["log_probs"].double()).sum(-1).mean().item()) * coef
        new = coef * 1.5 if kl_mean > cfg.desired_kl * 1.5 else coef
        new = new / 1.5 if kl_mean < cfg.desired_kl / 1.5 else new
        moved += new != coef
        coef = min(max(new, 1e-8), 1e2)
        assert policy.kl_coef(cfg) == pytest.approx(coef, rel=1e-5)
        on_lp, _ = pu.recurrent_on_policy(policy, args[0], args[1], args[2], *args[6:])
    assert moved > 0


def test_kbot_policy_update_from_a_rollout_with_filter_and_mirror_losses():
    """The K-Bot task's update on a rollout's own buffers: the actor's means are filtered in the rollout, so the on-policy
    pass has to replay the filter from the recorded first-step state and episode starts to reproduce the rollout's
    log-probabilities; then minibatch steps with both mirror losses (the mirrored pass starts from zero carries, which is
    what the task's rollout leaves in `actor_mirror`, `critic_mirror` and `lpf_params_mirror`)."""
    from ksim_amd import ppo_update as pu
    from ksim_amd.env_terms import sample_action_head

    N, T = 32, 8
    m, c, rnd_, _, ro, EnvState = build(N, T, seed=19, min_height=0.95, recurrent=True, head="kbot")
    ps = c.engine.reset(c.physics_model, 1.0, 3, N, rnd_)
    env = EnvState(ps, rnd_, torch.zeros(N, 2, device=DEV), None, seed=29)
    for _ in range(3):
        traj, rew = ro.unroll(env)
    assert ro.fresh.sum().item() > 0 and ro.lpf_carry0.abs().max().item() > 0
    K = c.terms.obs_dim
    rng = np.random.default_rng(3)
    operm, osign = rng.permutation(K), rng.choice([-1.0, 1.0], K)
    aperm, asign = pu.kbot_mirror_joints()
    policy = pu.RecurrentHeadPolicy(c.actor, c.critic, c.head.min_std, c.head.max_std, c.head.var_scale, c.head.mean_bias,
                                    lowpass=c.head.lowpass, mirror=pu.MirrorSpec(list(operm), list(osign), list(operm), list(osign), aperm, asign))
    policy.train_init()
    args = (traj.obs["noisy_obs"], traj.obs["obs"], traj.action, rew.total, traj.done, traj.success, ro.actor_carry0, ro.critic_carry0, ro.fresh)
    on_lp, on_v, loc = pu.recurrent_on_policy(policy, args[0], args[1], args[2], *args[6:], lpf0=ro.lpf_carry0, return_raw=True)
    assert torch.equal(on_v, ro.values[..., 0])
    # the replay (networks from the recorded carries, filter from the recorded state, both restarted at the recorded
    # episode starts) arrives at the last step with the very rows the rollout sampled its last action from
    assert torch.equal(loc[T - 1], ro.mean) and torch.isfinite(on_lp).all()
    without = pu.recurrent_on_policy(policy, args[0], args[1], args[2], *args[6:], lpf0=None)[0]
    assert not torch.equal(without, on_lp)  # the recorded filter state matters
    before = [p.clone() for cell in c.actor.cells for p in cell.parameters().values()]
    cfg = pu.PPOUpdateConfig(batch_size=16, num_passes=2, learning_rate=1e-3, actor_mirror_loss_scale=1.0, critic_mirror_loss_scale=0.5)
    out = pu.update_model_recurrent(policy, cfg, *args, seed=1, lpf0=ro.lpf_carry0)
    assert len(out) == 4 and all(torch.isfinite(o["grad_norm"]).all() and o["grad_norm"].item() > 0 for o in out)
    assert all(o["action_mirror_loss"].shape == (T, 16) and o["action_mirror_loss"].mean().item() > 0 for o in out)
    assert all(torch.isfinite(o["value_mirror_loss"]).all() for o in out)
    after = [p for cell in c.actor.cells for p in cell.parameters().values()]
    assert all(torch.isfinite(a).all() and not torch.equal(a, b) for a, b in zip(after, before))
    traj2, _ = ro.unroll(env)
    assert torch.isfinite(traj2.action).all() and torch.isfinite(env.lpf_state).all()


def test_split_rollout_equals_single_stream_rollout():
    """Two groups of envs on two streams give every env, bit for bit, the trajectory the single-stream rollout gives it
    for the same draws (resets and per-episode re-draws included); advantage normalisation spans both groups."""
    from ksim_amd.rollout import SplitRollout

    N, T, G = 64, 6, 2
    m, c, rnd_, _, ro, EnvState = build(N, T, seed=5, min_height=0.9, sim2real=True)
    rng = np.random.default_rng(17)
    K, nu, ned, n = c.terms.obs_dim, m.nu, 3 * m.nu + 4, N // G
    u0 = t32(rng.uniform(-1, 1, (N, m.nq + 1)))
    eu, ez = t32(rng.uniform(-1, 1, (N, ned))), t32(rng.normal(size=(N, ned)))
    cmd = t32(rng.normal(size=(N, 2)))
    sl = [slice(g * n, (g + 1) * n) for g in range(G)]
    cut = lambda x, g: x[sl[g]].contiguous()  # noqa: E731

    def start(rows, rnd_rows):
        ps = c.engine.reset(c.physics_model, 1.0, 0, rows.stop - rows.start, rnd_rows, reset_uniform=u0[rows].contiguous(),
                            episode_draws=dict(uniform=eu[rows].contiguous(), normal=ez[rows].contiguous()))
        low = (torch.arange(rows.start, rows.stop, device=DEV) % 3) == 0  # these start below the termination height
        ps.data.qpos[low, 2] = 0.87
        return EnvState(ps, rnd_rows, cmd[rows].contiguous(), None, seed=1)

    env = start(slice(0, N), rnd_)
    envs = [start(sl[g], {k: cut(v, g) for k, v in rnd_.items()}) for g in range(G)]
    sro = SplitRollout(c, N, T, splits=G)
    sro.fork()
    for t in range(T):
        noise = dict(obs_normal=t32(rng.normal(size=(N, K))), obs_uniform=t32(rng.random((N, K))),
                     action_normal=t32(rng.normal(size=(N, nu))), reset_uniform=t32(rng.uniform(-1, 1, (N, m.nq + 1))),
                     obs_bias_redraw=t32(np.stack([rng.normal(size=(N, K)), rng.uniform(-1, 1, (N, K))], -1)),
                     episode=dict(uniform=t32(rng.uniform(-1, 1, (N, ned))), normal=t32(rng.normal(size=(N, ned)))))
        ro.step_engine(env, t, 1.0, noise)
        parts = [{k: ({kk: cut(vv, g) for kk, vv in v.items()} if isinstance(v, dict) else cut(v, g)) for k, v in noise.items()}
                 for g in range(G)]
        torch.cuda.synchronize()  # the per-group copies above were made on the current stream
        sro.step_engine(envs, t, 1.0, parts)
    sro.join()
    torch.cuda.synchronize()
    assert int(ro.done.sum().item()) > 0, "no env was reset: the reset path was not compared"
    for name in ("qpos", "qvel", "xpos", "xquat", "ctrl", "action", "obs", "noisy_obs", "done", "success", "timestep", "values"):
        whole = getattr(ro, name)
        joined = torch.cat([getattr(p, name) for p in sro.parts], dim=1)
        assert torch.equal(whole, joined), name
    for name in ("action_latency", "zero_offset"):
        assert torch.equal(getattr(env.physics_state, name), torch.cat([getattr(e.physics_state, name) for e in envs])), name
    assert torch.equal(env.physics_state.data.qpos, torch.cat([e.physics_state.data.qpos for e in envs]))
    assert torch.equal(env.obs_bias, torch.cat([e.obs_bias for e in envs]))
    # rewards and GAE per group; normalised advantages over the union of the groups
    from ksim_amd.rewards import get_rewards
    rew = get_rewards(ro.trajectory(), c.rewards)
    rews = [get_rewards(p.trajectory(), c.rewards) for p in sro.parts]
    assert torch.equal(rew.total, torch.cat([r.total for r in rews], dim=1))
    whole = ro.ppo_inputs(rew, 0.99, 0.95, normalize_advantages=True)
    split = sro.ppo_inputs(rews, 0.99, 0.95, normalize_advantages=True)
    torch.cuda.synchronize()
    assert torch.equal(whole.gae_bt, torch.cat([s.gae_bt for s in split], dim=1))
    assert torch.equal(whole.value_targets_bt, torch.cat([s.value_targets_bt for s in split], dim=1))
    np.testing.assert_allclose(torch.cat([s.advantages_bt for s in split], dim=1).cpu().numpy(), whole.advantages_bt.cpu().numpy(),
                               rtol=2e-6, atol=2e-6)
    with pytest.raises(Exception, match="multiple"):
        SplitRollout(c, 63, T, splits=2)


def test_split_rollout_replayed_from_per_group_graphs_equals_its_eager_run():
    """`SplitRollout.unroll(graph=True)`: one HIP graph per group, replayed side by side on the groups' streams, gives the eager
    split rollout's bits on every replay (Philox draws, resets on the way)."""
    from ksim_amd.rollout import SplitRollout

    N, T, G = 64, 5, 2
    outs = []
    for graph in (False, True):
        m, c, rnd_, _, _, EnvState = build(N, T, seed=6, min_height=0.9, sim2real=True)
        n = N // G
        envs = []
        for g in range(G):
            rows = {k: v[g * n:(g + 1) * n].contiguous() for k, v in rnd_.items()}
            ps = c.engine.reset(c.physics_model, 1.0, 3 + g, n, rows)
            ps.data.qpos[::3, 2] = 0.87
            envs.append(EnvState(ps, rows, torch.zeros(n, 2, device=DEV), None, seed=11 + g))
        sro = SplitRollout(c, N, T, splits=G)
        run = []
        for k in range(4):
            res = sro.unroll(envs, graph=graph)
            torch.cuda.synchronize()
            run.append([x.clone() for traj, rew in res for x in (traj.qpos, traj.action, traj.done, rew.total)])
        assert sum(int(r[2].sum()) + int(r[6].sum()) for r in run) > 0, "no env was reset"
        outs.append(run)
    for a, b in zip(*outs):
        for x, y in zip(a, b):
            assert torch.equal(x, y)


def test_motion_resets_symmetry_rewards_and_imu_misalignment_in_the_rollout():
    """The pieces an AMP / sim-to-real task adds, together in one rollout on a model read from MJCF: episodes that start from
    a frame of a reference motion with a random pitch / roll and heading, a misaligned IMU site per env read by the gyro,
    the accelerometer and the site-orientation observation, contact flags over a geom list, symmetry rewards with their
    rollout-mean carry.  Checked: reset envs restart on a motion frame at time frame * dt, and the HIP-graph replay gives the eager
    rollout's bits."""
    from ksim_amd import actuators, engine, observation as ob, physics, randomization as rnd, resets as rs
    from ksim_amd import rewards as rw, terminations as tm
    from ksim_amd.env_terms import EnvTerms
    from ksim_amd.mjcf import load_mjcf
    from ksim_amd.mlp import MLP
    from ksim_amd.priors import MotionReferenceData
    from ksim_amd.rollout import Rollout, RolloutConstants, RolloutEnvState

    m = load_mjcf(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mini_biped.mjcf"), integrator="implicitfast")
    N, T, F = 64, 10, 9
    rng = np.random.default_rng(41)
    mq = np.tile(m.qpos0, (F, 1))
    mq[:, 7:] += rng.uniform(-0.2, 0.2, (F, m.nq - 7))
    motion = MotionReferenceData(qpos=mq, qvel=np.zeros((F, m.nv)), cartesian_poses={}, ctrl_dt=0.02)
    resets = [rs.InitialMotionStateReset(reference_motion=motion), rs.RandomPitchRollReset(pitch_range=(-0.2, 0.2), roll_range=(-0.1, 0.1)),
              rs.RandomHeadingReset()]
    act = actuators.PositionActuators(kps=(40.0,) * m.nu, kds=(1.0,) * m.nu, ctrl_clip=(30.0,) * m.nu)
    eng = engine.get_physics_engine("hip", resets, {}, act, engine.EngineConfig(dt=m.dt, ctrl_dt=0.02))
    observations = {"jp": ob.JointPositionObservation(noise=0.01), "jv": ob.JointVelocityObservation(),
                    "gyro": ob.SensorObservation(sensor_name="imu_gyro", site_pose_per_env=True, noise=0.01),
                    "acc": ob.SensorObservation(sensor_name="imu_acc", site_pose_per_env=True),
                    "imu_rot": ob.SiteOrientationObservation(site_names=("imu_site",), site_pose_per_env=True),
                    "contact": ob.ContactObservation(geom_idxs=tuple(range(m.ns)) + (ob.FLOOR_GEOM,)),
                    "a": ob.LastActionObservation()}
    z0 = float(m.qpos0[2])
    terms = EnvTerms(m, observations, {"h": tm.MinimumHeightTermination(z0 - 0.008)}, resets)
    nj = m.nq - 7
    rewards = {"alive": rw.StayAliveReward(scale=1.0),
               "sym": rw.SymmetryReward(scale=0.5, joint_indices=tuple(range(nj)), joint_targets=(0.0,) * nj, alpha=0.3),
               "pair": rw.PairwiseSymmetryReward(scale=0.2, left_joint_index=0, right_joint_index=nj // 2, flipped=True)}
    dims = (terms.obs_dim, 32, m.nu)
    ws = [rng.normal(scale=0.3 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])]
    cws = [rng.normal(scale=1 / np.sqrt(terms.obs_dim), size=(1, terms.obs_dim)).astype(np.float32)]
    consts = RolloutConstants(physics_model=physics.DeviceModel(m), engine=eng, terms=terms, rewards=rewards,
                              actor=MLP(ws, [np.zeros(o, np.float32) for o in dims[1:]], dtype="f32"),
                              critic=MLP(cws, [np.zeros(1, np.float32)], dtype="f32"), log_std=t32(np.full(m.nu, -1.0)))

    # eager, then the graph replay from an identical start
    runs = []
    for graph in (False, True):
        gen = torch.Generator(device=DEV); gen.manual_seed(100)
        rnd_ = rnd.get_physics_randomizers(m, {"imu": rnd.IMUAlignmentRandomizer(site_name="imu_site", tilt_std_rad=0.05, yaw_std_rad=0.05,
                                                                                   translate_std_m=0.01),
                                               "f": rnd.FloorFrictionRandomizer(0.5, 1.0)}, N, gen)
        ps = eng.reset(consts.physics_model, 1.0, 7, N, rnd_)
        env = RolloutEnvState(ps, rnd_, torch.zeros(N, 0, device=DEV), None, seed=5)
        ro = Rollout(consts, N, T)
        outs = []
        for k in range(3):
            traj, rew = ro.unroll(env, graph=graph)
            outs.append((traj.qpos.clone(), traj.obs["obs"].clone() if isinstance(traj.obs, dict) and "obs" in traj.obs else ro.obs.clone(),
                         traj.done.clone(), rew.total.clone(), env.reward_carry.clone(), traj.timestep.clone()))
        runs.append(outs)
    for a, b in zip(runs[0], runs[1]):
        for x, y in zip(a, b):
            assert torch.equal(x, y)
    qpos, obs, done, total, carry, tstep = runs[0][-1]
    assert torch.isfinite(total).all() and torch.isfinite(obs).all()
    alld = torch.cat([r[2] for r in runs[0]])
    assert int(alld.sum()) > 10, "no episode ended: the motion reset was not exercised"
    # an env that is reset at step t shows, at step t + 1, a state that started one control step earlier on a motion frame:
    # its recorded time is frame * dt + 0.02 for some frame, and the carry of the symmetry reward is not stuck at its start
    tt = torch.cat([r[5] for r in runs[0]]).cpu().numpy()
    dd = alld.cpu().numpy().astype(bool)
    after = tt[1:][dd[:-1]]
    frames = (after - 0.02) / 0.02
    assert np.abs(frames - np.round(frames)).max() < 1e-4 and frames.min() > -1e-4 and frames.max() < F - 1 + 1e-4
    assert float(carry.abs().max()) > 1e-3


def test_site_frame_sensors_follow_the_live_state_in_a_rollout():
    """A task whose only observations of derived fields are site frame sensors (`framepos` reads xpos and, to turn the
    site offset, xquat; `framequat` and `magnetometer` read xquat): the rollout must keep both fields of the live state
    up to date, so the observation of step t + 1 equals the sensor formula on what step t recorded.  With a stale
    quaternion the foot position would stay that of the reset pose's orientation."""
    from ksim_amd import _lib_terms as T, actuators, engine, observation as ob, physics, resets as rs, rewards as rw
    from ksim_amd import terminations as tm
    from ksim_amd.env_terms import EnvTerms
    from ksim_amd.mjcf import load_mjcf
    from ksim_amd.mlp import MLP
    from ksim_amd.rollout import Rollout, RolloutConstants, RolloutEnvState

    m = load_mjcf(os.path.join(os.path.dirname(__file__), "golden", "mini_biped.mjcf"))
    N, Tn = 16, 6
    rng = np.random.default_rng(41)
    act = actuators.PositionActuators(kps=(30.0,) * m.nu, kds=(1.0,) * m.nu, ctrl_clip=(20.0,) * m.nu)
    resets = [rs.RandomJointPositionReset(scale=0.2, scale_by_curriculum=False)]
    eng = engine.get_physics_engine("hip", resets, {}, act, engine.EngineConfig(dt=m.dt, ctrl_dt=4 * m.dt))
    observations = {"jp": ob.JointPositionObservation(),
                    "foot": ob.SensorObservation.create(physics_model=m, sensor_name="left_foot_pos"),
                    "quat": ob.SensorObservation.create(physics_model=m, sensor_name="imu_quat")}
    terms = EnvTerms(m, observations, {"h": tm.MinimumHeightTermination(0.05)}, resets)
    assert T.SRC_XQUAT in terms.sources_used and T.SRC_XPOS in terms.sources_used
    dims = (terms.obs_dim, 32, m.nu)
    ws = [rng.normal(scale=1 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])]
    bs = [np.zeros(o, np.float32) for o in dims[1:]]
    consts = RolloutConstants(physics_model=physics.DeviceModel(m), engine=eng, terms=terms,
                              rewards={"alive": rw.StayAliveReward(scale=1.0)}, actor=MLP(ws, bs, dtype="f32"), critic=None,
                              log_std=t32(np.full(m.nu, -1.0)))
    ro = Rollout(consts, N, Tn)
    assert {"xpos", "xquat"} <= ro._live
    ps = eng.reset(consts.physics_model, 1.0, 0, N, {})
    env = RolloutEnvState(ps, {}, None, None, seed=3)
    for t in range(Tn):
        ro.step_engine(env, t, 1.0)
    sl = terms.obs_slices
    obs = ro.obs.cpu().numpy().astype(np.float64)
    xp = ro.xpos.cpu().numpy().reshape(Tn, N, m.nb, 3).astype(np.float64)
    xq = ro.xquat.cpu().numpy().reshape(Tn, N, m.nb, 4).astype(np.float64)
    done = ro.done.cpu().numpy().astype(bool)
    fb, fpos, _ = m.sites["left_foot"]
    ib, _, iquat = m.sites["imu_site"]
    checked = 0
    for t in range(Tn - 1):
        keep = ~done[t]  # an env that was reset observes its new pose, which the slot of step t does not hold
        np.testing.assert_allclose(obs[t + 1][keep][:, sl["foot"]], ot.site_frame_position(xp[t][keep][:, fb], xq[t][keep][:, fb], fpos),
                                   rtol=1e-5, atol=2e-6)
        np.testing.assert_allclose(obs[t + 1][keep][:, sl["quat"]], ot.site_frame_quaternion(xq[t][keep][:, ib], iquat), rtol=1e-5, atol=2e-6)
        checked += int(keep.sum())
    assert checked > N
    # the poses do change over the rollout, so a stale field could not have passed
    assert np.abs(xq[Tn - 1][:, fb] - xq[0][:, fb]).max() > 1e-3


def test_reset_forward_inside_the_next_step_gives_the_same_trajectories():
    """The forward pass a reset owes (engine.py:213), run inside the next control step's physics launch for the envs still
    flagged in the reset mask (`RolloutConstants.defer_reset_forward`), against the masked forward launch right after the
    termination pass: every recorded array of a rollout with many resets bit for bit, and the states the rollouts end in
    once the pending forward pass has been run."""
    import dataclasses

    N, T = 64, 12
    runs = []
    for defer, fuse in ((False, False), (True, False), (True, True)):
        m, c, rnd_, _, _, EnvState = build(N, T, seed=9, min_height=0.86)
        # `fuse`: the next step's observation also rides in the launch that ends a step (ks_terminate_reset_observe)
        c = dataclasses.replace(c, defer_reset_forward=defer, fuse_next_observation=fuse)
        from ksim_amd.rollout import Rollout
        ro = Rollout(c, N, T)
        assert ro._defer == defer and ro._fuse_obs == fuse
        ps = c.engine.reset(c.physics_model, 1.0, 5, N, rnd_)
        env = EnvState(ps, rnd_, torch.zeros(N, 2, device=DEV), None, seed=31)
        snaps = []
        for _ in range(3):
            traj, rew = ro.unroll(env)
            snaps.append([x.clone() for x in (traj.qpos, traj.qvel, traj.action, traj.done, traj.obs["obs"], traj.obs["noisy_obs"],
                                              traj.xpos, traj.ctrl, ro.values, rew.total)])
        if defer:  # what the last step's resets still owe
            c.engine.forward(c.physics_model, ps, ro.reset_mask, rnd_, live=ro._live)
        snaps.append([ps.data.qpos.clone(), ps.data.qvel.clone(), ps.data.qacc_warmstart.clone()])
        runs.append(snaps)
        assert sum(int(s[3].sum().item()) for s in snaps[:3]) > N // 4, "too few resets to tell the modes apart"
    for other in runs[1:]:
        for a, b in zip(runs[0], other):
            for x, y in zip(a, b):
                assert torch.equal(x, y)
