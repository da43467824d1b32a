"""Parity of the fused per-env term kernels (observations, terminations/resets, actions, rewards)."""
import json
import os

import numpy as np
import pytest
import torch

from ksim_amd import model as km
from oracle import terms as ot

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def t32(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32, device=DEV).contiguous()


def _state(m, N, seed):
    rng = np.random.default_rng(seed)
    qpos = rng.normal(size=(N, m.nq))
    qpos[:, 3:7] /= np.linalg.norm(qpos[:, 3:7], axis=1, keepdims=True)
    return dict(qpos=qpos, qvel=rng.normal(size=(N, m.nv)), qacc=rng.normal(size=(N, m.nv)),
                ctrl=rng.normal(size=(N, m.nu)), last=rng.normal(size=(N, m.nu)), cmd=rng.normal(size=(N, 2)),
                time=rng.random(N) * 3, zero=rng.normal(size=(N, m.nu)) * 0.01, rng=rng)


def test_observation_assembly_and_noise():
    from ksim_amd import _lib_terms as T, model as km, noise, observation as ob
    from ksim_amd.env_terms import EnvTerms

    m = km.humanoid_model()
    N = 37
    s = _state(m, N, 0)
    observations = {
        "joint_position": ob.JointPositionObservation(noise=0.01),
        "joint_velocity": ob.JointVelocityObservation(noise=noise.MultiplicativeUniformNoise(mag=0.1)),
        "projected_gravity": ob.ProjectedGravityObservation(),
        "base_angular_velocity": ob.BaseAngularVelocityObservation(in_robot_frame=True, noise=noise.AdditiveUniformNoise(mag=0.2, mean=0.1)),
        "last_action": ob.LastActionObservation(),
        "command": ob.CommandObservation(),
        "base_linear_velocity": ob.BaseLinearVelocityObservation(noise=noise.MultiplicativeGaussianNoise(std=0.05),
                                                                 bias=noise.MultiplicativeUniformBias(mag=0.1)),
        "timestep": ob.TimestepObservation(),
        "actuator_force": ob.ActuatorForceObservation(
            noise=noise.ChainedNoise([noise.AdditiveGaussianNoise(std=0.3), noise.MultiplicativeUniformNoise(mag=0.2),
                                      noise.AdditiveUniformGaussianNoise(std=0.05, mag=0.1)]), bias=0.02),
    }
    terms = EnvTerms(m, observations, {}, [], command_dim=2)
    assert terms.obs_dim == 21 + 21 + 3 + 3 + 21 + 2 + 3 + 1 + 21
    assert terms.obs_dim - 25 == 71  # the first six are the 71-wide actor input of benchmark config 3
    K = terms.obs_dim
    nn, uu = s["rng"].normal(size=(N, K)), s["rng"].random((N, K))
    bias0 = np.stack([s["rng"].normal(size=(N, K)), s["rng"].uniform(-1, 1, size=(N, K))], axis=-1)  # an older episode's draws
    bias1 = np.stack([s["rng"].normal(size=(N, K)), s["rng"].uniform(-1, 1, size=(N, K))], axis=-1)  # what fresh envs take
    fresh = np.arange(N) % 4 == 1
    bias_draw = t32(bias0)
    level = 0.7
    src = {T.SRC_QPOS: t32(s["qpos"]), T.SRC_QVEL: t32(s["qvel"]), T.SRC_QACC: t32(s["qacc"]), T.SRC_CTRL: t32(s["ctrl"]),
           T.SRC_LAST_ACTION: t32(s["last"]), T.SRC_COMMAND: t32(s["cmd"]), T.SRC_TIME: t32(s["time"])}
    obs = torch.empty(N, K, device=DEV); noisy = torch.empty(N, K, device=DEV)
    terms.observe(src, N, level=level, zero_offset=t32(s["zero"]), bias_draw=bias_draw, bias_redraw=t32(bias1),
                  fresh=torch.from_numpy(fresh.astype(np.uint8)).to(DEV), noise_normal=t32(nn), noise_uniform=t32(uu), obs=obs,
                  noisy_obs=noisy)
    # envs that start an episode took new bias draws, the others kept theirs, bit for bit
    bias = np.where(fresh[:, None, None], bias1, bias0)
    got_draw = bias_draw.cpu().numpy()
    for name in ("base_linear_velocity", "actuator_force"):
        a = terms.obs_slices[name]
        np.testing.assert_array_equal(got_draw[:, a], bias[:, a].astype(np.float32))
    a = terms.obs_slices["joint_position"]
    np.testing.assert_array_equal(got_draw[:, a], bias0[:, a].astype(np.float32))  # no bias there: never touched
    q, v = s["qpos"], s["qvel"]
    g = ot.rotate_vector_by_quat(np.broadcast_to([0, 0, -9.81], (N, 3)), q[:, 3:7], inverse=True)
    w = ot.rotate_vector_by_quat(v[:, 3:6], q[:, 3:7], inverse=True)
    want = np.concatenate([q[:, 7:] - s["zero"], v[:, 6:], g, w, s["last"], s["cmd"], v[:, 0:3], s["time"][:, None],
                           s["ctrl"]], axis=1)
    np.testing.assert_allclose(obs.cpu().numpy(), want, rtol=2e-6, atol=2e-6)
    sl = terms.obs_slices
    wn = want.copy()
    a = sl["joint_position"]; wn[:, a] = want[:, a] + nn[:, a] * 0.01 * level            # noise.py:102
    a = sl["joint_velocity"]; wn[:, a] = want[:, a] * ((1.0 - 0.1 * level) + 2 * 0.1 * level * uu[:, a])  # noise.py:86
    a = sl["base_angular_velocity"]; wn[:, a] = want[:, a] + (0.1 - 0.2 * level) + 2 * 0.2 * level * uu[:, a]
    ww = 2 * uu - 1
    a = sl["base_linear_velocity"]
    wn[:, a] = ot.add_noise(want[:, a], [("mul_gaussian", 1.0, 0.05)], ("mul_uniform", 1.0, 0.1), nn[:, a], ww[:, a],
                            bias[:, a, 0], bias[:, a, 1], level)
    a = sl["actuator_force"]
    wn[:, a] = ot.add_noise(want[:, a], [("add_gaussian", 0.0, 0.3), ("mul_uniform", 1.0, 0.2), ("add_uniform_gaussian", 0.0, 0.05, 0.1)],
                            ("add_gaussian", 0.0, 0.02), nn[:, a], ww[:, a], bias[:, a, 0], bias[:, a, 1], level)
    np.testing.assert_allclose(noisy.cpu().numpy(), wn, rtol=3e-6, atol=3e-6)
    # in-kernel Philox: deterministic for a (seed, step), different across steps, unit-variance normals
    a1 = torch.empty(N, K, device=DEV); a2 = torch.empty(N, K, device=DEV); a3 = torch.empty(N, K, device=DEV)
    all_fresh = torch.ones(N, dtype=torch.uint8, device=DEV)
    d1, d2 = torch.zeros(N, K, 2, device=DEV), torch.zeros(N, K, 2, device=DEV)
    terms.observe(src, N, seed=5, step=1, zero_offset=t32(s["zero"]), noisy_obs=a1, bias_draw=d1, fresh=all_fresh)
    terms.observe(src, N, seed=5, step=1, zero_offset=t32(s["zero"]), noisy_obs=a2, bias_draw=d2, fresh=all_fresh)
    terms.observe(src, N, seed=5, step=2, zero_offset=t32(s["zero"]), noisy_obs=a3, bias_draw=d2)
    assert torch.equal(a1, a2) and not torch.equal(a1, a3) and torch.equal(d1, d2)  # step 2 had no fresh env: draws kept
    # the Philox bias draws: a standard normal and the uniform the same bits give
    zb, wb = d1[:, sl["actuator_force"], 0].flatten().cpu().numpy(), d1[:, sl["actuator_force"], 1].flatten().cpu().numpy()
    assert abs(zb.mean()) < 0.15 and abs(zb.std() - 1.0) < 0.15
    np.testing.assert_allclose(wb, ot.same_key_uniform(zb), atol=2e-6)
    with pytest.raises(Exception, match="bias_draw"):
        terms.observe(src, N, zero_offset=t32(s["zero"]), noisy_obs=a1)
    # a fresh mask alone makes the kernel re-draw the biases into bias_draw: refused on the host before any launch
    with pytest.raises(Exception, match="bias_draw"):
        terms.observe(src, N, zero_offset=t32(s["zero"]), obs=a1, fresh=torch.ones(N, dtype=torch.uint8, device=DEV))
    z = ((a1 - obs)[:, sl["joint_position"]] / 0.01).flatten()
    assert abs(z.mean().item()) < 0.15 and abs(z.std().item() - 1.0) < 0.15


def test_termination_kats_and_masks_bit_exact():
    from ksim_amd import model as km, terminations as tm
    from ksim_amd.env_terms import EnvTerms

    m = km.kbot_scale_model()
    # the reference's known answers (tests/test_terminations.py:66-99) on its dummy qpos
    for kat in json.load(open(os.path.join(GOLD, "termination_kats.json"))):
        if kat["fn"] == "illegal_contact":
            # contact k of the known answer becomes sphere k of the model: its distance, and illegal when either of its
            # two geoms is in the illegal set
            dist = np.full((1, m.ns), 1.0); dist[0, :kat["ncon"]] = kat["dist"][:kat["ncon"]]
            bad = tuple(k for k in range(kat["ncon"]) if kat["geom1"][k] in kat["illegal"] or kat["geom2"][k] in kat["illegal"])
            terms = EnvTerms(m, {}, {"t": tm.IllegalContactTermination(illegal_sphere_idxs=bad)}, [])
            comps = torch.zeros(1, 1, dtype=torch.int8, device=DEV)
            done = torch.zeros(1, dtype=torch.uint8, device=DEV); succ = torch.ones(1, dtype=torch.uint8, device=DEV)
            qpos = np.zeros((1, m.nq)); qpos[0, 3] = 1.0
            terms.terminate_reset(dict(qpos=t32(qpos), qvel=torch.zeros(1, m.nv, device=DEV)), components=comps, done=done, success=succ,
                                  contact_dist=t32(dist), apply_reset=False)
            assert comps.item() == kat["expected"] and done.item() == (kat["expected"] != 0) and succ.item() == 0
            continue
        term = tm.NotUprightTermination(kat["max_radians"]) if kat["fn"] == "not_upright" else tm.MinimumHeightTermination(kat["min_height"])
        terms = EnvTerms(m, {}, {"t": term}, [])
        qpos = np.zeros((1, m.nq)); qpos[0, :9] = kat["qpos"]
        comps = torch.zeros(1, 1, dtype=torch.int8, device=DEV)
        done = torch.zeros(1, dtype=torch.uint8, device=DEV); succ = torch.zeros(1, dtype=torch.uint8, device=DEV)
        terms.terminate_reset(dict(qpos=t32(qpos), qvel=torch.zeros(1, m.nv, device=DEV)), components=comps, done=done,
                              success=succ, apply_reset=False)
        assert comps.item() == kat["expected"] and done.item() == (kat["expected"] != 0) and succ.item() == 0
    # all term kinds on random states, against the oracle, bit-exact
    N = 500
    s = _state(m, N, 3)
    s["qpos"][:, :3] *= 2.0
    term_objs = {
        "min_height": tm.MinimumHeightTermination(0.5), "bad_z": tm.BadZTermination(-1.0, 2.0, -0.5, 1.5),
        "not_upright": tm.NotUprightTermination(1.2), "bad_vel": tm.BadVelocityTermination(2.5),
        "far": tm.FarFromOriginTermination(3.0), "length": tm.EpisodeLengthTermination(1.5),
        # the curriculum switch of the length term (terminations.py:188-190) on both sides of the level, and the
        # negative variants of the two terms that default to a positive termination
        "length_off": tm.EpisodeLengthTermination(1.5, disable_at_curriculum_level=1),
        "length_on": tm.EpisodeLengthTermination(1.5, disable_at_curriculum_level=0.25, pos_termination=False),
        "length_at": tm.EpisodeLengthTermination(1.5, disable_at_curriculum_level=0.4),
        "far_neg": tm.FarFromOriginTermination(6.0, pos_termination=False),
    }
    terms = EnvTerms(m, {}, term_objs, [])
    level = 0.4
    comps = torch.zeros(len(term_objs), N, dtype=torch.int8, device=DEV)
    done = torch.zeros(N, dtype=torch.uint8, device=DEV); succ = torch.zeros(N, dtype=torch.uint8, device=DEV)
    q32, v32, t32_ = s["qpos"].astype(np.float32), s["qvel"].astype(np.float32), s["time"].astype(np.float32)
    terms.terminate_reset(dict(qpos=t32(q32), qvel=t32(v32), time=t32(t32_)), level=level, components=comps, done=done,
                          success=succ, apply_reset=False)
    want = [ot.minimum_height_termination(q32, np.float32(0.5)), ot.bad_z_termination(q32, -1.0, 2.0, np.float32(level), -0.5, 1.5),
            ot.not_upright_termination(q32, 1.2), ot.bad_velocity_termination(v32, 2.5),
            ot.far_from_origin_termination(q32, 3.0), ot.episode_length_termination(t32_, 1.5),
            ot.episode_length_termination(t32_, 1.5, True, np.float32(level), 1),
            ot.episode_length_termination(t32_, 1.5, False, np.float32(level), 0.25),
            ot.episode_length_termination(t32_, 1.5, True, np.float32(level), np.float32(0.4)),
            ot.far_from_origin_termination(q32, 6.0, pos_termination=False)]
    assert not want[6].any() and (want[7] == -1).sum() > 20 and np.array_equal(want[8], want[5])
    got = comps.cpu().numpy()
    # exclude the measure-zero band where fp32 and float64 evaluation of a norm/acos straddle the threshold
    near = np.zeros(N, bool)
    near |= np.abs(np.linalg.norm(v32[:, :3], axis=1) - 2.5) < 1e-5
    near |= np.abs(np.linalg.norm(q32[:, :3], axis=1) - 3.0) < 1e-5
    near |= np.abs(np.linalg.norm(q32[:, :3], axis=1) - 6.0) < 1e-5
    for j, w in enumerate(want):
        assert np.array_equal(got[j][~near], w[~near]), list(term_objs)[j]
    wd, ws = ot.combine_terminations([g for g in got])
    assert np.array_equal(done.cpu().numpy().astype(bool), wd) and np.array_equal(succ.cpu().numpy().astype(bool), ws)
    assert wd.sum() > 20 and ws.sum() > 5


def test_reset_predication():
    from ksim_amd import model as km, resets as rs, terminations as tm
    from ksim_amd.env_terms import EnvTerms

    m = km.kbot_scale_model()
    N = 64
    nj = m.nq - 7
    zeros = tuple(np.linspace(-0.2, 0.2, nj))
    resets = [rs.RandomJointPositionReset(scale=0.1, scale_by_curriculum=False, zeros=zeros, mins=(-0.25,) * nj, maxs=(0.25,) * nj),
              rs.RandomJointVelocityReset(scale=0.5), rs.RandomHeightReset(range=(0.0, 0.2)), rs.RandomHeadingReset()]
    terms = EnvTerms(m, {}, {"h": tm.MinimumHeightTermination(0.5)}, resets)
    s = _state(m, N, 4)
    s["qpos"][:, 2] = np.where(np.arange(N) % 3 == 0, 0.2, 0.9)
    u = s["rng"].uniform(-1, 1, size=(N, m.nq + 1))
    st = dict(qpos=t32(s["qpos"]), qvel=t32(s["qvel"]), qacc_warmstart=t32(s["qacc"]), time=t32(s["time"]), last_ctrl=t32(s["last"]))
    before = {k: v.clone() for k, v in st.items()}
    done = torch.zeros(N, dtype=torch.uint8, device=DEV); mask = torch.zeros(N, dtype=torch.uint8, device=DEV)
    tq = torch.zeros(N, m.nq, device=DEV); ep = torch.full((N,), 7, dtype=torch.int32, device=DEV)
    terms.terminate_reset(st, done=done, reset_mask=mask, traj_qpos=tq, episode_length=ep, reset_uniform=t32(u))
    dn = np.arange(N) % 3 == 0
    assert np.array_equal(done.cpu().numpy().astype(bool), dn) and torch.equal(done, mask)
    assert torch.equal(tq, before["qpos"])  # the transition records the pre-reset state
    keep = torch.from_numpy(~dn).to(DEV)
    for k in st:
        assert torch.equal(st[k][keep], before[k][keep]), k  # surviving envs are untouched, bit for bit
    q = st["qpos"].cpu().numpy()[dn]
    base = m.qpos0.copy(); base[2] += 0.1
    np.testing.assert_allclose(q[:, :2], np.broadcast_to(base[:2], q[:, :2].shape), atol=1e-7)
    np.testing.assert_allclose(q[:, 2], base[2] + 0.1 * u[dn, 2], atol=1e-6)
    np.testing.assert_allclose(q[:, 7:], np.clip(np.array(zeros) + 0.1 * u[dn, 7:m.nq], -0.25, 0.25), atol=1e-6)
    yaw = np.pi * u[dn, m.nq]
    np.testing.assert_allclose(q[:, 3:7], np.stack([np.cos(yaw / 2), 0 * yaw, 0 * yaw, np.sin(yaw / 2)], 1), atol=1e-6)
    for k in ("qvel", "qacc_warmstart", "time", "last_ctrl"):
        assert st[k].cpu().numpy()[dn].any() == False  # noqa: E712
    e = ep.cpu().numpy()
    assert (e[dn] == 0).all() and (e[~dn] == 8).all()
    # Philox draws: in range, reproducible
    st2 = {k: v.clone() for k, v in before.items()}; st3 = {k: v.clone() for k, v in before.items()}
    terms.terminate_reset(st2, seed=9, step=3); terms.terminate_reset(st3, seed=9, step=3)
    assert torch.equal(st2["qpos"], st3["qpos"])
    j = st2["qpos"].cpu().numpy()[dn][:, 7:]
    assert (np.abs(j) <= 0.25 + 1e-6).all() and j.std() > 0.03


def test_motion_height_field_and_pitch_roll_resets_match_the_reference_list_order():
    """InitialMotionStateReset, HFieldXYPositionReset / PlaneXYPositionReset and RandomPitchRollReset (resets.py:45-120,
    284-354) through the reset kernel, in three reset lists whose order matters, against the oracle's restatement applied
    in list order with the same draws; then with the kernel's own draws, through what the draws must satisfy."""
    from ksim_amd import model as km, resets as rs, terminations as tm
    from ksim_amd.env_terms import EnvTerms
    from ksim_amd.priors import MotionReferenceData

    m = km.kbot_scale_model()
    N, F = 96, 11
    rng = np.random.default_rng(21)
    mq = rng.normal(size=(F, m.nq)) * 0.3
    mq[:, 3:7] /= np.linalg.norm(mq[:, 3:7], axis=1, keepdims=True)
    motion = MotionReferenceData(qpos=mq, qvel=np.zeros((F, m.nv)), cartesian_poses={}, ctrl_dt=0.02)
    hf = rng.uniform(0.0, 0.4, size=(9, 7))
    hreset = rs.HFieldXYPositionReset(bounds=(4.0, 3.0, 0.25, 0.1), padded_bounds=(-3.0, 3.0, -2.0, 2.0), x_range=5.0, y_range=2.5,
                                      hfield_data=hf, robot_base_height=0.9)
    preset = rs.PlaneXYPositionReset(bounds=(5.0, 5.0, 0.05), padded_bounds=(-1.0, 1.0, -4.0, 4.0), x_range=2.0, y_range=3.0,
                                     robot_base_height=0.8)
    pr = rs.RandomPitchRollReset(pitch_range=(-0.3, 0.5), roll_range=(0.2, -0.4))
    cases = {
        "motion joints, height, pitch/roll then heading": [rs.InitialMotionStateReset(reference_motion=motion), rs.RandomHeightReset(range=(0.1, 0.3)), pr, rs.RandomHeadingReset()],
        "height field, heading then pitch/roll": [hreset, rs.RandomHeadingReset(), pr],
        "whole motion frame, plane overrides the position": [rs.InitialMotionStateReset(reference_motion=motion, freejoint=True), preset, pr],
    }
    u = rng.uniform(-1, 1, size=(N, m.nq + 1))
    upr = rng.random(N)
    frames = rng.integers(0, F, N).astype(np.int32)
    for name, resets in cases.items():
        terms = EnvTerms(m, {}, {"h": tm.MinimumHeightTermination(0.5)}, resets)
        s = _state(m, N, 5)
        st = dict(qpos=t32(s["qpos"]), qvel=t32(s["qvel"]), qacc_warmstart=t32(s["qacc"]), time=t32(s["time"]), last_ctrl=t32(s["last"]))
        draws = dict(reset_pitch_roll_uniform=t32(upr), reset_frame=torch.tensor(frames, device=DEV))
        terms.terminate_reset(st, level=0.7, apply_reset=2, reset_uniform=t32(u), episode=draws)
        got_q, got_t = st["qpos"].cpu().numpy(), st["time"].cpu().numpy()
        assert np.abs(st["qvel"].cpu().numpy()).max() == 0
        for e in range(N):
            q, t = m.qpos0.astype(np.float64).copy(), 0.0
            for r in resets:  # engine.py:209-211
                if isinstance(r, rs.InitialMotionStateReset):
                    q, t = ot.initial_motion_state_reset(q, int(frames[e]), mq, 0.02, r.freejoint)
                elif isinstance(r, rs.RandomHeightReset):
                    q[2] += r.range[0] + 0.5 * (u[e, 2] + 1) * (r.range[1] - r.range[0])
                elif isinstance(r, rs.RandomPitchRollReset):
                    q = ot.random_pitch_roll_reset(q, upr[e], r.pitch_range, r.roll_range)
                elif isinstance(r, rs.RandomHeadingReset):
                    q = ot.random_heading_reset(q, u[e, m.nq])
                elif isinstance(r, rs.HFieldXYPositionReset):
                    q = ot.xy_position_reset(q, u[e, 0], u[e, 1], x_range=r.x_range, y_range=r.y_range, padded_bounds=r.padded_bounds,
                                             hfield=hf.astype(np.float32), hfield_bounds=r.bounds[:3], robot_base_height=r.robot_base_height)
                else:
                    q = ot.xy_position_reset(q, u[e, 0], u[e, 1], x_range=r.x_range, y_range=r.y_range, padded_bounds=r.padded_bounds,
                                             z=r.bounds[2], robot_base_height=r.robot_base_height)
            np.testing.assert_allclose(got_q[e], q, atol=2e-6, err_msg=f"{name}, env {e}")
            assert got_t[e] == pytest.approx(t, abs=1e-6), name
        terms.close()
    # a height-field cell boundary is a discontinuity: no unclipped x above may sit near one (the clipped ones land on
    # cells 1 and 7 exactly, in float32 as in float64)
    x = u[:, 0] * 5.0
    cells = ((x[np.abs(x) < 3] + 4.0) / 8.0) * 8
    assert np.abs(cells - np.round(cells)).min() > 1e-4

    # the kernel's own draws: frames cover the motion, time = frame * dt, the joints are that frame's, and the base
    # orientation is quat0 * euler(roll, pitch, 0) with roll and pitch at the same fraction of their ranges
    N2 = 4096
    terms = EnvTerms(m, {}, {}, [rs.InitialMotionStateReset(reference_motion=motion), pr])
    st = dict(qpos=torch.zeros(N2, m.nq, device=DEV), qvel=torch.zeros(N2, m.nv, device=DEV), time=torch.zeros(N2, device=DEV))
    terms.terminate_reset(st, apply_reset=2, seed=3, step=5)
    q, t = st["qpos"].cpu().numpy().astype(np.float64), st["time"].cpu().numpy()
    fr = np.round(t / 0.02).astype(int)
    assert np.abs(t - fr * 0.02).max() < 1e-6 and set(fr) == set(range(F))
    counts = np.bincount(fr, minlength=F)
    assert counts.min() > 0.7 * N2 / F and counts.max() < 1.3 * N2 / F
    np.testing.assert_allclose(q[:, 7:], mq[fr][:, 7:], atol=1e-6)
    w, x, y, z = q[:, 3], q[:, 4], q[:, 5], q[:, 6]  # base quat0 is the identity here
    roll = np.arctan2(2 * (w * x + y * z), 1 - 2 * (x * x + y * y))
    pitch = np.arcsin(np.clip(2 * (w * y - z * x), -1, 1))
    fp, frl = (pitch + 0.3) / 0.8, (roll - 0.2) / -0.6
    assert fp.min() >= -1e-5 and fp.max() <= 1 + 1e-5 and fp.std() > 0.25
    np.testing.assert_allclose(fp, frl, atol=2e-5)
    np.testing.assert_allclose(np.arctan2(2 * (w * z + x * y), 1 - 2 * (y * y + z * z)), 0.0, atol=1e-5)  # no yaw
    st2 = dict(qpos=torch.zeros(N2, m.nq, device=DEV), qvel=torch.zeros(N2, m.nv, device=DEV), time=torch.zeros(N2, device=DEV))
    terms.terminate_reset(st2, apply_reset=2, seed=3, step=5)
    assert torch.equal(st2["qpos"], st["qpos"])  # same key, same draws
    terms.terminate_reset(st2, apply_reset=2, seed=3, step=6)
    assert not torch.equal(st2["time"], st["time"])


def test_reset_redraws_per_episode_quantities():
    """An env that is reset mid-rollout gets a new action latency, zero offset and actuator state, as MjxEngine.reset draws
    them under cond(done) (ksim/engine.py:222-245, ksim/actuators.py:219-238); a continuing env keeps its own."""
    from ksim_amd import actuators, engine, model as km, noise, physics, resets as rs, terminations as tm
    from ksim_amd.env_terms import EnvTerms

    m = km.kbot_scale_model()
    N, nu = 70, m.nu
    act = actuators.PositionActuators(kps=(50.0,) * nu, kds=(1.0,) * nu, action_bias=noise.UniformRandomVariable(0.0, 0.05),
                                      torque_bias=noise.GaussianRandomVariable(0.1, 0.5), kp_scale=noise.UniformRandomVariable(1.0, 0.2),
                                      kd_scale=0.9, torque_limit_scale=noise.GaussianRandomVariable(1.0, 0.05))
    cfg = engine.EngineConfig(dt=0.005, ctrl_dt=0.02, action_latency_range=(0.005, 0.015), zero_offset_std=0.01, zero_offset_mag=0.02)
    resets = [rs.RandomJointPositionReset(scale=0.1, scale_by_curriculum=False)]
    eng = engine.get_physics_engine("hip", resets, {}, act, cfg)
    dm = physics.DeviceModel(m)
    rng = np.random.default_rng(11)
    ned = 3 * nu + 4
    level = 0.6
    spec = dict(latency_range=(1.0, 3.0), zero_offset=dict(mean=0.0, mag=0.02, std=0.01, same_key=True),
                action_bias=dict(mean=0.0, mag=0.05, std=0.0), torque_bias=dict(mean=0.1, mag=0.0, std=0.5),
                kp_scale=dict(mean=1.0, mag=0.2, std=0.0), kd_scale=dict(mean=0.9, mag=0.0, std=0.0),
                torque_limit_scale=dict(mean=1.0, mag=0.0, std=0.05))

    def check(ps, rows, u, z):
        ast = ps.actuator_state
        got = dict(action_latency=ps.action_latency, zero_offset=ps.zero_offset, action=ast["action"], torque=ast["torque"],
                   kp_scale=ast["kp_scale"], kd_scale=ast["kd_scale"], torque_limit_scale=ast["torque_limit_scale"])
        got = {k: v.cpu().numpy() for k, v in got.items()}
        for e in rows:
            want = ot.engine_reset_draws(nu, level, u[e], z[e], **spec)
            for k, w in want.items():
                np.testing.assert_allclose(got[k][e], w, rtol=2e-6, atol=2e-7, err_msg=f"{k} of env {e}")

    # the first reset of every env draws them through the same kernel
    u0, z0 = rng.uniform(-1, 1, (N, ned)), rng.normal(size=(N, ned))
    ps = eng.reset(dm, level, 3, N, episode_draws=dict(uniform=t32(u0), normal=t32(z0)))
    check(ps, range(N), u0, z0)
    lat = ps.action_latency.cpu().numpy()
    assert (lat >= 1.0 * level - 1e-6).all() and (lat <= 3.0 * level + 1e-6).all() and lat.std() > 0.1
    # a control step later some envs have fallen: only those re-draw
    terms = EnvTerms(m, {}, {"h": tm.MinimumHeightTermination(0.5)}, resets)
    d = ps.data
    fallen = np.arange(N) % 5 == 2
    d.qpos[:, 2] = torch.from_numpy(np.where(fallen, 0.3, 0.9).astype(np.float32)).to(DEV)
    keep_before = {k: v.clone() for k, v in dict(lat=ps.action_latency, zo=ps.zero_offset, **ps.actuator_state).items()}
    u1, z1 = rng.uniform(-1, 1, (N, ned)), rng.normal(size=(N, ned))
    st = dict(qpos=d.qpos, qvel=d.qvel, qacc_warmstart=d.qacc_warmstart, time=d.time, last_ctrl=ps.last_ctrl)
    done = torch.zeros(N, dtype=torch.uint8, device=DEV)
    terms.terminate_reset(st, level=level, done=done, episode=eng.episode_args(ps, dict(uniform=t32(u1), normal=t32(z1))))
    assert np.array_equal(done.cpu().numpy().astype(bool), fallen)
    check(ps, np.nonzero(fallen)[0], u1, z1)
    after = dict(lat=ps.action_latency, zo=ps.zero_offset, **ps.actuator_state)
    keep = torch.from_numpy(~fallen).to(DEV)
    for k, v in after.items():
        assert torch.equal(v[keep], keep_before[k][keep]), k           # continuing envs: bit for bit the same
        assert not torch.equal(v[~keep], keep_before[k][~keep]) or k == "kd_scale", k  # reset envs: new values
    # Philox draws: reproducible for a (seed, step), in range, and different between steps
    snaps = []
    for step in (4, 4, 5):
        d.qpos[:, 2] = 0.3
        terms.terminate_reset(st, level=level, seed=21, step=step, episode=eng.episode_args(ps))
        snaps.append({k: v.clone() for k, v in dict(lat=ps.action_latency, zo=ps.zero_offset, **ps.actuator_state).items()})
    for k in snaps[0]:
        assert torch.equal(snaps[0][k], snaps[1][k]), k
    assert not torch.equal(snaps[0]["lat"], snaps[2]["lat"]) and not torch.equal(snaps[0]["zo"], snaps[2]["zo"])
    lat = snaps[0]["lat"].cpu().numpy()
    assert (lat >= 0.6 - 1e-6).all() and (lat <= 1.8 + 1e-6).all()
    kp = snaps[0]["kp_scale"].cpu().numpy()
    assert (np.abs(kp - 1.0) <= 0.2 + 1e-6).all() and kp.std() > 0.05
    zo = snaps[0]["zo"].cpu().numpy()
    assert (np.abs(zo) <= level * (0.02 + 5 * 0.01)).all() and zo.std() > 0.003


def test_constant_per_episode_quantities_are_not_streamed(monkeypatch):
    """A per-episode buffer whose random variable is a constant 0 (offsets, biases) or 1 (gain scales) holds that constant
    in every row, the step kernel's default for a null pointer: the engine hands the kernel only the buffers that vary
    (ksim/engine.py:117-138, ksim/actuators.py:90-95), and the step is bit for bit the one with all of them passed."""
    from ksim_amd import actuators, engine, model as km, noise, physics

    m = km.kbot_scale_model()
    N, nu = 48, m.nu
    dm = physics.DeviceModel(m)
    seen = []
    real_step = physics.control_step

    def spy(model, buf, **kw):
        seen.append({k: v is not None for k, v in buf.items()})
        return real_step(model, buf, **kw)

    monkeypatch.setattr(physics, "control_step", spy)
    action = t32(np.random.default_rng(5).normal(scale=0.2, size=(N, nu)))
    names = ("zero_offset", "action_bias", "torque_bias", "kp_scale", "kd_scale", "torque_limit_scale")

    def run(act, cfg, all_buffers=False):
        eng = engine.get_physics_engine("hip", [], {}, act, cfg)
        ps = eng.reset(dm, 1.0, 3, N)
        with monkeypatch.context() as mp:
            if all_buffers:
                mp.setattr(engine, "_constant", lambda rv, value: False)
            for _ in range(3):
                eng.step(action, dm, ps, 1.0, 7)
        return ps

    plain = actuators.PositionActuators(kps=(50.0,) * nu, kds=(1.0,) * nu)
    cfg0 = engine.EngineConfig(dt=0.005, ctrl_dt=0.02)
    a = run(plain, cfg0)
    assert not any(seen[-1][k] for k in names)
    b = run(plain, cfg0, all_buffers=True)
    assert all(seen[-1][k] for k in names)
    for k in ("qpos", "qvel", "qacc_warmstart"):
        assert torch.equal(getattr(a.data, k), getattr(b.data, k)), k
    assert torch.equal(a.last_ctrl, b.last_ctrl)
    # a scale that is a constant other than 1, or anything drawn, is streamed
    varied = actuators.PositionActuators(kps=(50.0,) * nu, kds=(1.0,) * nu, kd_scale=0.9,
                                         torque_bias=noise.GaussianRandomVariable(0.0, 0.5))
    run(varied, engine.EngineConfig(dt=0.005, ctrl_dt=0.02, zero_offset_std=0.01))
    want = dict(zero_offset=True, action_bias=False, torque_bias=True, kp_scale=False, kd_scale=True, torque_limit_scale=False)
    assert {k: seen[-1][k] for k in names} == want


def test_sample_action_scrub_and_clip():
    from ksim_amd.env_terms import sample_action

    N, nu = 33, 20
    rng = np.random.default_rng(1)
    mean = rng.normal(size=(N, nu)).astype(np.float32)
    mean[0, 0], mean[1, 1], mean[2, 2] = np.nan, 1e9, -1e9
    ls = rng.normal(size=nu).astype(np.float32) * 0.3
    z = rng.normal(size=(N, nu)).astype(np.float32)
    got = sample_action(t32(mean), t32(ls), noise=t32(z), clip_max=1e3).cpu().numpy()
    want = ot.scrub_action(mean.astype(np.float64) + np.exp(ls.astype(np.float64)) * z, 1e3)
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=2e-6)
    assert got[0, 0] == 0.0 and got[1, 1] == 1e3 and got[2, 2] == -1e3
    det = sample_action(t32(mean), None).cpu().numpy()
    np.testing.assert_array_equal(det, ot.scrub_action(mean, 1e3).astype(np.float32))
    a = sample_action(t32(mean), t32(ls), seed=3, step=4); b = sample_action(t32(mean), t32(ls), seed=3, step=4)
    assert torch.equal(a, b)


def _traj(Tn, N, nq, nv, nu, seed, p_done=0.1):
    rng = np.random.default_rng(seed)
    q = rng.normal(size=(Tn, N, nq)); q[..., 3:7] /= np.linalg.norm(q[..., 3:7], axis=-1, keepdims=True)
    done = rng.random((Tn, N)) < p_done
    return dict(qpos=q, qvel=rng.normal(size=(Tn, N, nv)), action=rng.normal(size=(Tn, N, nu)), done=done,
                success=done & (rng.random((Tn, N)) < 0.3))


def test_reward_kats_through_the_kernel():
    """The reference's own action-penalty vectors (tests/test_rewards.py:63-271), evaluated by the HIP kernel."""
    from ksim_amd import rewards as rw
    from ksim_amd.types import Trajectory

    cls = {"velocity": rw.ActionVelocityPenalty, "acceleration": rw.ActionAccelerationPenalty, "jerk": rw.ActionJerkPenalty}
    for kat in json.load(open(os.path.join(GOLD, "reward_kats.json"))):
        a = np.array(kat["actions"])[:, None, :]  # (T, N=1, 3)
        Tn = a.shape[0]
        done = np.zeros((Tn, 1), bool) if kat["done"] is None else np.array(kat["done"])[:, None]
        traj = Trajectory(qpos=None, qvel=None, xpos=None, xquat=None, ctrl=None, obs={}, command={}, event_state={},
                          action=t32(a), done=torch.from_numpy(done).to(DEV), success=None, timestep=None)
        out = rw.get_rewards(traj, {"p": cls[kat["fn"]](scale=1.0, norm=kat["norm"])})
        # a *Penalty enters the total with a negative sign (rl.py:219-221); the KAT is the raw term
        np.testing.assert_allclose(-out.total.cpu().numpy()[:, 0], kat["expected"], atol=kat["atol"], rtol=0)


def test_rewards_against_oracle():
    from ksim_amd import rewards as rw
    from ksim_amd.types import Trajectory

    Tn, N, nq, nv, nu = 40, 19, 27, 26, 20
    tr = _traj(Tn, N, nq, nv, nu, 7)
    rewards = {"stay_alive": rw.StayAliveReward(scale=1.0, success_reward=2.0), "height": rw.BaseHeightReward(scale=0.5, height_target=0.9),
               "range": rw.BaseHeightRangeReward(scale=0.3, z_lower=-0.5, z_upper=0.5, dropoff=2.0),
               "vel": rw.ActionVelocityPenalty(scale=0.01, norm="l1"), "acc": rw.ActionAccelerationPenalty(scale=0.02),
               "jerk": rw.ActionJerkPenalty(scale=0.03), "upright": rw.UprightReward(scale=0.7)}
    traj = Trajectory(qpos=t32(tr["qpos"]), qvel=t32(tr["qvel"]), xpos=None, xquat=None, ctrl=None, obs={}, command={},
                      event_state={}, action=t32(tr["action"]), done=torch.from_numpy(tr["done"]).to(DEV),
                      success=torch.from_numpy(tr["success"]).to(DEV), timestep=None)
    out = rw.get_rewards(traj, rewards, clip_min=-0.5, clip_max=2.5)
    comps = {}
    for e in range(N):
        a, dn, sc, q, v = tr["action"][:, e], tr["done"][:, e], tr["success"][:, e], tr["qpos"][:, e], tr["qvel"][:, e]
        up = ot.upright_reward(q, v)
        c = {"stay_alive": ot.stay_alive_reward(dn, sc, success_reward=2.0), "height": ot.base_height_reward(q, 0.9),
             "range": ot.base_height_range_reward(q, -0.5, 0.5, 2.0), "vel": ot.action_velocity_penalty(a, dn, "l1"),
             "acc": ot.action_acceleration_penalty(a, dn), "jerk": ot.action_jerk_penalty(a, dn),
             "upright/angvel": up["angvel"], "upright/linvel": up["linvel"], "upright/pose": up["pose"]}
        for k, val in c.items():
            comps.setdefault(k, []).append(val)
    scales = {"stay_alive": 1.0, "height": 0.5, "range": 0.3, "vel": 0.01, "acc": 0.02, "jerk": 0.03,
              "upright/angvel": 0.7, "upright/linvel": 0.7, "upright/pose": 0.7}
    pen = {k: k in ("vel", "acc", "jerk") for k in scales}
    stacked = {k: np.stack(v, axis=1) for k, v in comps.items()}
    total, scaled = ot.total_reward(stacked, scales, pen, clip_min=-0.5, clip_max=2.5)
    assert list(out.components) == list(scales)
    for k in scales:
        np.testing.assert_allclose(out.components[k].cpu().numpy(), scaled[k], rtol=1e-5, atol=2e-5, err_msg=k)
    np.testing.assert_allclose(out.total.cpu().numpy(), total, rtol=1e-5, atol=5e-5)


def test_amp_reward_from_discriminator_logits():
    """Discriminator forward (benchmark config 5 shape, 71 -> 256 -> 256 -> 1) and the AMP reward on its logits."""
    import torch.nn.functional as F
    from ksim_amd import rewards as rw
    from ksim_amd.mlp import MLP
    from ksim_amd.types import Trajectory

    Tn, N, dim = 32, 50, 71
    rng = np.random.default_rng(1005)
    dims = (dim, 256, 256, 1)
    ws = [rng.normal(scale=1 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])]
    bs = [rng.normal(scale=0.1, size=o).astype(np.float32) for o in dims[1:]]
    frames = rng.normal(size=(Tn, N, dim)).astype(np.float32)
    disc = MLP(ws, bs, activation="relu", dtype="f32")
    logits = disc(t32(frames.reshape(Tn * N, dim))).reshape(Tn, N)
    h = torch.from_numpy(frames.reshape(-1, dim)).double()
    for i, (w, b) in enumerate(zip(ws, bs)):
        h = F.linear(h, torch.from_numpy(w).double(), torch.from_numpy(b).double())
        if i + 1 < len(ws):
            h = F.relu(h)
    want_logits = h.numpy().reshape(Tn, N)
    np.testing.assert_allclose(logits.cpu().numpy(), want_logits, rtol=0, atol=2e-5 * np.abs(want_logits).max())
    done = torch.zeros(Tn, N, dtype=torch.bool, device=DEV)
    traj = Trajectory(qpos=None, qvel=None, xpos=None, xquat=None, ctrl=None, obs={}, command={}, event_state={},
                      action=None, done=done, success=done.clone(), timestep=None,
                      aux_outputs={rw.DISCRIMINATOR_OUTPUT_KEY: logits})
    out = rw.get_rewards(traj, {"amp_reward": rw.AMPReward(scale=0.5)})
    got_logits = logits.cpu().numpy().astype(np.float64)
    np.testing.assert_allclose(out.total.cpu().numpy(), 0.5 * ot.amp_reward(got_logits), rtol=1e-5, atol=1e-6)
    assert list(out.components) == ["amp_reward"]
    traj_missing = Trajectory(qpos=None, qvel=None, xpos=None, xquat=None, ctrl=None, obs={}, command={}, event_state={},
                              action=None, done=done, success=done.clone(), timestep=None)
    with pytest.raises(ValueError, match="auxiliary output is missing"):
        rw.get_rewards(traj_missing, {"amp_reward": rw.AMPReward(scale=0.5)})


def test_stateful_and_contact_observations():
    """Delay lines, the lagged and biased gravity reading and feet contact flags over several control steps, with
    some envs restarting in between (their carries are initialised from the state they restart in)."""
    from ksim_amd import _lib_terms as T, model as km, observation as ob
    from ksim_amd.env_terms import EnvTerms

    m = km.kbot_scale_model()
    N, steps = 19, 7
    rng = np.random.default_rng(3)
    observations = {
        "joint_position": ob.JointPositionObservation(),
        "delayed_position": ob.DelayedJointPositionObservation(delay_steps=3, noise=0.01),
        "gravity": ob.ProjectedGravityObservation(min_lag=0.3, max_lag=0.8, imu_bias=0.05),
        "contact": ob.FeetContactObservation(foot_left=(0, 1, 2, 3), foot_right=(4, 5, 6, 7)),
        "delayed_velocity": ob.DelayedJointVelocityObservation(delay_steps=1),
    }
    terms = EnvTerms(m, observations, {}, [])
    nj = m.nu
    assert terms.carry_dim == 3 * nj + 7 + nj and terms.obs_dim == nj + nj + 3 + 8 + nj
    K, C = terms.obs_dim, terms.carry_dim
    zero = rng.normal(size=(N, nj)) * 0.01
    carry = torch.full((N, C), float("nan"), device=DEV)  # never read before it is initialised
    # oracle-side carries
    dpos, dvel = [None] * N, [None] * N
    gx, glag, gbias = np.zeros((N, 3)), np.zeros(N), np.zeros((N, 3))
    sl = terms.obs_slices
    for k in range(steps):
        s = _state(m, N, 100 + k)
        dist = rng.normal(size=(N, m.ns)) * 0.01
        fresh = np.ones(N, bool) if k == 0 else (rng.random(N) < 0.3 if k in (3, 4) else np.zeros(N, bool))
        cu = rng.random((N, C))
        src = {T.SRC_QPOS: t32(s["qpos"]), T.SRC_QVEL: t32(s["qvel"]), T.SRC_CONTACT_DIST: t32(dist)}
        obs = torch.empty(N, K, device=DEV)
        terms.observe(src, N, zero_offset=t32(zero), carry=carry, fresh=torch.from_numpy(fresh.astype(np.uint8)).to(DEV),
                      carry_uniform=t32(cu), obs=obs)
        got = obs.cpu().numpy()
        g0 = 3 * nj  # the gravity carry follows the position delay line: x(3), lag, bias(3)
        for e in range(N):
            q, v = s["qpos"][e], s["qvel"][e]
            if fresh[e]:
                dpos[e], dvel[e] = np.tile(q[7:], (3, 1)), np.tile(v[6:], (1, 1))
                gx[e] = 0.0
                glag[e] = 0.3 + cu[e, g0 + 3] * 0.5
                gbias[e] = -0.05 + cu[e, g0 + 4:g0 + 7] * 0.1
            want_dp, dpos[e] = ot.delayed_observation(dpos[e], q[7:], zero[e])
            want_dv, dvel[e] = ot.delayed_observation(dvel[e], v[6:])
            gx[e] = ot.projected_gravity_ema(gx[e], glag[e], gbias[e], q[3:7])
            np.testing.assert_allclose(got[e, sl["delayed_position"]], want_dp, rtol=1e-6, atol=1e-6)
            np.testing.assert_allclose(got[e, sl["delayed_velocity"]], want_dv, rtol=1e-6, atol=1e-6)
            np.testing.assert_allclose(got[e, sl["gravity"]], gx[e], rtol=1e-5, atol=1e-5)
            want_c = ot.feet_contact_observation(dist[e].astype(np.float32), (0, 1, 2, 3), (4, 5, 6, 7))
            assert np.array_equal(got[e, sl["contact"]].reshape(4, 2), want_c)
            np.testing.assert_allclose(got[e, sl["joint_position"]], q[7:] - zero[e], rtol=1e-6, atol=1e-6)
    # the carry row holds what the reference keeps: delay slots oldest first, then x, lag, bias
    cr = carry.cpu().numpy()
    np.testing.assert_allclose(cr[:, :3 * nj].reshape(N, 3, nj), np.array(dpos), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(cr[:, g0 + 3], glag, rtol=1e-6)
    # Philox initial carries: lag and bias inside their ranges, reproducible for a seed
    c1, c2 = torch.zeros(N, C, device=DEV), torch.zeros(N, C, device=DEV)
    ones = torch.ones(N, dtype=torch.uint8, device=DEV)
    terms.observe(src, N, carry=c1, fresh=ones, seed=3, step=5, obs=obs)
    terms.observe(src, N, carry=c2, fresh=ones, seed=3, step=5, obs=obs)
    assert torch.equal(c1, c2)
    lag, bias = c1[:, g0 + 3], c1[:, g0 + 4:g0 + 7]
    assert ((lag >= 0.3) & (lag <= 0.8)).all() and (bias.abs() <= 0.05).all() and lag.std() > 0.05
    with pytest.raises(Exception, match="carry"):
        terms.observe(src, N, obs=obs)


def test_stateful_rewards_scan_against_oracle():
    """FeetAirTimeReward and SparseTargetHeightReward over two consecutive rollouts (the carry continues, and restarts
    for the envs whose rollout ends finished), mixed with stateless terms, total and components."""
    from ksim_amd import rewards as rw
    from ksim_amd.scales import LinearScale
    from ksim_amd.types import Trajectory

    Tn, N, nq, nv, nu = 24, 33, 27, 26, 20
    rng = np.random.default_rng(12)
    obs_slices = {"pad": slice(0, 5), "contact": slice(5, 9), "feet_pos": slice(9, 15), "tail": slice(15, 17)}
    rewards = {
        "alive": rw.StayAliveReward(scale=0.5),
        "air_time": rw.FeetAirTimeReward(scale=2.0, gait_period=LinearScale(scale=0.2, bias=0.1), air_time_percent=0.4,
                                         ctrl_dt=0.02, contact_obs="contact", bias=0.05, ground_penalty=0.2),
        "vel": rw.ActionVelocityPenalty(scale=0.01),
        "height": rw.SparseTargetHeightReward(scale=3.0, contact_obs="contact", position_obs="feet_pos", height=0.12),
        "cmd_air": rw.FeetAirTimeReward(scale=1.0, gait_period=0.25, air_time_percent=0.5, ctrl_dt=0.02, contact_obs="contact",
                                        linvel_cmd="lin", angvel_cmd="ang", linvel_moving_threshold=0.3),
    }
    level = 0.5
    period = np.float32(0.2 * level + 0.1)
    air1 = float(np.round(period * np.float32(0.4) / np.float32(0.02))); gnd1 = float(np.round(period * np.float32(0.6) / np.float32(0.02)))
    air2 = float(np.round(np.float32(0.25) * np.float32(0.5) / np.float32(0.02))); gnd2 = air2
    assert (air1, gnd1, air2) == (4.0, 6.0, 6.0)
    carry = None
    ocarry = [dict(a=(np.zeros(2, int),) * 3, h=np.zeros(2), c=(np.zeros(2, int),) * 3) for _ in range(N)]
    for rollout in range(2):
        obs = rng.normal(size=(Tn, N, 17)).astype(np.float32)
        obs[..., 5:9] = (rng.random((Tn, N, 4)) < 0.6)            # (c=2, n=2) contact flags, long stance phases
        obs[..., 9:15] = np.abs(rng.normal(size=(Tn, N, 6))) * 0.1
        qvel = rng.normal(size=(Tn, N, nv)).astype(np.float32) * 0.3
        cmd = rng.normal(size=(Tn, N, 3)).astype(np.float32) * 0.4
        done = rng.random((Tn, N)) < 0.05
        action = rng.normal(size=(Tn, N, nu)).astype(np.float32)
        traj = Trajectory(qpos=t32(rng.normal(size=(Tn, N, nq))), qvel=t32(qvel), xpos=None, xquat=None, ctrl=None,
                          obs={"obs": t32(obs)}, command={"_buffer": t32(cmd)}, event_state={}, action=t32(action),
                          done=torch.from_numpy(done).to(DEV), success=None, timestep=None)
        st = rw.get_rewards(traj, rewards, clip_max=5.0, rewards_carry=carry, obs_slices=obs_slices,
                            command_slices={"lin": slice(0, 1), "ang": slice(2, 3)}, level=level)
        carry = st.carry["_buffer"]
        assert list(st.components) == ["alive", "air_time/air", "air_time/gnd", "air_time/stationary_gnd", "vel", "height",
                                       "cmd_air/air", "cmd_air/gnd", "cmd_air/stationary_gnd"]
        comp = {k: v.cpu().numpy() for k, v in st.components.items()}
        total = st.total.cpu().numpy()
        for e in range(N):
            oc = ocarry[e]
            if done[-1, e]:  # ksim/task/rl.py:206-214: the carry this rollout starts from is the initial one
                oc = dict(a=(np.zeros(2, int),) * 3, h=np.zeros(2), c=(np.zeros(2, int),) * 3)
            con = obs[:, e, 5:9].reshape(Tn, 2, 2)
            a, oc["a"] = ot.feet_air_time_reward(con, qvel[:, e], done[:, e], oc["a"], air_steps=air1, gnd_steps=gnd1, bias=0.05,
                                                 ground_penalty=0.2)
            h, oc["h"] = ot.sparse_target_height_reward(con, obs[:, e, 9:15].reshape(Tn, 2, 3), qvel[:, e], done[:, e], oc["h"],
                                                        height=0.12)
            c, oc["c"] = ot.feet_air_time_reward(con, qvel[:, e], done[:, e], oc["c"], air_steps=air2, gnd_steps=gnd2,
                                                 linvel_threshold=0.3, lin_cmd_t=cmd[:, e, 0], ang_cmd_t=cmd[:, e, 2])
            ocarry[e] = oc
            for k in ("air", "gnd", "stationary_gnd"):
                np.testing.assert_allclose(comp[f"air_time/{k}"][:, e], 2.0 * a[k], rtol=1e-6, atol=1e-6)
                np.testing.assert_allclose(comp[f"cmd_air/{k}"][:, e], c[k], rtol=1e-6, atol=1e-6)
            np.testing.assert_allclose(comp["height"][:, e], 3.0 * h, rtol=1e-6, atol=1e-6)
        want_total = np.minimum(sum(comp.values()), 5.0)
        np.testing.assert_allclose(total, want_total, rtol=1e-5, atol=1e-5)
        cr = carry.cpu().numpy()
        np.testing.assert_allclose(cr[:, 0:6], [np.concatenate(o["a"]) for o in ocarry])
        np.testing.assert_allclose(cr[:, 6:8], [o["h"] for o in ocarry], rtol=1e-6)
        np.testing.assert_allclose(cr[:, 8:14], [np.concatenate(o["c"]) for o in ocarry])
    with pytest.raises(KeyError, match="contact"):
        rw.get_rewards(traj, rewards, obs_slices={"feet_pos": slice(0, 6)}, command_slices={"lin": slice(0, 1), "ang": slice(2, 3)})


def test_symmetry_and_joint_position_rewards_against_oracle():
    """SymmetryReward, PairwiseSymmetryReward (stateful: the carry follows the rollout mean, restarts at the targets when
    the rollout ended on a done step) and JointPositionReward over two consecutive rollouts, beside a stateless term."""
    from ksim_amd import rewards as rw
    from ksim_amd.types import Trajectory

    Tn, N, nq, nv, nu = 16, 37, 27, 26, 20
    rng = np.random.default_rng(31)
    joints, targets = (0, 5, 3, 12, 19), (0.1, -0.2, 0.0, 0.3, -0.05)
    cmd_idx = (2, 7, 11)
    rewards = {
        "alive": rw.StayAliveReward(scale=0.5),
        "sym": rw.SymmetryReward(scale=1.5, joint_indices=joints, joint_targets=targets, alpha=0.2),
        "hips": rw.PairwiseSymmetryReward(scale=0.7, left_joint_index=1, right_joint_index=6, left_zero=0.05, right_zero=-0.1,
                                          flipped=True, alpha=0.3, kernel_scale=0.4, sq_scale=0.2, abs_scale=0.15),
        "arms": rw.JointPositionReward(scale=2.0, command_name="arm_cmd", indices=cmd_idx, pos_scale=0.3, vel_scale=0.6,
                                       sq_scale=0.05, abs_scale=0.1),
    }
    command_slices = {"other": slice(0, 2), "arm_cmd": slice(2, 2 + 2 * 3 + 3)}
    carry = None
    oc_sym = [np.array(targets) for _ in range(N)]
    oc_pair = [np.array([0.05, -0.1]) for _ in range(N)]
    for rollout in range(2):
        qpos = rng.normal(size=(Tn, N, nq)).astype(np.float32) * 0.3
        qvel = rng.normal(size=(Tn, N, nv)).astype(np.float32) * 0.5
        cmd = rng.normal(size=(Tn, N, 11)).astype(np.float32) * 0.4
        cmd[..., 8] = rng.uniform(0.1, 1.0, (Tn, N))                       # total_time
        cmd[..., 9] = np.ceil(cmd[..., 8] / 0.02)                          # num_steps
        cmd[..., 10] = np.floor(rng.random((Tn, N)) * (cmd[..., 9] + 1))   # step_id
        done = rng.random((Tn, N)) < 0.05
        done[-1] = rng.random(N) < 0.4
        traj = Trajectory(qpos=t32(qpos), qvel=t32(qvel), xpos=None, xquat=None, ctrl=None, obs={}, command={"_buffer": t32(cmd)},
                          event_state={}, action=t32(rng.normal(size=(Tn, N, nu))), done=torch.from_numpy(done).to(DEV), success=None,
                          timestep=None)
        st = rw.get_rewards(traj, rewards, rewards_carry=carry, command_slices=command_slices)
        carry = st.carry["_buffer"]
        assert list(st.components) == ["alive", "sym", "hips/lr", "hips/self", "arms/pos", "arms/vel"]
        comp = {k: v.cpu().numpy() for k, v in st.components.items()}
        want_total = np.zeros((Tn, N))
        for e in range(N):
            r, oc_sym[e] = ot.symmetry_reward(qpos[:, e], oc_sym[e], bool(done[-1, e]), joints, targets, alpha=0.2)
            pr, oc_pair[e] = ot.pairwise_symmetry_reward(qpos[:, e], oc_pair[e], bool(done[-1, e]), 1, 6, 0.05, -0.1, flipped=True, alpha=0.3,
                                                         kernel_scale=0.4, sq_scale=0.2, abs_scale=0.15)
            jp = ot.joint_position_reward(qpos[:, e].astype(np.float64), qvel[:, e].astype(np.float64), cmd[:, e, 2:5].astype(np.float64),
                                          cmd[:, e, 5:8].astype(np.float64), cmd[:, e, 8].astype(np.float64), cmd[:, e, 9].astype(np.float64),
                                          cmd[:, e, 10].astype(np.float64), cmd_idx, pos_scale=0.3, vel_scale=0.6, sq_scale=0.05, abs_scale=0.1)
            np.testing.assert_allclose(comp["sym"][:, e], 1.5 * r, rtol=2e-5, atol=2e-6)
            np.testing.assert_allclose(comp["hips/lr"][:, e], 0.7 * pr["lr"], rtol=2e-5, atol=2e-6)
            np.testing.assert_allclose(comp["hips/self"][:, e], 0.7 * pr["self"], rtol=2e-5, atol=2e-6)
            np.testing.assert_allclose(comp["arms/pos"][:, e], 2.0 * jp["pos"], rtol=2e-5, atol=2e-6)
            np.testing.assert_allclose(comp["arms/vel"][:, e], 2.0 * jp["vel"], rtol=2e-5, atol=2e-6)
            want_total[:, e] = 1.5 * r + 0.7 * (pr["lr"] + pr["self"]) + 2.0 * (jp["pos"] + jp["vel"]) + comp["alive"][:, e]
        np.testing.assert_allclose(st.total.cpu().numpy(), want_total, rtol=2e-5, atol=1e-5)
        cr = carry.cpu().numpy()
        np.testing.assert_allclose(cr[:, :5], np.array(oc_sym), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(cr[:, 5:7], np.array(oc_pair), rtol=1e-5, atol=1e-6)
    assert rw.reward_carry_size(rewards) == 7
    with pytest.raises(ValueError, match="not found"):
        rw.get_rewards(traj, rewards, command_slices={"other": slice(0, 2)})


def test_gaussian_head_with_state_dependent_deviation():
    """mean | raw deviation head (examples/kbot/train.py:915-932): softplus, floor, scale and cap of the deviation, the
    sample, its log-density against scipy, scrub and clip."""
    from scipy.stats import norm
    from ksim_amd.env_terms import sample_action_head

    rng = np.random.default_rng(8)
    N, nu = 77, 20
    raw = rng.normal(size=(N, 2 * nu)) * 2.0
    raw[0, nu] = 50.0        # softplus in its linear range -> capped by max_std
    raw[1, nu + 1] = -40.0   # softplus underflows -> the floor min_std
    raw[2, 3] = np.nan       # a NaN mean is scrubbed to 0 after sampling
    bias = rng.normal(size=nu) * 0.1
    z = rng.normal(size=(N, nu))
    out, mean, std, logp = sample_action_head(t32(raw), min_std=0.01, max_std=1.5, var_scale=0.5, mean_bias=t32(bias),
                                              noise=t32(z), clip_max=2.0, want_stats=True)
    w_mean = raw[:, :nu] + bias
    w_std = np.minimum((np.logaddexp(0.0, raw[:, nu:]) + 0.01) * 0.5, 1.5)
    assert std[0, 0].item() == 1.5 and abs(std[1, 1].item() - 0.005) < 1e-7
    np.testing.assert_allclose(std.cpu().numpy(), w_std, rtol=2e-6)
    ok = ~np.isnan(w_mean)
    np.testing.assert_allclose(mean.cpu().numpy()[ok], w_mean[ok], rtol=1e-6, atol=1e-6)
    sample = w_mean + w_std * z
    want = np.clip(np.where(np.isnan(sample), 0.0, sample), -2.0, 2.0)
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=1e-5, atol=1e-5)
    assert out[2, 3].item() == 0.0 and (np.abs(sample[ok]) > 2.0).any()
    np.testing.assert_allclose(logp.cpu().numpy()[ok], norm.logpdf(sample[ok], w_mean[ok], w_std[ok]), rtol=1e-4, atol=1e-4)
    det = sample_action_head(t32(raw), min_std=0.01, max_std=1.5, var_scale=0.5, mean_bias=t32(bias), deterministic=True, clip_max=10.0)
    np.testing.assert_allclose(det.cpu().numpy()[ok], w_mean[ok], rtol=1e-6, atol=1e-6)
    # Philox: reproducible per (seed, step), standard normal scores
    a1 = sample_action_head(t32(raw), min_std=0.01, max_std=1.5, seed=4, step=9, clip_max=1e3, want_stats=True)
    a2 = sample_action_head(t32(raw), min_std=0.01, max_std=1.5, seed=4, step=9, clip_max=1e3)
    a3 = sample_action_head(t32(raw), min_std=0.01, max_std=1.5, seed=4, step=10, clip_max=1e3)
    assert torch.equal(a1[0], a2) and not torch.equal(a2, a3)
    zs = ((a1[0] - a1[1]) / a1[2]).cpu().numpy()[ok]
    assert abs(zs.mean()) < 0.1 and abs(zs.std() - 1.0) < 0.1
    with pytest.raises(Exception, match="2 nu"):
        sample_action_head(t32(raw[:, :-1]), min_std=0.01, max_std=1.0)


def test_body_velocity_inertia_and_debug_observations():
    """Observations over the step kernel's extra outputs (cvel, cinert) and the small gather classes."""
    from ksim_amd import _lib_terms as T, model as km, observation as ob
    from ksim_amd.env_terms import EnvTerms

    m = km.kbot_scale_model()
    N = 9
    s = _state(m, N, 21)
    rng = s["rng"]
    cvel, cinert, xquat = rng.normal(size=(N, m.nb * 6)), rng.normal(size=(N, m.nb * 10)), rng.normal(size=(N, m.nb * 4))
    observations = {"inertia": ob.CenterOfMassInertiaObservation(), "body_vel": ob.BodyVelocityObservation(body_idxs=(3, 1)),
                    "feet_quat": ob.FeetOrientationObservation(body_ids=(5, 9)), "act_pos": ob.ActPosObservation(ctrl_idx=4, qpos_idx=11)}
    terms = EnvTerms(m, observations, {}, [])
    assert terms.obs_dim == (m.nb - 1) * 10 + 12 + 8 + 2 and T.SRC_CINERT in terms.sources_used
    src = {T.SRC_QPOS: t32(s["qpos"]), T.SRC_CVEL: t32(cvel), T.SRC_CINERT: t32(cinert), T.SRC_XQUAT: t32(xquat),
           T.SRC_LAST_ACTION: t32(s["last"])}
    obs = torch.empty(N, terms.obs_dim, device=DEV)
    terms.observe(src, N, obs=obs)
    want = np.concatenate([cinert[:, 10:], cvel[:, 18:24], cvel[:, 6:12], xquat[:, 20:24], xquat[:, 36:40],
                           s["last"][:, 4:5], s["qpos"][:, 11:12]], axis=1)
    np.testing.assert_allclose(obs.cpu().numpy(), want.astype(np.float32), rtol=0, atol=0)
    with pytest.raises(ValueError):
        ob.FeetOrientationObservation(body_ids=(1, 2, 3))


def test_command_tracking_rest_and_force_rewards():
    """The rewards of the shipped walking tasks that read commands and contact forces, against the oracle."""
    from ksim_amd import rewards as rw
    from ksim_amd.types import Trajectory

    Tn, N, nq, nv = 16, 29, 27, 26
    rng = np.random.default_rng(31)
    qpos = rng.normal(size=(Tn, N, nq)); qpos[..., 3:7] /= np.linalg.norm(qpos[..., 3:7], axis=-1, keepdims=True)
    qvel = rng.normal(size=(Tn, N, nv)) * 0.5
    cmd = rng.normal(size=(Tn, N, 8)) * 0.5
    cmd[::3, :, 1] = 0.003            # some zero linear commands
    cmd[1::4, :, 7] = 0.01            # some yaw commands inside the dead band
    obs = rng.normal(size=(Tn, N, 12)) * 30
    done = rng.random((Tn, N)) < 0.05
    rewards = {"lin": rw.LinearVelocityReward(scale=1.5, cmd="lin_cmd", vel_length_scale=0.3, yaw_length_scale=0.5),
               "ang": rw.AngularVelocityReward(scale=0.7, cmd="ang_cmd"),
               "off": rw.OffAxisVelocityReward(scale=0.2, ang_length_scale=0.4),
               "rest": rw.MotionlessAtRestPenalty(scale=0.1),
               "force": rw.ForcePenalty(scale=0.05, force_obs="feet_force", expected_weight=40.0, bias=5.0),
               "alive": rw.StayAliveReward(scale=1.0)}
    traj = Trajectory(qpos=t32(qpos), qvel=t32(qvel), xpos=None, xquat=None, ctrl=None, obs={"obs": t32(obs)},
                      command={"_buffer": t32(cmd)}, event_state={}, action=None, done=torch.from_numpy(done).to(DEV), success=None,
                      timestep=None)
    st = rw.get_rewards(traj, rewards, obs_slices={"x": slice(0, 4), "feet_force": slice(4, 10)},
                        command_slices={"lin_cmd": slice(1, 7), "ang_cmd": slice(7, 8)})
    f32 = lambda a: a.astype(np.float32).astype(np.float64)  # noqa: E731
    q, v, c, o = f32(qpos), f32(qvel), f32(cmd), f32(obs)
    lin = ot.linear_velocity_reward(q, v, c[..., 1:5], vel_length_scale=0.3, yaw_length_scale=0.5)
    ang = ot.angular_velocity_reward(v, c[..., 7])
    off = ot.off_axis_velocity_reward(v, ang_length_scale=0.4)
    want = {**{f"lin/{k}": 1.5 * x for k, x in lin.items()}, **{f"ang/{k}": 0.7 * x for k, x in ang.items()},
            **{f"off/{k}": 0.2 * x for k, x in off.items()}, "rest": -0.1 * ot.motionless_at_rest_penalty(v),
            "force": -0.05 * ot.force_penalty(o[..., 4:10].reshape(Tn, N, 2, 3), 40.0, 5.0)}
    assert list(st.components)[:-1] == list(want)
    for k, w in want.items():
        got = st.components[k].cpu().numpy()
        if k == "lin/yaw":  # atan2 near the branch cut +-pi can land on the other side in fp32
            close = np.abs(got - w) < 2e-4
            assert close.mean() > 0.995
        else:
            np.testing.assert_allclose(got, w, rtol=2e-5, atol=2e-5, err_msg=k)
    assert (st.components["lin/x"][::3] == 0).all() and (st.components["ang/dir"].abs() == 0.7).all()
    total = sum(st.components[k] for k in st.components)
    np.testing.assert_allclose(st.total.cpu().numpy(), total.cpu().numpy(), rtol=1e-5, atol=1e-5)
    with pytest.raises(KeyError, match="nope"):
        rw.get_rewards(traj, {"lin": rw.LinearVelocityReward(cmd="nope")}, command_slices={"lin_cmd": slice(0, 4)})
    with pytest.raises(Exception, match="command"):
        rw.get_rewards(traj, {"ang": rw.AngularVelocityReward(cmd="a")}, command_slices={"a": slice(8, 9)})


def test_smoothness_limits_effort_and_body_frame_rewards():
    """The remaining stateless rewards of ksim/rewards.py against the oracle: joint and link smoothness (with episode ends
    inside the rollout and at its first steps), limit avoidance, torque and energy, joint deviation, flat bodies, position
    tracking, roll, feet slip."""
    from ksim_amd import model as km
    from ksim_amd import rewards as rw
    from ksim_amd.types import Trajectory

    m = km.kbot_scale_model(joint_range=(-0.8, 0.9))
    Tn, N, nq, nv, nu, nb = 24, 13, m.nq, m.nv, m.nu, m.nb
    rng = np.random.default_rng(77)
    qpos = rng.normal(size=(Tn, N, nq)) * 0.7; qpos[..., 3:7] /= np.linalg.norm(qpos[..., 3:7], axis=-1, keepdims=True)
    qpos[..., 7:] = np.cumsum(rng.normal(size=(Tn, N, nq - 7)) * 0.1, axis=0)   # smooth enough that the kernels are not all ~0
    qvel = rng.normal(size=(Tn, N, nv))
    ctrl = rng.normal(size=(Tn, N, nu)) * 10
    xpos = np.cumsum(rng.normal(size=(Tn, N, nb, 3)) * 0.05, axis=0)
    xquat = rng.normal(size=(Tn, N, nb, 4)); xquat /= np.linalg.norm(xquat, axis=-1, keepdims=True)
    cmd = rng.normal(size=(Tn, N, 5)) * 0.2
    obs = rng.normal(size=(Tn, N, 20)); obs[..., 2:6] = rng.random((Tn, N, 4)) < 0.4   # contact flags (c = 2, n = 2)
    done = rng.random((Tn, N)) < 0.12
    done[0, :4] = True; done[1, 2:6] = True
    targets = (0.1, -0.2, 0.3)
    rewards = {"jv": rw.SmallJointVelocityReward(scale=0.5, kernel_scale=0.2), "ja": rw.SmallJointAccelerationReward(scale=0.6),
               "jj": rw.SmallJointJerkReward(scale=0.7, kernel_scale=0.4),
               "limits": rw.AvoidLimitsPenalty.create(m, factor=0.05, scale=0.3),
               "torque": rw.TorquePenalty(ctrl_scales=tuple(float(x) for x in np.linspace(5.0, 40.0, nu)), scale=0.01),
               "energy": rw.EnergyPenalty(ctrl_scales=tuple(float(x) for x in np.linspace(40.0, 5.0, nu)), scale=0.02),
               "dev": rw.JointDeviationPenalty(scale=0.4, norm="l1", joint_indices=(0, 7, 19), joint_targets=targets, joint_weights=(1.0, 2.0, 0.5)),
               "dev2": rw.JointDeviationPenalty.create(m, [m.body_names[3], m.body_names[5]], (0.0, 0.5), scale=0.2),
               "flat": rw.FlatBodyReward(scale=0.9, body_indices=(1, 4, nb - 1), plane=(0.0, 0.6, 0.8)),
               "track": rw.PositionTrackingReward(scale=1.1, tracked_body_idx=6, base_body_idx=1, command_name="hand", norm="l2", kernel_scale=0.5),
               "roll": rw.NoRollReward(scale=0.8, roll_scale=0.5, angvel_abs_scale=0.2),
               "lacc": rw.LinkAccelerationPenalty(scale=2.0, norm="l1"), "ljerk": rw.LinkJerkPenalty(scale=3.0),
               "slip": rw.FeetSlipPenalty(scale=0.1, contact_obs="contact", velocity_obs="feet_vel")}
    traj = Trajectory(qpos=t32(qpos), qvel=t32(qvel), xpos=t32(xpos.reshape(Tn, N, -1)), xquat=t32(xquat), ctrl=t32(ctrl),
                      obs={"obs": t32(obs)}, command={"_buffer": t32(cmd)}, event_state={}, action=None,
                      done=torch.from_numpy(done).to(DEV), success=None, timestep=None)
    st = rw.get_rewards(traj, rewards, obs_slices={"contact": slice(2, 6), "feet_vel": slice(7, 19)}, command_slices={"hand": slice(1, 4)})
    f32 = lambda a: a.astype(np.float32).astype(np.float64)  # noqa: E731
    q, v, c, xp, xq, cm, ob = f32(qpos), f32(qvel), f32(ctrl), f32(xpos), f32(xquat), f32(cmd), f32(obs)
    lim = ot.avoid_limits_create(m.jnt_range[1:m.nb], np.asarray(m.jnt_limited[1:m.nb]).astype(bool), 0.05)
    t_scales, e_scales = np.linspace(5.0, 40.0, nu), np.linspace(40.0, 5.0, nu)
    qa = [int(m.body_qadr[3]) - 7, int(m.body_qadr[5]) - 7]
    want = {k: [] for k in ("jv", "ja", "jj", "limits", "torque", "energy", "dev", "dev2", "flat", "track", "roll/angvel", "roll/pose",
                            "lacc", "ljerk", "slip")}
    for e in range(N):
        dn = done[:, e]
        ang, pose = ot.no_roll_reward(q[:, e], v[:, e], s=0.25, sq=0.1, ab=0.2)
        _, pose = ot.no_roll_reward(q[:, e], v[:, e], s=0.5, sq=0.1, ab=0.1)
        vals = {"jv": 0.5 * ot.small_joint_reward(q[:, e], dn, 1, 0.2), "ja": 0.6 * ot.small_joint_reward(q[:, e], dn, 2),
                "jj": 0.7 * ot.small_joint_reward(q[:, e], dn, 3, 0.4), "limits": -0.3 * ot.avoid_limits_penalty(q[:, e], lim),
                "torque": -0.01 * ot.torque_penalty(c[:, e], t_scales), "energy": -0.02 * ot.energy_penalty(c[:, e], v[:, e], e_scales),
                "dev": -0.4 * ot.joint_deviation_penalty(q[:, e], (0, 7, 19), targets, (1.0, 2.0, 0.5), "l1"),
                "dev2": -0.2 * ot.joint_deviation_penalty(q[:, e], qa, (0.0, 0.5), None, "l2"),
                "flat": 0.9 * ot.flat_body_reward(xq[:, e], (1, 4, nb - 1), (0.0, 0.6, 0.8)),
                "track": 1.1 * ot.position_tracking_reward(xp[:, e], cm[:, e, 1:4], 6, 1, "l2", 0.5),
                "roll/angvel": 0.8 * ang, "roll/pose": 0.8 * pose,
                "lacc": -2.0 * ot.link_smoothness_penalty(xp[:, e], dn, 2, "l1"), "ljerk": -3.0 * ot.link_smoothness_penalty(xp[:, e], dn, 3, "l2"),
                "slip": -0.1 * ot.feet_slip_penalty(ob[:, e, 2:6].reshape(Tn, 2, 2), ob[:, e, 7:19].reshape(Tn, 2, 6))}
        for k, x in vals.items():
            want[k].append(x)
    assert list(st.components) == list(want)
    assert np.isfinite(lim).all() and (ot.avoid_limits_penalty(q[:, 0], lim) > 0).any()
    for k, w in want.items():
        w = np.stack(w, axis=1)
        assert np.abs(w).max() > 1e-3, k
        np.testing.assert_allclose(st.components[k].cpu().numpy(), w, rtol=3e-5, atol=3e-5, err_msg=k)
    total = sum(st.components[k] for k in st.components)
    np.testing.assert_allclose(st.total.cpu().numpy(), total.cpu().numpy(), rtol=1e-5, atol=1e-5)
    # error paths: a joint or body outside the model, a table that does not fit, missing leaves
    with pytest.raises(Exception, match="joint"):
        rw.get_rewards(traj, {"dev": rw.JointDeviationPenalty(joint_indices=(nq,), joint_targets=(0.0,))})
    with pytest.raises(Exception, match="body"):
        rw.get_rewards(traj, {"flat": rw.FlatBodyReward(body_indices=(nb,))})
    with pytest.raises(Exception, match="constants"):
        rw.get_rewards(traj, {"limits": rw.AvoidLimitsPenalty(joint_limits=((-1.0, 1.0),) * 3)})
    with pytest.raises(Exception, match="zero control scale"):
        rw.get_rewards(traj, {"t": rw.TorquePenalty(ctrl_scales=(0.0,) * nu)})
    with pytest.raises(ValueError, match="sorted"):
        rw.AvoidLimitsPenalty(joint_limits=((1.0, -1.0),))
    import dataclasses
    with pytest.raises(Exception, match="trajectory.ctrl"):
        rw.get_rewards(dataclasses.replace(traj, ctrl=None), {"t": rewards["torque"]})


def test_reachability_and_intersection_penalties():
    from ksim_amd import rewards as rw
    from ksim_amd.types import Trajectory

    Tn, N, nu = 9, 21, 6
    rng = np.random.default_rng(5)
    qpos = rng.normal(size=(Tn, N, nu + 7)) * 0.3
    action = rng.normal(size=(Tn, N, nu)) * 0.3
    obs = rng.normal(size=(Tn, N, 11)) * 0.12
    dm = tuple(float(x) for x in np.linspace(0.05, 0.3, nu))
    traj = Trajectory(qpos=t32(qpos), qvel=None, xpos=None, xquat=None, ctrl=None, obs={"obs": t32(obs)}, command={}, event_state={},
                      action=t32(action), done=torch.zeros(Tn, N, dtype=torch.bool, device=DEV), success=None, timestep=None)
    st = rw.get_rewards(traj, {"reach": rw.ReachabilityPenalty(scale=2.0, delta_max_j=dm), "reach1": rw.ReachabilityPenalty(delta_max_j=dm, squared=False),
                               "cross": rw.IntersectionPenalty(scale=0.5, position_obs="feet", min_distance=0.15)},
                        obs_slices={"feet": slice(1, 10)})
    f32 = lambda a: a.astype(np.float32).astype(np.float64)  # noqa: E731
    q, a, o = f32(qpos), f32(action), f32(obs)
    for e in range(N):
        np.testing.assert_allclose(st.components["reach"][:, e].cpu().numpy(), -2.0 * ot.reachability_penalty(a[:, e], q[:, e], dm), rtol=2e-5, atol=1e-6)
        np.testing.assert_allclose(st.components["reach1"][:, e].cpu().numpy(), -ot.reachability_penalty(a[:, e], q[:, e], dm, False), rtol=2e-5, atol=1e-6)
        np.testing.assert_array_equal(st.components["cross"][:, e].cpu().numpy(), -0.5 * ot.intersection_penalty(o[:, e, 1:10].reshape(Tn, 3, 3), 0.15))
    frac = float((st.components["cross"] != 0).float().mean())
    assert 0.1 < frac < 0.9
    short = Trajectory(qpos=t32(qpos[..., :10]), qvel=None, xpos=None, xquat=None, ctrl=None, obs={}, command={}, event_state={},
                       action=t32(action), done=torch.zeros(Tn, N, dtype=torch.bool, device=DEV), success=None, timestep=None)
    with pytest.raises(Exception, match="one joint per action"):
        rw.get_rewards(short, {"reach": rw.ReachabilityPenalty(delta_max_j=dm)})


def test_velocity_commands_against_oracle():
    """LinearVelocityCommand / AngularVelocityCommand over several control steps with explicit draws: episode starts,
    slewing, switches, zero and backward targets; the recorded copy is the incoming command."""
    from ksim_amd import _lib_terms as T
    from ksim_amd.commands import AngularVelocityCommand, CommandSet, ConstantCommand, LinearVelocityCommand
    from ksim_amd.scales import LinearScale

    N, steps, level = 41, 12, 0.5
    rng = np.random.default_rng(41)
    lp = dict(min_vel=0.3, max_vel=LinearScale(scale=2.0, bias=0.5), max_yaw=0.4, zero_prob=0.2, backward_prob=0.3, switch_prob=0.15,
              ctrl_dt=0.02, linear_accel=3.0, angular_accel=2.0)
    ap = dict(max_vel=1.0, min_vel=0.1, zero_prob=0.25, switch_prob=0.2, ctrl_dt=0.02, angular_accel=1.5)
    cs = CommandSet({"pad": ConstantCommand(size=3), "lin": LinearVelocityCommand(**lp), "ang": AngularVelocityCommand(**ap)})
    assert cs.command_dim == 11 and cs.slices["lin"] == slice(3, 9)
    lpo = dict(lp, max_vel=2.0 * level + 0.5)
    cmd = cs.initial(N, DEV)
    cmd[:, :3] = 7.0
    want = np.zeros((N, 11)); want[:, :3] = 7.0
    for k in range(steps):
        qpos = rng.normal(size=(N, 27)); qpos[:, 3:7] /= np.linalg.norm(qpos[:, 3:7], axis=1, keepdims=True)
        qvel = rng.normal(size=(N, 26))
        u = rng.random((N, 3, T.KS_COMMAND_DRAWS)).astype(np.float32)
        fresh = np.ones(N, bool) if k == 0 else rng.random(N) < 0.1
        rec = torch.empty(N, 11, device=DEV)
        cs.update(cmd, t32(qpos), t32(qvel), level=level, fresh=torch.from_numpy(fresh.astype(np.uint8)).to(DEV), record=rec, uniform=t32(u))
        np.testing.assert_allclose(rec.cpu().numpy(), want, rtol=1e-5, atol=1e-6)
        q32, v32 = qpos.astype(np.float32).astype(np.float64), qvel.astype(np.float32).astype(np.float64)
        for e in range(N):
            want[e, 3:9] = ot.linear_velocity_command(want[e, 3:9], q32[e], v32[e], u[e, 1].astype(np.float64), bool(fresh[e]), **lpo)
            want[e, 9:11] = ot.angular_velocity_command(want[e, 9:11], v32[e], u[e, 2].astype(np.float64), bool(fresh[e]), **ap)
        got = cmd.cpu().numpy()
        # heading measured at an episode start sits on atan2's branch cut for a robot moving straight backwards
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5)
    assert (want[:, 7] == 0).any() and (want[:, 7] < 0).any() and (cmd[:, :3] == 7.0).all()
    # Philox: reproducible, targets inside the ranges
    a, b = cs.initial(N, DEV), cs.initial(N, DEV)
    cs.update(a, t32(qpos), t32(qvel), all_fresh=True, seed=3, step=1); cs.update(b, t32(qpos), t32(qvel), all_fresh=True, seed=3, step=1)
    assert torch.equal(a, b) and (a[:, 7].abs() <= 2.5).all() and (a[:, 10].abs() <= 1.0).all() and a[:, 7].std() > 0.1
    with pytest.raises(Exception, match="uniform"):
        cs.update(a, t32(qpos), t32(qvel), uniform=t32(u[:, :2]))


def test_start_pose_and_base_height_commands():
    """StartPositionCommand / StartQuaternionCommand hold the pose an episode started from; BaseHeightCommand redraws its height
    at a start and, with one draw deciding both, when that draw falls under switch_prob."""
    from ksim_amd import _lib_terms as T
    from ksim_amd.commands import BaseHeightCommand, CommandSet, StartPositionCommand, StartQuaternionCommand

    N, steps = 37, 10
    rng = np.random.default_rng(43)
    hp = dict(min_height=0.6, max_height=1.1, switch_prob=0.3)
    cs = CommandSet({"pos": StartPositionCommand(), "height": BaseHeightCommand(**hp), "quat": StartQuaternionCommand()})
    assert cs.command_dim == 8 and cs.slices["quat"] == slice(4, 8)
    cmd = cs.initial(N, DEV)
    want = np.zeros((N, 8))
    switched = 0
    for k in range(steps):
        qpos = rng.normal(size=(N, 27)).astype(np.float32)
        qvel = rng.normal(size=(N, 26)).astype(np.float32)
        u = rng.random((N, 3, T.KS_COMMAND_DRAWS)).astype(np.float32)
        fresh = np.ones(N, bool) if k == 0 else rng.random(N) < 0.15
        rec = torch.empty(N, 8, device=DEV)
        cs.update(cmd, t32(qpos), t32(qvel), fresh=torch.from_numpy(fresh.astype(np.uint8)).to(DEV), record=rec, uniform=t32(u))
        np.testing.assert_allclose(rec.cpu().numpy(), want, rtol=1e-6, atol=1e-7)
        for e in range(N):
            want[e, :3] = ot.start_pose_command(want[e, :3], qpos[e], bool(fresh[e]))
            new = ot.base_height_command(want[e, 3], float(u[e, 1, 0]), bool(fresh[e]), **hp)
            switched += (not fresh[e]) and new != want[e, 3]
            want[e, 3] = new
            want[e, 4:] = ot.start_pose_command(want[e, 4:], qpos[e], bool(fresh[e]), quaternion=True)
        np.testing.assert_allclose(cmd.cpu().numpy(), want, rtol=1e-6, atol=1e-6)
    assert switched > 20
    # a switched height comes from a draw below switch_prob, so it sits in the lowest part of the range
    assert (want[:, 3] >= 0.6).all() and (want[:, 3] <= 1.1).all()
    with pytest.raises(Exception, match="floating base"):
        cs.update(cmd, t32(qpos[:, :5]), t32(qvel), all_fresh=True, seed=1, step=1)


def test_sinusoidal_gait_command_and_reward():
    from ksim_amd import rewards as rw
    from ksim_amd.commands import CommandSet, ConstantCommand, SinusoidalGaitCommand
    from ksim_amd.types import Trajectory

    N, steps = 33, 14
    rng = np.random.default_rng(47)
    kw = dict(gait_period=0.37, ctrl_dt=0.02 * 3, max_height=0.15, height_offset=0.02, num_feet=3, stance_ratio=0.55, moving_threshold=0.3)
    cs = CommandSet({"pad": ConstantCommand(size=1), "gait": SinusoidalGaitCommand(**kw)})
    assert cs.command_dim == 6 and cs.slices["gait"] == slice(1, 6)
    cmd = cs.initial(N, DEV)
    want = np.zeros((N, 6))
    rec_all, pos_all = [], []
    for k in range(steps):
        qpos = rng.normal(size=(N, 12)).astype(np.float32)
        qvel = (rng.normal(size=(N, 11)) * 0.5).astype(np.float32)
        fresh = np.ones(N, bool) if k == 0 else rng.random(N) < 0.1
        rec = torch.empty(N, 6, device=DEV)
        cs.update(cmd, t32(qpos), t32(qvel), fresh=torch.from_numpy(fresh.astype(np.uint8)).to(DEV), record=rec, seed=1, step=k)
        np.testing.assert_allclose(rec.cpu().numpy(), want, rtol=1e-5, atol=1e-6)
        for e in range(N):
            want[e, 1:] = ot.sinusoidal_gait_command(want[e, 1:], qvel[e].astype(np.float64), bool(fresh[e]), **kw)
        np.testing.assert_allclose(cmd.cpu().numpy(), want, rtol=1e-5, atol=2e-6)
        rec_all.append(want.copy()); pos_all.append(rng.normal(size=(N, 9)) * 0.1)
    assert (want[:, 1] == 0).any() and (want[:, 1] == 1).any() and (want[:, 3:] > 0.05).any()
    commands, pos = np.stack(rec_all), np.stack(pos_all)
    traj = Trajectory(qpos=None, qvel=None, xpos=None, xquat=None, ctrl=None, obs={"obs": t32(pos)}, command={"_buffer": t32(commands)},
                      event_state={}, action=None, done=torch.zeros(steps, N, dtype=torch.bool, device=DEV), success=None, timestep=None)
    st = rw.get_rewards(traj, {"gait": rw.SinusoidalGaitReward(scale=0.6, max_height=0.15, pos_obs="feet", pos_cmd="gait", num_feet=3)},
                        obs_slices={"feet": slice(0, 9)}, command_slices=cs.slices)
    f32 = lambda a: a.astype(np.float32).astype(np.float64)  # noqa: E731
    want_r = 0.6 * ot.sinusoidal_gait_reward(f32(pos).reshape(steps, N, 3, 3), f32(commands)[..., 3:6], 0.15)
    np.testing.assert_allclose(st.total.cpu().numpy(), want_r, rtol=2e-5, atol=2e-5)
    with pytest.raises(ValueError, match="not found"):
        rw.get_rewards(traj, {"gait": rw.SinusoidalGaitReward(pos_obs="feet", pos_cmd="nope")}, obs_slices={"feet": slice(0, 9)}, command_slices=cs.slices)


def test_joint_position_and_cartesian_commands():
    """JointPositionCommand (with JointPositionReward reading its value) and CartesianCoordinateCommand against the oracle on
    the same draws, episode starts mixed in."""
    from ksim_amd import _lib_terms as T
    from ksim_amd.commands import CartesianCoordinateCommand, CommandSet, JointPositionCommand

    N, steps = 41, 40
    rng = np.random.default_rng(59)
    jp = dict(indices=(3, 0, 11), ranges=((-0.5, 0.7), (0.1, 0.2), (-1.0, -0.2)), ctrl_dt=0.02, min_time=0.05, max_time=0.3)
    cc = dict(box_min=(-0.3, 0.1, 0.5), box_max=(0.4, 0.6, 1.2), dt=0.02, min_speed=0.8, max_speed=4.0, switch_prob=0.7, jump_prob=0.05, curriculum_scale=0.25)
    cs = CommandSet({"joints": JointPositionCommand(**jp), "hand": CartesianCoordinateCommand(**cc)})
    assert cs.command_dim == 9 + 7 and cs.slices["hand"] == slice(9, 16)
    cmd = cs.initial(N, DEV)
    want = np.zeros((N, 16))
    redrawn_j = redrawn_c = 0
    for k in range(steps):
        qpos = rng.normal(size=(N, 27)).astype(np.float32)
        qvel = rng.normal(size=(N, 26)).astype(np.float32)
        u = rng.random((N, 2, T.KS_COMMAND_DRAWS)).astype(np.float32)
        fresh = np.ones(N, bool) if k == 0 else rng.random(N) < 0.05
        rec = torch.empty(N, 16, device=DEV)
        cs.update(cmd, t32(qpos), t32(qvel), level=0.6, fresh=torch.from_numpy(fresh.astype(np.uint8)).to(DEV), record=rec, uniform=t32(u))
        np.testing.assert_allclose(rec.cpu().numpy(), want, rtol=1e-6, atol=1e-6)
        for e in range(N):
            new = ot.joint_position_command(want[e, :9], qpos[e], u[e, 0], bool(fresh[e]), **jp)
            redrawn_j += (not fresh[e]) and new[8] == 0
            want[e, :9] = new
            new = ot.cartesian_coordinate_command(want[e, 9:], u[e, 1].astype(np.float64), bool(fresh[e]), level=0.6, **cc)
            redrawn_c += (not fresh[e]) and not np.allclose(new[3:6], want[e, 12:15])
            want[e, 9:] = new
        got = cmd.cpu().numpy()
        np.testing.assert_allclose(got[:, :7], want[:, :7], rtol=1e-6, atol=1e-7)  # float32 on both sides, up to a fused multiply-add
        np.testing.assert_array_equal(got[:, 7:9], want[:, 7:9])                   # num_steps and step_id
        np.testing.assert_allclose(got[:, 9:], want[:, 9:], rtol=2e-5, atol=2e-6)
    assert redrawn_j > 50 and redrawn_c > 30
    with pytest.raises(Exception, match="outside qpos"):
        CommandSet({"j": JointPositionCommand(indices=(25,), ranges=((0.0, 1.0),))}).update(cs.initial(N, DEV)[:, :5].contiguous(), t32(qpos), t32(qvel), all_fresh=True)
    with pytest.raises(ValueError):
        JointPositionCommand(indices=(1, 2), ranges=((0.0, 1.0),))


def test_vector_commands():
    """FloatVectorCommand / IntVectorCommand: the properties the reference's own tests check (shape, bounds, a command
    that never switches stays what it was, reference tests/test_commands.py:64-96) and the draw arithmetic."""
    from ksim_amd import _lib_terms as T
    from ksim_amd.commands import CommandSet, FloatVectorCommand, IntVectorCommand

    N = 500
    cs = CommandSet({"f": FloatVectorCommand(ranges=((0.0, 2.0), (-1.0, 1.0))), "i": IntVectorCommand(ranges=((2, 5),), switch_prob=0.3, zero_prob=0.1)})
    assert cs.command_dim == 3
    q, v = torch.zeros(N, 7, device=DEV), torch.zeros(N, 6, device=DEV)
    cmd = cs.initial(N, DEV)
    cs.update(cmd, q, v, all_fresh=True, seed=1, step=0)
    first = cmd.clone()
    assert ((cmd[:, 0] >= 0) & (cmd[:, 0] <= 2) & (cmd[:, 1] >= -1) & (cmd[:, 1] <= 1)).all() and cmd[:, 0].std() > 0.3
    ints = cmd[:, 2]
    assert (ints == ints.round()).all() and set(ints.unique().tolist()) <= {0.0, 2.0, 3.0, 4.0, 5.0} and (ints == 5).any() and (ints == 2).any()
    for k in range(5):
        cs.update(cmd, q, v, seed=1, step=1 + k)
    assert torch.equal(cmd[:, :2], first[:, :2])          # switch_prob 0: unchanged
    assert (cmd[:, 2] != first[:, 2]).float().mean() > 0.3  # switch_prob 0.3 over five steps
    # explicit draws: u0 switch, u1 zero, u2.. values
    u = torch.zeros(N, 2, T.KS_COMMAND_DRAWS, device=DEV)
    u[:, 1, 0] = 0.2; u[:, 1, 1] = 0.5; u[:, 1, 2] = 0.999
    u[0, 1, 1] = 0.05  # env 0 draws the zero command
    cs.update(cmd, q, v, uniform=u)
    assert (cmd[1:, 2] == 5).all() and cmd[0, 2] == 0 and torch.equal(cmd[:, :2], first[:, :2])
    with pytest.raises(ValueError):
        FloatVectorCommand(ranges=())


def test_mixture_of_gaussians_head():
    """ks_sample_action_mixture against the oracle on the same draws: component (bit-exact), sample, log-density;
    deterministic mode; Philox reproducibility and component frequencies."""
    from ksim_amd.env_terms import sample_action_mixture

    rng = np.random.default_rng(33)
    N, nu, K = 300, 20, 5
    raw = rng.normal(size=(N, 3 * nu * K)) * 1.5
    raw[0, nu * K] = 60.0       # softplus in its linear range -> capped
    raw[1, nu * K + 1] = -50.0  # softplus underflows -> floor
    raw[2, 2 * nu * K: 2 * nu * K + K] = [30.0, -30.0, 0.0, 1.0, -5.0]  # one component takes (almost) all the weight
    bias = rng.normal(size=nu) * 0.2
    lo, hi = -np.ones(nu) * 0.9, np.ones(nu) * 1.2
    u, z = rng.random((N, nu)), rng.normal(size=(N, nu))
    # keep the draws away from the cumulative weights, where fp32 and float64 may pick neighbouring components
    kw = dict(min_std=0.01, max_std=1.0, var_scale=0.5)
    w_act, w_logp, w_comp = ot.mixture_head(raw, K, uniform=u, normal=z, mean_bias=bias, clip_lo=lo, clip_hi=hi, clip_max=2.0, **kw)
    logit = raw[:, 2 * nu * K:].reshape(N, nu, K)
    cum = np.cumsum(np.exp(logit - np.logaddexp.reduce(logit, -1, keepdims=True)), -1)
    safe = np.abs(cum - u[..., None]).min(-1) > 1e-5
    assert safe.mean() > 0.99
    out, logp, comp = sample_action_mixture(t32(raw), K, mean_bias=t32(bias), clip_lo=t32(lo), clip_hi=t32(hi), uniform=t32(u),
                                            noise=t32(z), clip_max=2.0, want_stats=True, **kw)
    assert np.array_equal(comp.cpu().numpy()[safe], w_comp[safe])
    np.testing.assert_allclose(out.cpu().numpy()[safe], w_act[safe], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(logp.cpu().numpy()[safe], w_logp[safe], rtol=2e-4, atol=2e-4)
    assert comp[2, 0].item() == 0
    det = sample_action_mixture(t32(raw), K, mean_bias=t32(bias), clip_lo=t32(lo), clip_hi=t32(hi), deterministic=True, **kw)
    w_det, _, _ = ot.mixture_head(raw, K, mean_bias=bias, clip_lo=lo, clip_hi=hi, deterministic=True, **kw)
    np.testing.assert_allclose(det.cpu().numpy(), w_det, rtol=1e-6, atol=1e-6)
    # in-kernel draws: reproducible per (seed, step); components follow the weights
    big = t32(np.tile(raw[5:6], (20000, 1)))
    a1 = sample_action_mixture(big, K, seed=3, step=7, want_stats=True, **kw)
    a2 = sample_action_mixture(big, K, seed=3, step=7, **kw)
    a3 = sample_action_mixture(big, K, seed=3, step=8, **kw)
    assert torch.equal(a1[0], a2) and not torch.equal(a2, a3)
    cb = a1[2].cpu().numpy()
    w5 = np.exp(logit[5] - np.logaddexp.reduce(logit[5], -1, keepdims=True))
    freq = np.stack([(cb == k).mean(0) for k in range(K)], -1)
    assert np.abs(freq - w5).max() < 0.015
    with pytest.raises(Exception, match="3 nu K"):
        sample_action_mixture(t32(raw), 7, **kw)
    with pytest.raises(Exception, match="components"):
        sample_action_mixture(t32(raw[:, :51]), 17, **kw)
    # the walking example's ten components (examples/walking.py:273-276)
    raw10 = rng.normal(size=(64, 3 * nu * 10))
    u10, z10 = rng.random((64, nu)), rng.normal(size=(64, nu))
    w10 = ot.mixture_head(raw10, 10, uniform=u10, normal=z10, **kw)
    g10 = sample_action_mixture(t32(raw10), 10, uniform=t32(u10), noise=t32(z10), want_stats=True, **kw)
    lg10 = raw10[:, 2 * nu * 10:].reshape(64, nu, 10)
    cum10 = np.cumsum(np.exp(lg10 - np.logaddexp.reduce(lg10, -1, keepdims=True)), -1)
    ok10 = np.abs(cum10 - u10[..., None]).min(-1) > 1e-5
    assert np.array_equal(g10[2].cpu().numpy()[ok10], w10[2][ok10])
    np.testing.assert_allclose(g10[1].cpu().numpy()[ok10], w10[1][ok10], rtol=2e-4, atol=2e-4)


def test_action_filters_against_oracle():
    """ks_action_filter through the reference-named wrappers, a few steps each, with episode starts in between."""
    from ksim_amd import actions as A

    rng = np.random.default_rng(71)
    N, nu, dt = 50, 20, 0.02
    fresh = rng.random((6, N)) < 0.2
    u8 = lambda a: torch.tensor(a, dtype=torch.uint8, device=DEV)  # noqa: E731
    xs = rng.normal(size=(6, N, nu))
    init = rng.normal(size=(N, nu)) * 0.1
    # low-pass
    p, w = A.LowPassFilterParams.initialize(N, nu), np.zeros((N, nu))
    for t in range(6):
        y, p = A.lowpass_one_pole(t32(xs[t]), dt, 3.0, p, fresh=u8(fresh[t]))
        w = ot.lowpass_one_pole(xs[t], np.where(fresh[t][:, None], 0.0, w), dt, 3.0)
        np.testing.assert_allclose(y.cpu().numpy(), w, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(p.y_last.cpu().numpy(), w, rtol=1e-5, atol=1e-6)
    ys, _ = A.lowpass_one_pole_scan(t32(xs), dt, 3.0, A.LowPassFilterParams.initialize(N, nu))
    w = np.zeros((N, nu))
    for t in range(6):
        w = ot.lowpass_one_pole(xs[t], w, dt, 3.0)
        np.testing.assert_allclose(ys[t].cpu().numpy(), w, rtol=1e-5, atol=1e-6)
    # acceleration clip, restarting from `init`
    p = A.ClipAccelerationParams.initialize_from(t32(init))
    wp, wv = init.copy(), np.zeros((N, nu))
    for t in range(6):
        p = A.clip_acceleration(t32(xs[t]), p, 40.0, dt, fresh=u8(fresh[t]), init=t32(init))
        wp, wv = np.where(fresh[t][:, None], init, wp), np.where(fresh[t][:, None], 0.0, wv)
        wp, wv = ot.clip_acceleration(xs[t], wp, wv, 40.0, dt)
        np.testing.assert_allclose(p.position.cpu().numpy(), wp, rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(p.velocity.cpu().numpy(), wv, rtol=1e-4, atol=1e-4)
    # integrators
    pv, wpv = A.IntegrateVelocityParams.initialize(N, nu), np.zeros((N, nu))
    pa, wpa, wva = A.IntegrateAccelerationParams.initialize(N, nu), np.zeros((N, nu)), np.zeros((N, nu))
    for t in range(6):
        pv = A.integrate_velocity(t32(xs[t]), pv, dt, fresh=u8(fresh[t]))
        wpv = ot.integrate_velocity(xs[t], np.where(fresh[t][:, None], 0.0, wpv), dt)
        np.testing.assert_allclose(pv.position.cpu().numpy(), wpv, rtol=1e-5, atol=1e-6)
        pa = A.integrate_acceleration(t32(xs[t] * 100), pa, dt, max_velocity=3.0, fresh=u8(fresh[t]))
        wpa, wva = ot.integrate_acceleration(xs[t] * 100, np.where(fresh[t][:, None], 0.0, wpa), np.where(fresh[t][:, None], 0.0, wva), dt, 3.0)
        np.testing.assert_allclose(pa.position.cpu().numpy(), wpa, rtol=1e-5, atol=1e-5)
        assert np.abs(pa.velocity.cpu().numpy()).max() <= 3.0 and (np.abs(wva) == 3.0).any()
    # ranges
    ranges = [(-1.0 - 0.1 * j, 0.5 + 0.05 * j) for j in range(nu)]
    lo, hi = np.array(ranges).T
    np.testing.assert_allclose(A.ClipPositions(ranges).clip(t32(xs[0] * 2)).cpu().numpy(), ot.clip_positions(xs[0] * 2, lo, hi), rtol=1e-6)
    tp = A.TanhPositions(ranges)
    np.testing.assert_allclose(tp.clip(t32(xs[0])).cpu().numpy(), ot.tanh_positions(xs[0], lo, hi), rtol=1e-5, atol=1e-6)
    zeros = t32(np.full((1, nu), 0.1))
    np.testing.assert_allclose(tp.clip(tp.get_bias(zeros)).cpu().numpy(), 0.1, rtol=1e-4, atol=1e-5)
    m = km.kbot_scale_model(joint_range=(-0.7, 0.9))
    assert A.ClipPositions.from_physics_model(m).num_joints == m.nu and A.ClipPositions.from_physics_model(m).max_ranges[0] == 0.9
    with pytest.raises(Exception, match="kind"):
        A._run(9, t32(xs[0]))


def test_sensor_observations_gyro_accelerometer_touch():
    """SensorObservation on a model read from MJCF: one physics step through the kernel, then the sensor elements of
    ks_observe against the oracle formulas on the step's own outputs; the gyro of a site with the base's orientation is
    the free joint's body-frame angular velocity the substep started from; touch is the foot body's normal contact force."""
    from ksim_amd import _lib_terms as T, observation as ob, physics
    from ksim_amd._lib_dyn import KS_ACT_TORQUE
    from ksim_amd.env_terms import EnvTerms
    from ksim_amd.mjcf import load_mjcf
    from dyn_common import random_states

    m = load_mjcf(os.path.join(GOLD, "mini_biped.mjcf"), integrator="implicitfast")
    dm = physics.DeviceModel(m)
    N = 64
    qpos, qvel = random_states(m, N, seed=93, vel_scale=0.8, joint_range=0.3)
    ctrl = np.random.default_rng(94).normal(size=(N, m.nu)) * 2
    z = lambda *s: torch.zeros(*s, device=DEV)  # noqa: E731
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=z(N, m.nv), time=z(N), last_ctrl=t32(ctrl), action=t32(ctrl),
               qacc=z(N, m.nv), xpos=z(N, m.nb * 3), xquat=z(N, m.nb * 4), cvel=z(N, m.nb * 6), cfrc_ext=z(N, m.nb * 6))
    physics.control_step(dm, buf, substeps=1, actuator_type=KS_ACT_TORQUE)
    observations = {n: ob.SensorObservation.create(physics_model=m, sensor_name=n)
                    for n in ("imu_gyro", "imu_acc", "left_foot_touch", "right_foot_touch")}
    terms = EnvTerms(m, observations, {}, [])
    assert terms.obs_dim == 3 + 3 + 1 + 1 and list(terms.obs_slices) == ["imu_gyro", "imu_acc", "left_foot_touch", "right_foot_touch"]
    src = {T.SRC_QPOS: buf["qpos"], T.SRC_QVEL: buf["qvel"], T.SRC_QACC: buf["qacc"], T.SRC_XQUAT: buf["xquat"],
           T.SRC_CVEL: buf["cvel"], T.SRC_CFRC_EXT: buf["cfrc_ext"]}
    obs = torch.empty(N, terms.obs_dim, device=DEV)
    terms.observe(src, N, obs=obs)
    got = obs.cpu().numpy()
    xq = buf["xquat"].cpu().numpy().reshape(N, m.nb, 4).astype(np.float64)
    cv = buf["cvel"].cpu().numpy().reshape(N, m.nb, 6).astype(np.float64)
    qa = buf["qacc"].cpu().numpy().astype(np.float64)
    cf = buf["cfrc_ext"].cpu().numpy().reshape(N, m.nb, 6)
    _, spos, squat = m.sites["imu_site"]
    np.testing.assert_allclose(got[:, 0:3], ot.site_gyro(xq[:, 1], cv[:, 1, :3], squat), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(got[:, 3:6], ot.site_accelerometer(qa[:, :6], xq[:, 1], cv[:, 1, :3], spos, squat, m.gravity),
                               rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(got[:, 6], cf[:, m.sites["left_foot"][0], 5], rtol=1e-6)
    np.testing.assert_allclose(got[:, 7], cf[:, m.sites["right_foot"][0], 5], rtol=1e-6)
    assert (got[:, 6:] >= 0).all() and (got[:, 6:] > 1.0).sum() > N // 4  # feet in the ground in many envs
    # the angular velocity the forward pass of this (single) substep saw is the state's own, in body axes
    np.testing.assert_allclose(ot.site_gyro(xq[:, 1], cv[:, 1, :3], [1, 0, 0, 0]), qvel[:, 3:6], rtol=1e-4, atol=1e-4)
    # a body at rest on the ground would read +9.81 along the world's up axis: here check the size in free fall instead
    air = (cf[:, :, 5].sum(1) == 0)
    if air.any():  # no contact: the base origin accelerates with gravity plus what the joints do; the reading stays moderate
        assert np.isfinite(got[air, 3:6]).all()

    # frame sensors: the foot site's position and its body's angular velocity in world axes, the IMU site's orientation,
    # and the model's magnetic field seen from the IMU site
    frame = {n: ob.SensorObservation.create(physics_model=m, sensor_name=n) for n in ("left_foot_pos", "left_foot_angvel", "imu_quat", "imu_mag")}
    terms_f = EnvTerms(m, frame, {}, [])
    assert terms_f.obs_dim == 3 + 3 + 4 + 3
    src_f = dict(src); src_f[T.SRC_XPOS] = buf["xpos"]
    of = torch.empty(N, terms_f.obs_dim, device=DEV)
    terms_f.observe(src_f, N, obs=of)
    gf = of.cpu().numpy()
    xp = buf["xpos"].cpu().numpy().reshape(N, m.nb, 3).astype(np.float64)
    fb, fpos, _ = m.sites["left_foot"]
    np.testing.assert_allclose(gf[:, 0:3], ot.site_frame_position(xp[:, fb], xq[:, fb], fpos), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gf[:, 3:6], cv[:, fb, :3], rtol=1e-6)
    np.testing.assert_allclose(gf[:, 6:10], ot.site_frame_quaternion(xq[:, 1], squat), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gf[:, 10:13], ot.site_magnetometer(xq[:, 1], squat, m.magnetic), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(np.linalg.norm(gf[:, 10:13], axis=1), np.linalg.norm(m.magnetic), rtol=1e-5)
    with pytest.raises(Exception, match="xpos"):
        terms_f.observe(src, N, obs=of)

    # IMUAlignmentRandomizer: every env has its own site pose; the sensors and the site's 6-D rotation follow it
    from ksim_amd import randomization as rnd

    zn = np.random.default_rng(95).normal(size=(N, 6))
    r = rnd.IMUAlignmentRandomizer(site_name="imu_site", tilt_std_rad=0.05, yaw_std_rad=0.1, translate_std_m=0.01)
    gen = torch.Generator(device=DEV); gen.manual_seed(1)
    pose = r(m, N, gen, normal=t32(zn))["site_pose"]
    want_pose = np.array([np.concatenate([ot.quat_mul(ot.imu_alignment_offset(0.05 * zn[e, 0], 0.05 * zn[e, 1], 0.1 * zn[e, 2]), np.array(squat)),
                                          np.array(spos) + 0.01 * zn[e, 3:6]]) for e in range(N)])
    np.testing.assert_allclose(pose.cpu().numpy(), want_pose, rtol=1e-6, atol=1e-7)
    drawn = r(m, N, gen)["site_pose"].cpu().numpy()  # the generator's own draws: unit quaternions, tilts of the right size
    np.testing.assert_allclose(np.linalg.norm(drawn[:, :4], axis=1), 1.0, atol=1e-6)
    assert 0.5 * 0.05 < 2 * np.abs(drawn[:, 1]).std() < 2 * 0.05
    obs2 = {"gyro": ob.SensorObservation(sensor_name="imu_gyro", site_pose_per_env=True),
            "acc": ob.SensorObservation(sensor_name="imu_acc", site_pose_per_env=True),
            "rot": ob.SiteOrientationObservation.create(physics_model=m, site_names=("imu_site", "left_foot")),
            "rot_env": ob.SiteOrientationObservation(site_names=("imu_site",), site_pose_per_env=True),
            "contact": ob.ContactObservation(geom_idxs=(0, ob.FLOOR_GEOM, m.ns - 1)),
            "no_floor": ob.ContactObservation(geom_idxs=(0, 1))}
    terms2 = EnvTerms(m, obs2, {}, [])
    dist = np.random.default_rng(96).normal(size=(N, m.ns)) * 0.02
    src[T.SRC_CONTACT_DIST] = t32(dist)
    o2 = torch.empty(N, terms2.obs_dim, device=DEV)
    with pytest.raises(Exception, match="site pose"):
        terms2.observe(src, N, obs=o2)
    terms2.observe(src, N, obs=o2, site_pose=pose)
    g2, sl = o2.cpu().numpy(), terms2.obs_slices
    lf_body, _, lf_quat = m.sites["left_foot"]
    for e in range(N):
        np.testing.assert_allclose(g2[e, sl["gyro"]], ot.site_gyro(xq[e, 1], cv[e, 1, :3], want_pose[e, :4]), rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(g2[e, sl["acc"]], ot.site_accelerometer(qa[e, :6], xq[e, 1], cv[e, 1, :3], want_pose[e, 4:], want_pose[e, :4], m.gravity),
                                   rtol=1e-4, atol=1e-3)
        np.testing.assert_allclose(g2[e, sl["rot"]], np.concatenate([ot.site_rotation6d(xq[e, 1], squat), ot.site_rotation6d(xq[e, lf_body], lf_quat)]),
                                   rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(g2[e, sl["rot_env"]], ot.site_rotation6d(xq[e, 1], want_pose[e, :4]), rtol=1e-5, atol=1e-5)
        assert np.array_equal(g2[e, sl["contact"]].astype(bool), ot.contact_observation(dist[e], (0, -1, m.ns - 1)))
        assert not g2[e, sl["no_floor"]].any()
    assert np.abs(g2[:, sl["gyro"]] - got[:, 0:3]).max() > 1e-3, "the mounting error changes nothing in this test"
