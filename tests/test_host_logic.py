"""Host-side logic that needs no GPU: config validation, table compilation, struct layouts, model builder."""
import ctypes
import os

import numpy as np
import pytest

from ksim_amd import _lib, _lib_dyn, _lib_terms as T
from ksim_amd import actuators, engine, model as km, noise, observation as ob, resets as rs, rewards as rw
from ksim_amd import terminations as tm
from ksim_amd.env_terms import compile_terms


def test_struct_layouts_match_the_library():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    lib.ks_abi_sizeof.restype = ctypes.c_int64
    lib.ks_abi_sizeof.argtypes = [ctypes.c_int32]
    structs = [_lib.KsPpoLossParams, _lib_dyn.KsModelDesc, _lib_dyn.KsStepIO, T.KsTermsDesc, T.KsObserveIO,
               T.KsTerminateIO, T.KsMlpDesc, T.KsRewardIO, T.KsObsElem, T.KsTermDesc, T.KsRewardDesc, T.KsRng,
               T.KsAdamParams, T.KsEventDesc, T.KsRewardScanIO, T.KsRewardScanDesc, T.KsGruDesc, T.KsLstmDesc, T.KsGaussianHead, T.KsCommandIO, T.KsMixtureHead,
               T.KsNoiseStage, T.KsRandomVar]
    for i, st in enumerate(structs):
        assert lib.ks_abi_sizeof(i) == ctypes.sizeof(st), st.__name__
    assert lib.ks_abi_sizeof(99) == -1


def test_engine_config_validation_matches_reference_rules():
    with pytest.raises(ValueError, match="`dt` is required"):
        engine.EngineConfig(ctrl_dt=0.02)
    with pytest.raises(ValueError, match="`ctrl_dt` is required"):
        engine.EngineConfig(dt=0.005)
    with pytest.raises(ValueError, match="non-negative"):
        engine.EngineConfig(dt=0.005, ctrl_dt=0.02, action_latency_range=(-0.1, 0.0))
    with pytest.raises(ValueError, match="less than or equal"):
        engine.EngineConfig(dt=0.005, ctrl_dt=0.02, action_latency_range=(0.02, 0.01))
    with pytest.raises(ValueError, match="drop_action_prob"):
        engine.EngineConfig(dt=0.005, ctrl_dt=0.02, drop_action_prob=1.0)
    cfg = engine.EngineConfig(dt=0.004, ctrl_dt=0.02, action_latency_range=(0.0, 0.008), actuator_update_dt=0.008)
    data = engine.EngineData.from_config(cfg)
    assert data.phys_steps_per_ctrl_steps == 5 and data.phys_steps_per_actuator_step == 2
    assert data.max_action_latency_step == pytest.approx(2.0) and data.min_action_latency_step == 0.0
    assert engine.EngineConfig(dt=0.005, ctrl_dt=0.02).phys_steps_per_actuator_step == 1
    with pytest.raises(ValueError, match="Unsupported physics model type"):
        engine.get_physics_engine("mjx", [], {}, actuators.TorqueActuators(), cfg)
    eng = engine.get_physics_engine("hip", [], {}, actuators.TorqueActuators(), cfg)
    hash(eng)  # engines must stay hashable (reference tests/test_resets.py:82-84 checks the same of resets)
    with pytest.raises(NotImplementedError):
        engine.HipEngine(actuators.TorqueActuators(), [], {"push": object()}, data)


def test_actuator_and_term_validation():
    with pytest.raises(ValueError, match="negative"):
        actuators.PositionActuators(kps=(1.0, -1.0), kds=(1.0, 1.0))
    with pytest.raises(ValueError):
        actuators.PositionActuators(kps=(1.0,), kds=(1.0, 1.0))
    with pytest.raises(ValueError):
        actuators.PositionActuators(kps=(1.0,), kds=(1.0,), ctrl_clip=(-5.0,))
    assert np.isinf(actuators.PositionActuators(kps=(1.0, 2.0), kds=(0.1, 0.1)).clip_array()).all()
    with pytest.raises(ValueError):
        tm.MinimumHeightTermination(0.0)
    with pytest.raises(ValueError):
        tm.NotUprightTermination(-1.0)
    assert tm.MinimumHeightTermination(0.5).termination_name == "minimum_height_termination"
    assert tm.FarFromOriginTermination(3.0).desc()[1] == 1 and tm.FarFromOriginTermination(3.0, False).desc()[1] == -1
    assert rw.ActionVelocityPenalty().is_penalty and not rw.StayAliveReward().is_penalty
    with pytest.raises(ValueError, match="Invalid norm"):
        rw.ActionJerkPenalty(norm="l3").descs()

    class Odd(rw.Reward):
        pass

    with pytest.raises(ValueError, match="does not end with"):
        Odd().is_penalty
    assert noise.convert_to_noise(0.01).kind == T.NOISE_ADD_GAUSSIAN and noise.convert_to_noise(None) is None
    with pytest.raises(ValueError):
        noise.convert_to_noise("x")


def test_term_tables_compile():
    m = km.humanoid_model()
    chain = noise.ChainedNoise([noise.AdditiveGaussianNoise(std=0.02), noise.MultiplicativeUniformNoise(mag=0.1)])
    observations = {"jp": ob.JointPositionObservation(noise=0.01),
                    "jv": ob.JointVelocityObservation(noise=chain, bias=noise.MultiplicativeUniformBias(mag=0.05)),
                    "g": ob.ProjectedGravityObservation(), "w": ob.BaseAngularVelocityObservation(in_robot_frame=True),
                    "a": ob.LastActionObservation(), "c": ob.CommandObservation()}
    resets = [rs.RandomJointPositionReset(scale=0.1, scale_by_curriculum=False), rs.RandomHeightReset(range=(0.0, 0.1)),
              rs.RandomHeadingReset(), rs.RandomJointVelocityReset()]
    d, slices, used, bias, tab = compile_terms(m, observations, {"h": tm.MinimumHeightTermination(0.5)}, resets, 2)
    assert d.obs_dim == 71 and slices["g"] == slice(42, 45) and slices["c"] == slice(69, 71)  # benchmark config 3: 71
    assert d.obs[0].kind == T.OBS_JOINT_POS and d.obs[0].index == 7
    assert d.obs[0].n_noise == 1 and d.obs[0].noise[0].kind == T.NOISE_ADD_GAUSSIAN and d.obs[0].bias.kind == T.NOISE_NONE
    jv = d.obs[slices["jv"].start]
    assert jv.n_noise == 2 and jv.noise[1].kind == T.NOISE_MUL_UNIFORM and jv.noise[1].mean == 1.0
    assert jv.bias.kind == T.NOISE_MUL_UNIFORM and jv.bias.scale == pytest.approx(0.05) and bias is True
    assert noise.convert_to_bias(0.1).kind == T.NOISE_ADD_GAUSSIAN and noise.convert_to_bias(None) is None
    zo = engine.EngineConfig(dt=0.005, ctrl_dt=0.02, zero_offset_std=0.01, zero_offset_mag=0.02).zero_offset_random_variable()
    assert zo.same_key and zo.std == 0.01 and zo.mag == 0.02  # one key draws both parts (engine.py:117-124)
    assert not engine.EngineConfig(dt=0.005, ctrl_dt=0.02, zero_offset_std=0.01).zero_offset_random_variable().same_key
    assert d.obs[42].kind == T.OBS_ROT_INV and d.obs[44].comp == 2 and d.obs[44].c2 == pytest.approx(-9.81)
    assert T.SRC_CVEL not in used and T.SRC_QPOS in used
    assert d.n_terms == 1 and d.terms[0].kind == T.TERM_MIN_HEIGHT and d.terms[0].value == -1
    assert d.random_heading == 1 and d.reset_by_level[7] == 0 and d.reset_mag[7] == pytest.approx(0.1)
    assert d.reset_base[2] == pytest.approx(m.qpos0[2] + 0.05) and d.reset_mag[2] == pytest.approx(0.05)
    assert d.reset_mag[0] == 0.0 and d.nonfinite_terminates == 1


def test_model_builder_rules_and_constants():
    mb = km.ModelBuilder()
    a = mb.add_body(0, (0, 0, 1), joint="free", mass=1.0, inertia=(0.1, 0.1, 0.1))
    b = mb.add_body(a, (0, 0, -0.2), mass=0.5, inertia=(0.01, 0.01, 0.01))
    c = mb.add_body(b, (0, 0, -0.2), mass=0.5, inertia=(0.01, 0.01, 0.01))
    mb.add_body(a, (0, 0.1, 0), mass=0.5, inertia=(0.01, 0.01, 0.01))  # back up to an ancestor: still depth-first
    with pytest.raises(ValueError, match="depth-first"):
        mb.add_body(c, (0, 0, -0.2), mass=0.5, inertia=(0.01, 0.01, 0.01))  # c's subtree was already closed
    with pytest.raises(ValueError, match="attach to the world"):
        mb.add_body(a, (0, 0, 0), joint="free", mass=1.0, inertia=(1, 1, 1))
    with pytest.raises(ValueError, match="hinge"):
        mb.add_actuator(a)
    m = mb.build()
    assert (m.nq, m.nv, m.nb) == (10, 9, 5)
    assert list(m.dof_parent) == [-1, 0, 1, 2, 3, 4, 5, 6, 5] and list(m.body_subtree_end) == [5, 5, 4, 4, 5]
    M = km.host_mass_matrix(m.arrays(), m.qpos0)
    assert m.meaninertia == pytest.approx(np.trace(M) / m.nv)
    assert m.body_invweight0[1, 0] > 0 and m.body_invweight0[0, 0] == 0
    desc = _lib_dyn.model_desc(m)
    assert desc.nb == 5 and desc.body_parent[3] == 2 and desc.act_lo[0] == 0.0
    h = km.humanoid_model()
    assert h.max_depth == 6 and km.humanoid_model(seed=1).body_mass[3] != h.body_mass[3]
    assert np.allclose(km.capsule_inertia(1.0, 1e-9, 1.0)[:2], 1.0 / 12.0, rtol=1e-6)  # thin rod limit


def test_scales_and_event_descriptors():
    """Curriculum scales (ksim/scales.py) and the event records the step kernel reads (ksim/events.py)."""
    from ksim_amd import _lib_terms as T, events as kev, scales as sc

    assert sc.convert_to_scale(2).get_scale(0.3) == 2.0
    assert sc.LinearScale.from_endpoints(0.5, 1.5).get_scale(0.5) == pytest.approx(1.0)
    assert sc.QuadraticScale(scale=2.0, bias=1.0).get_scale(0.5) == pytest.approx(1.5)
    assert sc.SquareRootScale(scale=2.0).get_scale(0.25) == pytest.approx(1.0)
    nz = sc.NonZeroScale(scale=3.0, bias=0.5)
    assert (nz.get_scale(0.0), nz.get_scale(0.1)) == (0.5, 3.0)
    for bad in (lambda: sc.ConstantScale(scale=-1.0), lambda: sc.LinearScale(scale=-2.0, bias=1.0),
                lambda: sc.LinearScale(scale=1.0, bias=-0.1), lambda: sc.convert_to_scale("x")):
        with pytest.raises(ValueError):
            bad()
    d = kev.LinearPushEvent(linvel=2.0, vel_range=(0.1, 0.9), interval_range=(1.0, 3.0),
                            scale=sc.LinearScale(scale=1.0, bias=0.5)).desc(0.25)
    assert (d.kind, d.mag, d.lo, d.hi, d.interval_lo, d.interval_hi) == (T.EVENT_LINEAR_PUSH, 2.0, pytest.approx(0.1),
                                                                        pytest.approx(0.9), 1.0, 3.0)
    assert d.level_scale == pytest.approx(0.75)
    j = kev.JumpEvent(jump_height_range=(0.1, 0.2), interval_range=(2.0, 4.0)).desc(1.0)
    assert (j.kind, j.lo, j.hi, j.level_scale) == (T.EVENT_JUMP, pytest.approx(0.1), pytest.approx(0.2), 1.0)
    a = kev.AngularPushEvent(angvel=1.5, interval_range=(0.5, 1.0)).desc(1.0)
    assert (a.kind, a.mag, a.lo, a.hi) == (T.EVENT_ANGULAR_PUSH, 1.5, 0.0, 1.0)
    from ksim_amd import model as km
    mdl = km.kbot_scale_model()
    name = mdl.body_names[3]
    fp = kev.ForcePushEvent.from_body_name(mdl, name, max_force=50.0, max_torque=5.0, duration_range=(0.1, 0.3),
                                           interval_range=(1.0, 2.0), scale=0.5)
    fd = fp.desc(1.0)
    assert (fd.kind, fd.mag, fd.mag2, fd.body, fd.level_scale) == (T.EVENT_FORCE_PUSH, 50.0, 5.0, 3, 0.5)
    assert (fd.lo, fd.hi, fd.duration_lo, fd.duration_hi) == (0.0, 1.0, pytest.approx(0.1), pytest.approx(0.3))
    with pytest.raises(ValueError, match="not found"):
        kev.ForcePushEvent.from_body_name(mdl, "no such body", max_force=1.0, max_torque=1.0, duration_range=(0.1, 0.2),
                                          interval_range=(1.0, 2.0))
    # the engine refuses events that are not compiled into the step kernel, and more than the kernel holds
    from ksim_amd import actuators, engine
    act = actuators.TorqueActuators()
    cfg = engine.EngineConfig(dt=0.005, ctrl_dt=0.02)
    with pytest.raises(NotImplementedError):
        engine.get_physics_engine("hip", [], {"x": object()}, act, cfg)
    many = {f"e{i}": kev.JumpEvent(interval_range=(1.0, 2.0)) for i in range(T.KS_MAX_EVENTS + 1)}
    with pytest.raises(ValueError):
        engine.get_physics_engine("hip", [], many, act, cfg)


def test_stateful_terms_compile_to_carry_layouts():
    """Stateful observations get consecutive slices of the carry row in dict order; stateful rewards validate the
    observations they name (no GPU involved)."""
    m = km.kbot_scale_model()
    observations = {"jp": ob.JointPositionObservation(),
                    "old": ob.DelayedJointPositionObservation(delay_steps=3),
                    "g": ob.ProjectedGravityObservation(min_lag=0.1, max_lag=0.5),
                    "oldv": ob.DelayedJointVelocityObservation(delay_steps=2),
                    "plain_g": ob.ProjectedGravityObservation(),
                    "contact": ob.FeetContactObservation(foot_left=(0, 1), foot_right=(4, 5))}
    d, slices, used, _, _ = compile_terms(m, observations, {}, [])
    nj = m.nu
    assert d.carry_dim == 3 * nj + 7 + 2 * nj and d.ns == m.ns
    old, g, oldv = d.obs[slices["old"].start], d.obs[slices["g"].start + 2], d.obs[slices["oldv"].start + 1]
    assert (old.kind, old.comp, old.carry, old.stride, old.index) == (T.OBS_DELAYED, 3, 0, nj, 7)
    assert (g.kind, g.comp, g.carry) == (T.OBS_GRAVITY_EMA, 2, 3 * nj) and (g.q0, g.q1) == (pytest.approx(0.1), 0.5)
    assert (oldv.carry, oldv.stride, oldv.src, oldv.index) == (3 * nj + 7 + 1, nj, T.SRC_QVEL, 7)
    assert d.obs[slices["plain_g"].start].kind == T.OBS_ROT_INV
    c = [d.obs[k] for k in range(slices["contact"].start, slices["contact"].stop)]
    assert [e.index for e in c] == [0, 4, 1, 5] and all(e.kind == T.OBS_CONTACT and e.src == T.SRC_CONTACT_DIST for e in c)
    assert T.SRC_CONTACT_DIST in used and T.SRC_QPOS in used
    for bad in (lambda: ob.DelayedJointPositionObservation(delay_steps=0), lambda: ob.ProjectedGravityObservation(max_lag=1.0),
                lambda: ob.ProjectedGravityObservation(imu_bias=-0.1), lambda: ob.FeetContactObservation(foot_left=(0,), foot_right=())):
        with pytest.raises(ValueError):
            bad()
    fc = ob.FeetContactObservation.create(physics_model=m, foot_left_body_names=m.body_names[int(m.sph_body[0])],
                                          foot_right_body_names=[m.body_names[int(m.sph_body[-1])]])
    assert len(fc.foot_left) == len(fc.foot_right) == 4 and set(fc.foot_left).isdisjoint(fc.foot_right)
    from ksim_amd.scales import LinearScale
    air = rw.FeetAirTimeReward(scale=1.0, gait_period=LinearScale(scale=0.2, bias=0.3), air_time_percent=0.25, ctrl_dt=0.02,
                               contact_obs="contact")
    sd = air.scan_desc(slices, {}, 1.0)
    assert (sd.kind, sd.n, sd.n_contact, sd.contact_index) == (T.SCAN_FEET_AIR_TIME, 2, 2, slices["contact"].start)
    assert (sd.air_steps, sd.gnd_steps, sd.linvel_cmd_index) == (6.0, 19.0, -1)  # round(0.5*0.25/0.02), round(0.5*0.75/0.02)
    assert rw.reward_carry_size({"a": air, "b": rw.StayAliveReward(), "c": rw.SparseTargetHeightReward(contact_obs="contact")}) == 8
    with pytest.raises(KeyError):
        rw.FeetAirTimeReward(contact_obs="nope").scan_desc(slices, {}, 1.0)
    with pytest.raises(KeyError):
        rw.FeetAirTimeReward(contact_obs="contact", linvel_cmd="v").scan_desc(slices, {}, 1.0)
    with pytest.raises(ValueError):
        rw.SparseTargetHeightReward(contact_obs="contact", position_obs="jp", num_bodies=2).scan_desc(slices, {}, 1.0)


def test_feet_force_observations_read_the_contact_force_rows():
    m = km.kbot_scale_model()
    d, slices, used, _, _ = compile_terms(m, {"f": ob.FeetForceObservation(foot_left=11, foot_right=6),
                                              "t": ob.FeetTorqueObservation(foot_left=11, foot_right=6)}, {}, [])
    idx = [d.obs[k].index for k in range(d.obs_dim)]
    assert idx == [66, 67, 68, 36, 37, 38, 69, 70, 71, 39, 40, 41] and used == {T.SRC_CFRC_EXT}
    assert all(d.obs[k].kind == T.OBS_COPY and d.obs[k].src == T.SRC_CFRC_EXT for k in range(d.obs_dim))


def test_joint_randomizers_leave_the_floating_base_alone():
    import torch
    from ksim_amd import randomization as rnd

    m = km.kbot_scale_model()
    gen = torch.Generator().manual_seed(0)
    out = rnd.get_physics_randomizers(m, {"a": rnd.ArmatureRandomizer(0.9, 1.1), "d": rnd.JointDampingRandomizer(0.5, 2.0),
                                          "m": rnd.MassMultiplicationRandomizer.from_body_name(m, m.body_names[2], 0.5, 0.6)}, 64, gen)
    a, d, ms = out["armature_scale"], out["damping_scale"], out["mass_scale"]
    assert tuple(a.shape) == (64, m.nv) and (a[:, :6] == 1).all() and (d[:, :6] == 1).all()
    assert ((a[:, 6:] >= 0.9) & (a[:, 6:] <= 1.1)).all() and ((d[:, 6:] >= 0.5) & (d[:, 6:] <= 2.0)).all() and d[:, 6:].std() > 0.2
    assert (ms[:, [0, 1, 3]] == 1).all() and ((ms[:, 2] >= 0.5) & (ms[:, 2] <= 0.6)).all()
    add = rnd.MassAdditionRandomizer(body_id=1, scale_lower=1.0, scale_upper=1.0)(m, 4, gen)["mass_scale"]
    assert torch.allclose(add[:, 1], torch.full((4,), (float(m.body_mass[1]) + 1.0) / float(m.body_mass[1])))
    with pytest.raises(ValueError, match="duplicate"):
        rnd.get_physics_randomizers(m, {"a": rnd.MassMultiplicationRandomizer(body_id=1), "b": rnd.AllBodiesMassMultiplicationRandomizer()}, 4, gen)
    with pytest.raises(ValueError, match="not found"):
        rnd.MassMultiplicationRandomizer.from_body_name(m, "nope")


def test_position_velocity_actuator_widths():
    act = actuators.PositionVelocityActuator(kps=(10.0, 20.0), kds=(1.0, 2.0))
    assert act.action_dim(2) == 4 and actuators.PositionActuators(kps=(1.0,), kds=(1.0,)).action_dim(1) == 1
    m = km.kbot_scale_model()
    d, slices, _, _, _ = compile_terms(m, {"a": ob.LastActionObservation(action_dim=2 * m.nu)}, {}, [], action_dim=2 * m.nu)
    assert d.action_dim == 2 * m.nu and d.obs_dim == 2 * m.nu


def test_curricula_hand_computed():
    """ksim/curriculum.py's level updates on small hand-made rollouts (time-major (T, N) arrays)."""
    import torch
    from ksim_amd import curriculum as cu
    from ksim_amd.types import Trajectory

    def traj(done, timestep, qpos=None):
        return Trajectory(qpos=qpos, qvel=None, xpos=None, xquat=None, ctrl=None, obs={}, command={}, event_state={}, action=None,
                          done=torch.tensor(done, dtype=torch.uint8), success=None, timestep=torch.tensor(timestep, dtype=torch.float32))

    # episode_length: per env, mean timestep over episode ends, the last step always counted (types.py:72-76)
    t = traj([[0, 1], [0, 0], [0, 0]], [[0.1, 0.5], [0.2, 0.02], [0.3, 0.04]])
    assert t.episode_length().tolist() == pytest.approx([0.3, (0.5 + 0.04) / 2])
    c = cu.ConstantCurriculum(level=0.7)
    s = c.get_initial_state()
    assert c(t, None, 5, s).level == 0.7
    lin = cu.LinearCurriculum(step_size=0.1, step_every_n_epochs=2, min_level=0.05, delay_steps=3)
    assert lin.get_initial_state().level == 0.05
    assert [lin(t, None, n, None).level for n in (0, 3, 4, 5, 9, 40)] == pytest.approx([0.05, 0.05, 0.05, 0.1, 0.3, 1.0])
    # episode length: EMA 0.5 * prev + 0.5 * mean length; a level step when the counter is at zero, then a pause
    el = cu.EpisodeLengthCurriculum(num_levels=10, increase_threshold=0.2, decrease_threshold=0.1, min_level_steps=2, ema_decay=0.5)
    s = el.get_initial_state()
    assert s.level == 0.0 and s.state == (2, 0.0)
    mean_len = (0.3 + 0.27) / 2
    s = el(t, None, 0, s); assert s.state == (1, pytest.approx(0.5 * mean_len)) and s.level == 0.0          # counter 2 -> 1
    s = el(t, None, 1, s); assert s.state[0] == 0 and s.level == 0.0                                          # 1 -> 0
    s = el(t, None, 2, s)                                                                                      # may step: EMA 0.249 > 0.2
    assert s.level == pytest.approx(0.1) and s.state[0] == 2 and s.state[1] == pytest.approx(mean_len * (1 - 0.5**3))
    short = traj([[1, 1], [1, 1], [1, 1]], [[0.02, 0.02]] * 3)
    for _ in range(6):
        s = el(short, None, 3, s)
    assert s.level == pytest.approx(0.0) and s.state[1] < 0.1                                                 # back down, clipped at min_level
    # distance from origin
    q = torch.zeros(3, 2, 7); q[2, 1, :3] = torch.tensor([3.0, 4.0, 0.0])
    dc = cu.DistanceFromOriginCurriculum(num_levels=4, increase_threshold=2.0, decrease_threshold=1.0, min_level_steps=1, ema_decay=0.0)
    s = dc.get_initial_state()
    s = dc(traj([[0, 0]] * 3, [[0.0, 0.0]] * 3, q), None, 0, s)
    assert s.state[1] == pytest.approx(5.0) and s.level == 0.25 and s.state[0] == 1
    s = dc(traj([[0, 0]] * 3, [[0.0, 0.0]] * 3, q), None, 1, s)
    assert s.level == 0.5
    # deaths per env
    sw = cu.StepWhenSaturated(num_levels=5, increase_threshold=0.6, decrease_threshold=1.5, min_level_steps=1)
    s = sw.get_initial_state()
    s = sw(t, None, 0, s); assert s == cu.CurriculumState(0.0, 0)              # waits one call
    s = sw(t, None, 1, s); assert s.level == pytest.approx(0.2) and s.state == 1   # 0.5 deaths per env < 0.6
    s = sw(short, None, 2, s); assert s.level == pytest.approx(0.2)              # waits
    s = sw(short, None, 3, s); assert s.level == pytest.approx(0.0)              # 3 deaths per env > 1.5


def test_remaining_randomizers_produce_the_kernel_inputs():
    """Static friction, centre-of-mass, inertia and collision-capsule randomisers (ksim/randomization.py:56-71, 290-487):
    shapes, ranges, which entries move, and the capsule geometry (both ends share the radius factor, the length factor
    moves them symmetrically about the jittered centre)."""
    import os
    import torch
    from ksim_amd import randomization as rnd
    from ksim_amd.mjcf import load_mjcf

    m = load_mjcf(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mini_biped.mjcf"))
    gen = torch.Generator(); gen.manual_seed(0)
    N = 200
    r = rnd.get_physics_randomizers(m, {"sf": rnd.StaticFrictionRandomizer(0.5, 2.0), "com": rnd.AllBodiesCOMRandomizer(0.01),
                                        "inertia": rnd.AllBodiesInertiaRandomizer(0.02),
                                        "feet": rnd.CollisionBodyRandomizer.from_geom_names(m, ["foot_l", "foot_r"], radius_scale=0.1,
                                                                                            length_scale=0.2, position_jitter_x=0.003,
                                                                                            position_jitter_y=0.0, position_jitter_z=0.001)}, N, gen)
    fl = r["frictionloss"].numpy()
    assert fl.shape == (N, m.nv) and (fl[:, :6] == 0).all()
    ratio = fl[:, 6:] / m.dof_frictionloss[6:]
    assert ratio.min() >= 0.5 and ratio.max() <= 2.0 and ratio.std() > 0.3
    ip = r["body_ipos"].numpy().reshape(N, m.nb, 3) - m.body_ipos
    assert np.abs(ip).max() <= 0.01 + 1e-7 and np.abs(ip).mean() > 0.003
    s = r["mass_scale"].numpy()
    inert = r["body_inertia"].numpy().reshape(N, m.nb, 3) / np.where(m.body_inertia > 0, m.body_inertia, 1.0)
    assert np.abs(s - 1).max() <= 0.02 + 1e-6
    shape = inert[:, 1:] / s[:, 1:, None]
    assert np.abs(shape - 1).max() <= 0.02 + 1e-5 and shape.std() > 0.005
    pos, rad = r["sph_pos"].numpy().reshape(N, m.ns, 3), r["sph_radius"].numpy()
    i, j = [k for k, n in enumerate(m.sph_names) if n == "foot_l"]
    assert np.allclose(rad[:, i], rad[:, j]) and np.abs(rad[:, i] / 0.02 - 1).max() <= 0.1 + 1e-6
    centre, half = 0.5 * (pos[:, i] + pos[:, j]), 0.5 * (pos[:, j] - pos[:, i])
    c0, h0 = 0.5 * (m.sph_pos[i] + m.sph_pos[j]), 0.5 * (m.sph_pos[j] - m.sph_pos[i])
    jit = centre - c0
    assert np.abs(jit[:, 0]).max() <= 0.003 + 1e-6 and np.abs(jit[:, 1]).max() < 1e-6 and np.abs(jit[:, 2]).max() <= 0.001 + 1e-6
    scale = np.linalg.norm(half, axis=1) / np.linalg.norm(h0)
    assert np.abs(scale - 1).max() <= 0.2 + 1e-5 and scale.std() > 0.05
    assert np.allclose(np.cross(half, h0[None]), 0, atol=1e-7)  # the capsule keeps its axis
    com1 = rnd.COMRandomizer.from_body_name(m, "knee_l", scale=0.02)(m, N, gen)["body_ipos"].numpy().reshape(N, m.nb, 3) - m.body_ipos
    assert np.abs(com1[:, 3]).max() > 0.01 and np.abs(np.delete(com1, 3, axis=1)).max() < 1e-7
    with pytest.raises(ValueError, match="not a collision capsule"):
        rnd.CollisionBodyRandomizer.from_geom_names(m, ["nope"])


def test_reward_constructors_from_a_model():
    """`create` of the rewards that read the model (ksim/rewards.py:535-553, 571-581, 641-662, 684-700)."""
    import os
    from ksim_amd import rewards as rw
    from ksim_amd.mjcf import load_mjcf

    m = load_mjcf(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mini_humanoid.mjcf"))
    lim = rw.AvoidLimitsPenalty.create(m, factor=0.1)
    lo, hi = np.deg2rad(-30), np.deg2rad(20)
    assert len(lim.joint_limits) == m.nq - 7
    np.testing.assert_allclose(lim.joint_limits[0], (lo - 0.1 * (hi - lo), hi + 0.1 * (hi - lo)), rtol=1e-6)
    assert rw.TorquePenalty.create(m).ctrl_scales == (1.0,) * m.nu      # control range -1..1 on every motor
    assert isinstance(rw.EnergyPenalty.create(m), rw.EnergyPenalty) and rw.EnergyPenalty(ctrl_scales=(1.0,)).is_penalty
    dev = rw.JointDeviationPenalty.create(m, ["shin_right", "thigh_left"], (0.1, 0.2), joint_weights=(1.0, 3.0))
    assert dev.joint_indices == (3, 6) and dev.joint_weights == (1.0, 3.0)
    flat = rw.FlatBodyReward.create(m, ("pelvis", "shin_left"))
    assert flat.body_indices == (1, 9)
    tr = rw.PositionTrackingReward.create(m, "cmd", "shin_left", "pelvis")
    assert (tr.tracked_body_idx, tr.base_body_idx, tr.norm) == (9, 1, "l1")
    with pytest.raises(ValueError, match="must match"):
        rw.JointDeviationPenalty(joint_indices=(0, 1), joint_targets=(0.0,)).descs()


def test_benchmark_workload_label_follows_the_model_flag():
    """The bench line's integrator text is derived from the model it actually builds, for both legs."""
    import re

    from ksim_amd import model as km
    from ksim_amd.configs import integrator_name

    euler = km.kbot_scale_model(seed=1004, integrator="euler")
    fast = km.kbot_scale_model(seed=1004, integrator="implicitfast")
    assert not euler.eulerdamp and not euler.arrays()["eulerdamp"]
    assert fast.eulerdamp and fast.arrays()["eulerdamp"]
    assert integrator_name(euler) == "semi-implicit Euler"
    assert integrator_name(fast).startswith("implicitfast")
    src = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py")).read()
    # no hard-coded integrator in the workload text, and both legs take the same argument
    assert "integrator_name(m)" in src and not re.search(r'"[^"\n]*implicitfast \(damping', src)
    assert "cpu_baseline(args.integrator)" in src and "timed_rollout(torch, args.integrator, N, T, args.steps, args.warmup, args.streams)" in src
    src_cfg = open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "ksim_amd", "configs.py")).read()
    assert "kbot_scale_model(seed=seed, integrator=integrator)" in src_cfg


def test_model_create_rejects_joint_addresses_outside_the_state():
    """ks_model_create validates before it touches the GPU: a body whose qpos or dof address (plus the joint's width) leaves
    qpos / qvel is refused, so the kernel's tables are never indexed out of range."""
    import ctypes

    from ksim_amd import _lib, _lib_dyn
    from ksim_amd import model as km

    lib = _lib.load()
    m = km.kbot_scale_model()

    def create(edit):
        desc = _lib_dyn.model_desc(m)
        edit(desc)
        h = ctypes.c_void_p()
        rc = lib.ks_model_create(ctypes.byref(desc), ctypes.byref(h))
        return rc, lib.ks_last_error().decode()

    def set_field(name, b, v):
        def edit(desc):
            getattr(desc, name)[b] = v
        return edit

    for name, b, v in (("body_dofadr", 5, m.nv), ("body_dofadr", 5, -1), ("body_qadr", 7, m.nq), ("body_qadr", 7, -3),
                       ("body_dofadr", 1, m.nv - 5),   # the free joint needs six dofs
                       ("body_qadr", 1, m.nq - 6)):    # and seven coordinates
        rc, msg = create(set_field(name, b, v))
        assert rc == -1 and f"body {b}" in msg and "outside" in msg, (name, b, v, rc, msg)


def test_mjcf_contact_dimension_follows_mujocos_rule(tmp_path):
    """condim of a geom-floor contact is the larger of the two geoms' (an explicit pair carries its own); the model takes
    the one value all contacts share: 1 = frictionless as in the reference's examples/data/scene.mjcf, 3 = friction pyramid."""
    from ksim_amd.mjcf import load_mjcf

    def robot(floor, foot, pair=""):
        return f"""<mujoco><worldbody>
          <geom name="floor" type="plane" size="0 0 .05" condim="{floor}"/>
          <body name="base" pos="0 0 0.5"><freejoint/>
            <geom name="torso" type="sphere" size="0.1" mass="1" contype="0" conaffinity="0"/>
            <geom name="foot" type="sphere" size="0.05" pos="0 0 -0.2" mass="0.2" condim="{foot}"/>
          </body></worldbody>{pair}</mujoco>"""

    for floor, foot, pair, want in ((1, 1, "", 1), (1, 3, "", 3), (3, 1, "", 3), (3, 3, "", 3),
                                    (3, 3, '<contact><pair geom1="foot" geom2="floor" condim="1"/></contact>', 1)):
        path = tmp_path / f"r{floor}{foot}{len(pair)}.xml"
        path.write_text(robot(floor, foot, pair))
        m = load_mjcf(str(path))
        assert m.condim == want and m.ns == 1, (floor, foot, pair)
    path = tmp_path / "bad.xml"
    path.write_text(robot(4, 1))
    with pytest.raises(ValueError, match="condim"):
        load_mjcf(str(path))


def test_generic_noise_and_bias_over_random_variables():
    """AdditiveNoise / MultiplicativeNoise / AdditiveBias / MultiplicativeBias over a random variable (ksim/noise.py:129-193)
    are the named convenience classes' stages."""
    from ksim_amd import noise as kn

    same = lambda a, b: (a.kind, a.mean, a.scale, a.scale2) == (b.kind, b.mean, b.scale, b.scale2)  # noqa: E731
    assert same(kn.AdditiveNoise(kn.GaussianRandomVariable(0.1, 0.3)), kn.AdditiveGaussianNoise(std=0.3, mean=0.1))
    assert same(kn.MultiplicativeNoise(kn.UniformRandomVariable(1.0, 0.2)), kn.MultiplicativeUniformNoise(mag=0.2))
    assert same(kn.AdditiveNoise(kn.UniformGaussianRandomVariable(0.0, 0.3, 0.4)), kn.AdditiveUniformGaussianNoise(std=0.3, mag=0.4))
    assert same(kn.MultiplicativeBias(kn.GaussianRandomVariable(1.0, 0.05)), kn.MultiplicativeGaussianBias(std=0.05))
    assert same(kn.AdditiveBias(kn.UniformRandomVariable(0.0, 0.5)), kn.AdditiveUniformBias(mag=0.5))
    assert isinstance(kn.AdditiveBias(kn.ZeroRandomVariable()), kn.Bias) and kn.AdditiveNoise(kn.ZeroRandomVariable()).scale == 0.0
    with pytest.raises(ValueError, match="one key"):
        kn.AdditiveNoise(kn.RandomVariable(mean=0.0, mag=0.1, std=0.1, same_key=False))


def test_observation_kinds_declare_every_source_they_read():
    """The rollout refreshes a derived field of the live state only when an observation declares it: a site position reads
    xpos and the body quaternion that turns the site offset, the other frame sensors the quaternion."""
    from ksim_amd.env_terms import KIND_SOURCES
    from ksim_amd.mjcf import load_mjcf

    m = load_mjcf(os.path.join(os.path.dirname(__file__), "golden", "mini_biped.mjcf"))
    one = lambda name: compile_terms(m, {name: ob.SensorObservation.create(physics_model=m, sensor_name=name)}, {}, [])[2]  # noqa: E731
    assert {T.SRC_XPOS, T.SRC_XQUAT} <= one("left_foot_pos")
    assert T.SRC_XQUAT in one("imu_quat") and T.SRC_XQUAT in one("imu_mag")
    assert {T.SRC_XQUAT, T.SRC_CVEL} <= one("imu_gyro") and {T.SRC_XQUAT, T.SRC_CVEL, T.SRC_QACC} <= one("imu_acc")
    site_kinds = (T.OBS_SITE_GYRO, T.OBS_SITE_ACCEL, T.OBS_SITE_ROT6D, T.OBS_SITE_POS, T.OBS_SITE_QUAT, T.OBS_SITE_MAGNETOMETER)
    assert all(T.SRC_XQUAT in KIND_SOURCES[k] for k in site_kinds)


def test_reset_orders_the_table_cannot_express_raise():
    m = km.kbot_scale_model()
    field = rs.HFieldXYPositionReset(bounds=(5.0, 5.0, 0.0, 0.0), hfield_data=np.zeros((4, 4)))
    with pytest.raises(ValueError, match="RandomHeightReset"):
        rs.compile_resets([field, rs.RandomHeightReset(range=(0.0, 0.2))], m)
    tab = rs.compile_resets([rs.RandomHeightReset(range=(0.0, 0.2)), field], m)  # listed first: replaced, as in the reference
    assert tab["mag"][2] == 0.0 and tab["base"][2] == 0.0
    tab = rs.compile_resets([field, rs.RandomHeightReset(range=(0.3, 0.3))], m)  # a single height only shifts the base
    assert tab["base"][2] == pytest.approx(0.3)

    class Motion:
        qpos = np.tile(m.qpos0, (5, 1)).astype(np.float32)
        ctrl_dt = 0.02

    for first in (rs.RandomHeadingReset(), rs.RandomPitchRollReset()):
        with pytest.raises(ValueError, match="freejoint"):
            rs.compile_resets([first, rs.InitialMotionStateReset(reference_motion=Motion, freejoint=True)], m)
        rs.compile_resets([first, rs.InitialMotionStateReset(reference_motion=Motion, freejoint=False)], m)
        rs.compile_resets([rs.InitialMotionStateReset(reference_motion=Motion, freejoint=True), first], m)
    with pytest.raises(ValueError, match="31 spheres"):
        big = type("M", (), {"ns": 40})()
        ob.ContactObservation(geom_idxs=(ob.FLOOR_GEOM, 3)).elements(big, 0)


def test_committed_traffic_profiles_carry_sane_calibration_factors():
    """The HBM-traffic summaries scale FETCH_SIZE / WRITE_SIZE by what the same counter reads for a 256 MiB copy: that factor
    is about 2 for reads and 1 for writes on this part.  A factor far from that means the calibration dispatch was mixed
    up with other launches, and every figure of the file is wrong by the same ratio."""
    import glob
    import re

    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "..", "profiles", "*traffic*.txt")))
    assert files
    for path in files:
        text = open(path).read()
        factors = [float(x) for x in re.findall(r"(?:FETCH|WRITE) x ([0-9.]+?)[,\s]", text)]
        factors += [float(x) for x in re.findall(r"factor ([0-9.]+)", text)]
        assert factors, f"{os.path.basename(path)} states no calibration factor"
        for f in factors:
            assert 0.5 <= f <= 4.0, f"{os.path.basename(path)}: calibration factor {f}"
        for ratio in re.findall(r"^[^#\n]*\|[^\n]*$", text, flags=re.M):  # data rows: the traffic / algorithmic column
            cols = [c.strip() for c in ratio.split("|")]
            if len(cols) >= 9 and re.fullmatch(r"[0-9.]+", cols[5]):
                assert float(cols[5]) < 4.0, f"{os.path.basename(path)}: traffic / algorithmic {cols[5]} in {cols[0]}"


def test_every_public_oracle_function_is_named_in_a_cpu_test():
    """The oracle is only as good as its pins: every public function of `oracle/*.py` must be called by name in a test that
    runs without a GPU, or be listed here as plumbing (conversions between containers, no arithmetic of the reference)."""
    import ast
    import glob
    import re

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    plumbing = {
        "dyn.make_model": "copies a model dictionary into the C struct of the compiled oracle",
        "recurrent.torch_sequence": "recurrent_sequence on torch tensors; recurrent_sequence_gradients, which calls it, is held "
                                    "against the numpy network and central differences",
        "recurrent.torch_parameters": "wraps arrays as tensors that record gradients",
        "recurrent.parameter_gradients": "reads .grad back into the parameter structure",
        "ppo_update.update_model": "the minibatch loop around loss_and_grads and optax_chain_step, both pinned; compared with the "
                                   "kernel path in the GPU suite",
    }
    text = ""
    for f in glob.glob(os.path.join(root, "tests", "test_*.py")):
        src = open(f).read()
        if "pytestmark = pytest.mark.gpu" in src or os.path.basename(f).startswith("test_gpu") or os.path.basename(f).startswith("test_zz"):
            continue
        text += src
    missing = []
    for f in sorted(glob.glob(os.path.join(root, "oracle", "*.py"))):
        mod = os.path.basename(f)[:-3]
        if mod.startswith("_"):
            continue
        for node in ast.parse(open(f).read()).body:
            if isinstance(node, ast.FunctionDef) and not node.name.startswith("_"):
                if f"{mod}.{node.name}" not in plumbing and not re.search(r"\b" + re.escape(node.name) + r"\b", text):
                    missing.append(f"{mod}.{node.name}")
    assert not missing, f"oracle functions that no CPU test names: {missing}"
