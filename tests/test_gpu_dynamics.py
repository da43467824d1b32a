"""Parity of the fused HIP control-step kernel against the CPU oracle (through the C ABI).

Tolerances are the benchmark definition's: qacc and one-step state 1e-4 relative, 10-step trajectories 1e-3
(fp32 kernel against the float64 oracle; "relative" = max abs error of an env's vector over
that vector's max magnitude).
"""
import numpy as np
import pytest
import torch

from dyn_common import oracle_forward, random_states, rel_err
from ksim_amd import model as km
from oracle import terms as oterms
from oracle.dyn import Oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MODELS = {"chain": km.pendulum_chain_model, "humanoid": km.humanoid_model, "kbot": km.kbot_scale_model,
          # the integrator ksim selects: velocity update implicit in joint damping
          "chain-implicit": lambda: km.pendulum_chain_model(integrator="implicitfast", damping=0.5),
          "kbot-implicit": lambda: km.kbot_scale_model(integrator="implicitfast"),
          "humanoid-implicit": lambda: km.humanoid_model(integrator="implicitfast"),
          # joint limits and dry joint friction (rows carried by the dof lanes), alone and together with contacts.  The test
          # states draw hinge angles from U(-0.6, 0.6), so about a fifth of the joints start up to 0.15 rad beyond a limit
          # (much deeper violations make the cost so large that its fp32 rounding hides the last Newton improvements).
          "chain-friction": lambda: km.pendulum_chain_model(integrator="implicitfast", frictionloss=0.3),
          # joint springs about the reference angles (a passive force)
          "chain-springs": lambda: km.pendulum_chain_model(integrator="implicitfast", damping=0.2, stiffness=6.0),
          "humanoid-limits": lambda: km.humanoid_model(joint_range=(-0.45, 0.5)),
          "kbot-limits": lambda: km.kbot_scale_model(integrator="implicitfast", joint_range=(-0.45, 0.5), frictionloss=0.2),
          # frictionless contacts (condim 1, what the reference's examples/data/scene.mjcf uses): one normal row per contact
          "kbot-frictionless": lambda: km.kbot_scale_model(integrator="implicitfast", condim=1),
          "humanoid-frictionless-limits": lambda: km.humanoid_model(joint_range=(-0.45, 0.5), condim=1),
          # the real K-Bot's contact parameters (robot.mjcf:24): five times stiffer rows than MuJoCo's defaults
          "kbot-stiff-feet": lambda: km.kbot_scale_model(integrator="implicitfast", joint_range=(-0.45, 0.5), frictionloss=0.2,
                                                         solref=(0.02, 0.8), solimp=(0.98, 0.99, 0.1, 0.5, 2.0),
                                                         dof_solref=(0.02, 1.0), dof_solimp=(0.9, 0.95, 0.001, 0.5, 2.0))}
# fp32 against float64 on the stiff-feet model: the constraint stiffness D = d / ((1 - d) invweight) with d = 0.98..0.99 is
# five times the default one, and so is the amplification of rounding in H = M + J^T D J.  This is single precision's own
# floor on that model, not the kernel's: the float32 build of the C oracle, the same source as the float64 reference, is
# 2.5e-4 away from it on these very states (tests/test_oracle_dyn.py::test_single_precision_floor_on_the_stiff_contact_model)
STIFF_TOL = 5e-4
ONE_STEP_TOL, TEN_STEP_TOL = 1e-4, 1e-3


def t32(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32, device=DEV).contiguous()


def zeros(*shape, dtype=torch.float32):
    return torch.zeros(*shape, dtype=dtype, device=DEV)


@pytest.fixture(scope="module", params=list(MODELS))
def setup(request):
    from ksim_amd import physics

    m = MODELS[request.param]()
    return request.param, m, physics.DeviceModel(m)


def test_forward_quantities_match_oracle(setup):
    from ksim_amd import physics

    name, m, dm = setup
    N = 48
    qpos, qvel = random_states(m, N, seed=11)
    rng = np.random.default_rng(12)
    ctrl = rng.normal(size=(N, m.nu)) * 5
    fr = rng.uniform(0.4, 1.2, size=N)
    ms = rng.uniform(0.9, 1.1, size=(N, m.nb))
    warm = rng.normal(size=(N, m.nv))
    want = oracle_forward(m, qpos, qvel, ctrl, fr, ms, warm)
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=t32(warm), ctrl_in=t32(ctrl), friction=t32(fr),
               mass_scale=t32(ms), qacc=zeros(N, m.nv), xpos=zeros(N, m.nb * 3), xquat=zeros(N, m.nb * 4),
               cvel=zeros(N, m.nb * 6), nefc=zeros(N, dtype=torch.int32), solver_niter=zeros(N, dtype=torch.int32),
               dbg_M=zeros(N, m.nv * m.nv), dbg_bias=zeros(N, m.nv), dbg_qacc_smooth=zeros(N, m.nv),
               contact_dist=zeros(N, m.ns), cinert=zeros(N, m.nb * 10), cfrc_ext=torch.full((N, m.nb * 6), 7.0, device=DEV))
    q0 = buf["qpos"].clone()
    physics.forward(dm, buf)
    g = {k: v.cpu().numpy() for k, v in buf.items()}
    assert torch.equal(buf["qpos"], q0), "forward must not integrate"
    for got, ref, tol in [("dbg_M", "M", 1e-5), ("dbg_bias", "qfrc_bias", 1e-5), ("xpos", "xpos", 1e-5),
                          ("xquat", "xquat", 1e-5), ("cvel", "cvel", 1e-5), ("cinert", "cinert", 1e-5),
                          # contact forces are -D (J qacc - aref) with D ~ 1e3..1e4: they amplify the rounding of qacc
                                                    ("cfrc_ext", "cfrc_ext", 1e-2 if name == "kbot-stiff-feet" else 2e-3),
                          ("dbg_qacc_smooth", "qacc_smooth", 1e-4),
                          ("qacc", "qacc", STIFF_TOL if name == "kbot-stiff-feet" else ONE_STEP_TOL),
                          ("qacc_warmstart", "qacc", STIFF_TOL if name == "kbot-stiff-feet" else ONE_STEP_TOL)]:
        err = rel_err(g[got], want[ref]).max()
        assert err <= tol, f"{name}.{ref}: rel err {err:.2e} > {tol}"
    if m.ns:
        assert np.abs(g["contact_dist"] - want["con_dist"]).max() < 1e-6
        assert np.array_equal(g["nefc"], want["nefc"]), "active contact sets differ"  # integer: bit-exact
        assert (want["nefc"] > 0).sum() >= N // 4


@pytest.mark.parametrize("steps,tol", [(1, ONE_STEP_TOL), (10, TEN_STEP_TOL)])
def test_torque_driven_trajectories(setup, steps, tol):
    """`steps` physics steps (one substep per call, constant torque) against the oracle."""
    from ksim_amd import physics
    from ksim_amd._lib_dyn import KS_ACT_TORQUE

    name, m, dm = setup
    N = 32
    qpos, qvel = random_states(m, N, seed=21, vel_scale=0.3)
    rng = np.random.default_rng(22)
    ctrl = rng.normal(size=(N, m.nu)) * 3
    orc = Oracle(m.arrays())
    wq, wv = [], []
    for e in range(N):
        d = orc.data(qpos[e], qvel[e])
        d.ctrl = ctrl[e]
        for _ in range(steps):
            orc.step(d)
        wq.append(np.array(d.qpos)); wv.append(np.array(d.qvel))
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=zeros(N, m.nv), time=zeros(N), last_ctrl=t32(ctrl),
               action=t32(ctrl))
    for _ in range(steps):
        physics.control_step(dm, buf, substeps=1, actuator_type=KS_ACT_TORQUE)
    eq, ev = rel_err(buf["qpos"].cpu().numpy(), wq).max(), rel_err(buf["qvel"].cpu().numpy(), wv).max()
    assert eq <= tol and ev <= tol, f"{name}: qpos {eq:.2e} qvel {ev:.2e} > {tol}"
    # the vector-wise measure above lets a small coordinate be far off relatively: every coordinate of qpos on its own, against
    # its own magnitude with a floor of 0.1 (rad or m)
    dq = np.abs(buf["qpos"].cpu().numpy().astype(np.float64) - np.array(wq))
    worst = (dq / np.maximum(np.abs(np.array(wq)), 0.1)).max()
    assert worst <= tol, f"{name}: a coordinate of qpos is off by {worst:.2e} of its own size > {tol}"
    np.testing.assert_allclose(buf["time"].cpu().numpy(), steps * m.dt, rtol=1e-5)


def _oracle_control_steps(m, qpos, qvel, actions, kp, kd, clip, S, latency, friction, mass_scale, period=1, arm=None, damp=None):
    """Python composition of the oracle's pieces: engine.py:287-320 + actuators.py:198-217 + the C step."""
    orc = Oracle(m.arrays())
    N = qpos.shape[0]
    rq, rv = (7, 6) if m.has_free_root else (0, 0)
    datas = [orc.data(qpos[e], qvel[e], friction=friction[e], mass_scale=mass_scale[e],
                      armature_scale=None if arm is None else arm[e], damping_scale=None if damp is None else damp[e]) for e in range(N)]
    last = np.zeros((N, m.nu))
    for action in actions:
        for e, d in enumerate(datas):
            torque = np.zeros(m.nu)
            for s in range(S):
                c = oterms.latency_blend(float(s), latency[e], last[e], action[e], np.zeros(m.nu, bool))
                if s % period == 0:
                    torque = oterms.position_actuator_torque(c, np.array(d.qpos[rq:]), np.array(d.qvel[rv:]), kp, kd, clip)
                d.ctrl = torque
                orc.step(d)
        last = action.copy()
    return datas


@pytest.mark.parametrize("name,S,T,period", [("chain", 1, 10, 1), ("kbot", 4, 2, 1), ("humanoid", 4, 2, 2),
                                             ("chain-implicit", 1, 10, 1), ("kbot-implicit", 4, 2, 1),
                                             ("kbot-implicit", 1, 1, 1), ("humanoid-implicit", 4, 2, 2),
                                             ("kbot-limits", 4, 2, 1), ("chain-friction", 1, 10, 1)])
def test_position_controlled_steps(name, S, T, period):
    """Fused control step (latency blend + PD + S substeps) with per-env friction / mass scale."""
    from ksim_amd import physics

    m = MODELS[name]()
    dm = physics.DeviceModel(m)
    N = 24
    qpos, qvel = random_states(m, N, seed=31, vel_scale=0.2, joint_range=0.3)
    rng = np.random.default_rng(32)
    actions = rng.uniform(-0.5, 0.5, size=(T, N, m.nu))
    kp, kd = rng.uniform(20, 150, m.nu), rng.uniform(1, 5, m.nu)
    clip = np.where(rng.random(m.nu) < 0.5, 40.0, np.inf)
    latency = rng.uniform(0.0, 1.5, N)
    fr, ms = rng.uniform(0.4, 1.2, N), rng.uniform(0.9, 1.1, (N, m.nb))
    # per-env armature and damping factors (ArmatureRandomizer, JointDampingRandomizer) on the implicit models
    arm = rng.uniform(0.8, 1.2, (N, m.nv)) if "implicit" in name else None
    damp = rng.uniform(0.5, 1.5, (N, m.nv)) if "implicit" in name else None
    datas = _oracle_control_steps(m, qpos, qvel, actions, kp, kd, clip, S, latency, fr, ms, period, arm, damp)
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=zeros(N, m.nv), time=zeros(N), last_ctrl=zeros(N, m.nu),
               armature_scale=None if arm is None else t32(arm), damping_scale=None if damp is None else t32(damp),
               latency=t32(latency), kp=t32(kp), kd=t32(kd), ctrl_clip=t32(clip), friction=t32(fr), mass_scale=t32(ms),
               ctrl_out=zeros(N, m.nu), xpos=zeros(N, m.nb * 3), xquat=zeros(N, m.nb * 4), qacc=zeros(N, m.nv))
    for k in range(T):
        buf["action"] = t32(actions[k])
        physics.control_step(dm, buf, substeps=S, actuator_period=period)
    tol = ONE_STEP_TOL if S * T == 1 else TEN_STEP_TOL
    for field, ref in [("qpos", "qpos"), ("qvel", "qvel"), ("ctrl_out", "ctrl"), ("qacc", "qacc")]:
        want = np.array([np.array(getattr(d, ref)) for d in datas])
        err = rel_err(buf[field].cpu().numpy(), want).max()
        assert err <= tol, f"{name}.{field}: {err:.2e} > {tol}"
    # xpos / xquat are those of the start of the last substep (mjx.step runs kinematics before integrating)
    want = np.array([np.array(d.xpos).reshape(-1) for d in datas])
    assert rel_err(buf["xpos"].cpu().numpy(), want).max() <= tol
    assert torch.equal(buf["last_ctrl"], buf["action"])  # engine.py:355


def test_cfg1_chain_200_steps():
    """benchmark config 1: 128 envs, 200 steps, targets resampled every step; checked at steps 1, 10, 200."""
    from ksim_amd import physics

    m = km.pendulum_chain_model()
    dm = physics.DeviceModel(m)
    rng = np.random.default_rng(1001)
    N, T = 128, 200
    qpos = rng.uniform(-0.5, 0.5, (N, 3))
    targets = rng.uniform(-1.0, 1.0, (T, N, 3))
    kp, kd, clip = np.full(3, 20.0), np.full(3, 1.0), np.full(3, np.inf)
    orc = Oracle(m.arrays())
    datas = [orc.data(qpos[e]) for e in range(N)]
    buf = dict(qpos=t32(qpos), qvel=zeros(N, 3), qacc_warmstart=zeros(N, 3), time=zeros(N), last_ctrl=zeros(N, 3),
               kp=t32(kp), kd=t32(kd), ctrl_clip=t32(clip), qacc=zeros(N, 3))
    # latency 1 substep back: the reference's blend applies the new target from substep 1 on, so with one substep
    # per control step each step is driven by the previous target (engine.py:287-288)
    last = np.zeros((N, 3))
    for k in range(T):
        buf["action"] = t32(targets[k])
        physics.control_step(dm, buf, substeps=1)
        for e, d in enumerate(datas):
            d.ctrl = oterms.position_actuator_torque(last[e], np.array(d.qpos), np.array(d.qvel), kp, kd, clip)
            orc.step(d)
        last = targets[k]
        if k + 1 in (1, 10, 200):
            want_q = np.array([np.array(d.qpos) for d in datas])
            want_v = np.array([np.array(d.qvel) for d in datas])
            tol = ONE_STEP_TOL if k == 0 else (TEN_STEP_TOL if k == 9 else 5e-3)
            eq = rel_err(buf["qpos"].cpu().numpy(), want_q).max()
            ev = rel_err(buf["qvel"].cpu().numpy(), want_v).max()
            assert eq <= tol and ev <= tol, f"step {k + 1}: qpos {eq:.2e} qvel {ev:.2e}"
            if k == 0:
                want_a = np.array([np.array(d.qacc) for d in datas])
                assert rel_err(buf["qacc"].cpu().numpy(), want_a).max() <= ONE_STEP_TOL


def test_step_is_deterministic_and_env_independent():
    from ksim_amd import physics

    m = km.kbot_scale_model()
    dm = physics.DeviceModel(m)
    N = 64
    qpos, qvel = random_states(m, N, seed=41)
    rng = np.random.default_rng(42)
    act = rng.uniform(-0.3, 0.3, (N, m.nu))
    kp, kd, clip = np.full(m.nu, 60.0), np.full(m.nu, 2.0), np.full(m.nu, 80.0)

    def run(idx):
        buf = dict(qpos=t32(qpos[idx]), qvel=t32(qvel[idx]), qacc_warmstart=zeros(len(idx), m.nv),
                   last_ctrl=zeros(len(idx), m.nu), action=t32(act[idx]), kp=t32(kp), kd=t32(kd), ctrl_clip=t32(clip))
        physics.control_step(dm, buf, substeps=4)
        return buf["qpos"].clone(), buf["qvel"].clone()

    a = run(np.arange(N))
    b = run(np.arange(N))
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    perm = np.random.default_rng(0).permutation(N)[:17]  # ragged subset in another order: same per-env bits
    c = run(perm)
    assert torch.equal(c[0], a[0][torch.from_numpy(perm).to(DEV)])


def test_errors_are_reported():
    from ksim_amd import _lib, physics

    m = km.kbot_scale_model()
    dm = physics.DeviceModel(m)
    N = 4
    good = dict(qpos=zeros(N, m.nq), qvel=zeros(N, m.nv), qacc_warmstart=zeros(N, m.nv), last_ctrl=zeros(N, m.nu),
                action=zeros(N, m.nu), kp=zeros(m.nu), kd=zeros(m.nu), ctrl_clip=zeros(m.nu))
    with pytest.raises(_lib.KsError):
        physics.control_step(dm, dict(good, qvel=zeros(N, m.nv + 1)), substeps=4)
    with pytest.raises(_lib.KsError):
        physics.control_step(dm, dict(good, kp=None), substeps=4)
    with pytest.raises(_lib.KsError):
        physics.control_step(dm, good, substeps=0)
    with pytest.raises(_lib.KsError):
        physics.control_step(dm, dict(good, qpos=torch.zeros(N, m.nq)), substeps=4)
    physics.control_step(dm, dict(qpos=zeros(0, m.nq), qvel=zeros(0, m.nv), last_ctrl=zeros(0, m.nu),
                                  action=zeros(0, m.nu), kp=zeros(m.nu), kd=zeros(m.nu), ctrl_clip=zeros(m.nu)),
                         substeps=4)  # empty batch is a no-op
    with pytest.raises(ValueError):
        km.ModelBuilder().add_body(0, (0, 0, 0), joint=None, mass=1.0, inertia=(1, 1, 1))


def test_velocity_events_inside_the_substep_loop():
    """Linear / angular push and jump events (ksim/events.py) fired from explicit draws: the fused step against
    the oracle with the same impulses applied before each physics substep, and the timers bit for bit."""
    from ksim_amd import events as kev, physics

    m = MODELS["kbot"]()
    dm = physics.DeviceModel(m)
    N, S, T = 16, 4, 3
    qpos, qvel = random_states(m, N, seed=41, vel_scale=0.1, joint_range=0.2)
    rng = np.random.default_rng(42)
    actions = rng.uniform(-0.3, 0.3, size=(T, N, m.nu))
    kp, kd, clip = rng.uniform(20, 150, m.nu), rng.uniform(1, 3, m.nu), np.full(m.nu, 40.0)
    evs = [kev.LinearPushEvent(linvel=1.0, vel_range=(0.2, 0.8), interval_range=(0.004, 0.03), scale=0.5),
           kev.AngularPushEvent(angvel=2.0, vel_range=(0.0, 1.0), interval_range=(0.01, 0.05)),
           kev.JumpEvent(jump_height_range=(0.02, 0.1), interval_range=(0.02, 0.06))]
    kinds = [("linear", dict(linvel=1.0, vel_range=(0.2, 0.8), interval_range=(0.004, 0.03)), 0.5),
             ("angular", dict(angvel=2.0, vel_range=(0.0, 1.0), interval_range=(0.01, 0.05)), 1.0),
             ("jump", dict(jump_height_range=(0.02, 0.1), interval_range=(0.02, 0.06)), 1.0)]
    u = rng.random(size=(T, S, N, 3, 12)).astype(np.float32)  # the velocity events use the first three draws
    left0 = rng.uniform(0.0, 0.03, size=(3, N)).astype(np.float32)
    # oracle: per env, per substep: PD torque from the pre-event state, events, physics step (engine.py:290-335)
    orc = Oracle(m.arrays())
    datas = [orc.data(qpos[e], qvel[e]) for e in range(N)]
    left = left0.astype(np.float64).copy()
    last = np.zeros((N, m.nu))
    fired = 0
    for k in range(T):
        for e, d in enumerate(datas):
            for s in range(S):
                c = oterms.latency_blend(float(s), 0.0, last[e], actions[k, e], np.zeros(m.nu, bool))
                d.ctrl = oterms.position_actuator_torque(c, np.array(d.qpos[7:]), np.array(d.qvel[6:]), kp, kd, clip)
                for j, (kind, prm, scale) in enumerate(kinds):
                    imp, left[j, e] = oterms.velocity_event(kind, prm, left[j, e], m.dt, u[k, s, e, j], scale)
                    left[j, e] = float(np.float32(left[j, e]))
                    fired += bool(imp.any())
                    for i in range(6):
                        d.qvel[i] += imp[i]
                orc.step(d)
        last = actions[k].copy()
    assert fired >= 20, "the draws did not fire enough events to test anything"
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=zeros(N, m.nv), time=zeros(N), last_ctrl=zeros(N, m.nu),
               kp=t32(kp), kd=t32(kd), ctrl_clip=t32(clip))
    state = t32(left0)
    descs = [ev.desc(1.0) for ev in evs]
    for k in range(T):
        buf["action"] = t32(actions[k])
        physics.control_step(dm, buf, substeps=S, events=(descs, state, t32(u[k]), None))
    for field in ("qpos", "qvel"):
        want = np.array([np.array(getattr(d, field)) for d in datas])
        assert rel_err(buf[field].cpu().numpy(), want).max() <= TEN_STEP_TOL, field
    np.testing.assert_allclose(state.cpu().numpy(), left, rtol=0, atol=1e-6)  # timers: float32 arithmetic on both sides
    # without draws the kernel's own counter-based stream is used: reproducible, and the timers stay inside their ranges
    outs = []
    for _ in range(2):
        b2 = {k: v.clone() for k, v in buf.items()}
        st = t32(left0)
        from ksim_amd import _lib_terms as T_
        for k in range(20):
            physics.control_step(dm, b2, substeps=S, events=(descs, st, None, T_.KsRng(7, k, None)))
        outs.append((b2["qvel"].clone(), st.clone()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    hi = torch.tensor([0.03, 0.05, 0.06], device=DEV)[:, None]
    assert (outs[0][1] <= hi).all() and (outs[0][1] > -0.006).all()


def test_force_push_event_holds_a_wrench_on_one_body():
    """ForcePushEvent (ksim/events.py:240-365) from explicit draws, on a foot and on the torso of the biped, together with a
    linear push: state machine and trajectories against the oracle, which applies the same wrench as xfrc_applied."""
    from ksim_amd import events as kev, physics

    m = MODELS["kbot"]()
    dm = physics.DeviceModel(m)
    N, S, T = 16, 4, 4
    qpos, qvel = random_states(m, N, seed=51, vel_scale=0.1, joint_range=0.2)
    rng = np.random.default_rng(52)
    actions = rng.uniform(-0.3, 0.3, size=(T, N, m.nu))
    kp, kd, clip = rng.uniform(20, 150, m.nu), rng.uniform(1, 3, m.nu), np.full(m.nu, 40.0)
    foot = m.nb - 1
    prm = [dict(max_force=80.0, max_torque=10.0, force_range=(0.3, 1.0), duration_range=(0.01, 0.04), interval_range=(0.02, 0.06)),
           None,
           dict(max_force=30.0, max_torque=4.0, force_range=(0.5, 1.0), duration_range=(0.005, 0.03), interval_range=(0.01, 0.05))]
    push = dict(linvel=1.0, vel_range=(0.2, 0.8), interval_range=(0.004, 0.03))
    scales = [0.9, 1.0, 1.0]
    # only the last force push in the list acts (each clears the applied forces of all bodies, events.py:302), so the
    # first one is listed to check exactly that: its state advances, its wrench never reaches the body
    evs = [kev.ForcePushEvent(body_id=1, scale=scales[0], **prm[0]), kev.LinearPushEvent(**push),
           kev.ForcePushEvent(body_id=foot, scale=scales[2], **prm[2])]
    bodies = [1, None, foot]
    u = rng.random(size=(T, S, N, 3, 12)).astype(np.float32)
    left0 = rng.uniform(0.0, 0.03, size=(3, N)).astype(np.float32)
    force0 = np.zeros((3, N, 8), np.float32)
    force0[0, :, 0] = rng.uniform(0.0, 0.02, N); force0[0, :, 1:7] = rng.normal(size=(N, 6)) * 5   # a push already under way
    force0[2, :, 0] = rng.uniform(0.0, 0.02, N); force0[2, :, 1:7] = rng.normal(size=(N, 6)) * 5
    orc = Oracle(m.arrays())
    datas = [orc.data(qpos[e], qvel[e]) for e in range(N)]
    left = left0.astype(np.float64).copy()
    fstate = [[(float(left0[j, e]), float(force0[j, e, 0]), force0[j, e, 1:7].astype(np.float64)) for e in range(N)] for j in range(3)]
    last = np.zeros((N, m.nu))
    applied_steps = 0
    for k in range(T):
        for e, d in enumerate(datas):
            for s in range(S):
                c = oterms.latency_blend(float(s), 0.0, last[e], actions[k, e], np.zeros(m.nu, bool))
                d.ctrl = oterms.position_actuator_torque(c, np.array(d.qpos[7:]), np.array(d.qvel[6:]), kp, kd, clip)
                d.xfrc_applied = 0.0
                for j in range(3):
                    if prm[j] is None:
                        imp, left[j, e] = oterms.velocity_event("linear", push, left[j, e], m.dt, u[k, s, e, j], 1.0)
                        left[j, e] = float(np.float32(left[j, e]))
                        for i in range(6):
                            d.qvel[i] += imp[i]
                    else:
                        ap, st = oterms.force_push_event(prm[j], fstate[j][e], m.dt, u[k, s, e, j], scales[j])
                        fstate[j][e] = (float(np.float32(st[0])), float(np.float32(st[1])), st[2].astype(np.float32).astype(np.float64))
                        d.xfrc_applied = 0.0           # events.py:302: every force push clears all bodies first
                        d.xfrc_applied[bodies[j]] = ap
                        applied_steps += bool(ap.any()) and j == 2
                orc.step(d)
        last = actions[k].copy()
    assert applied_steps >= 40, "the draws did not hold a force long enough to test anything"
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=zeros(N, m.nv), time=zeros(N), last_ctrl=zeros(N, m.nu),
               kp=t32(kp), kd=t32(kd), ctrl_clip=t32(clip))
    state, force = t32(left0), t32(force0)
    descs = [ev.desc(1.0) for ev in evs]
    with pytest.raises(Exception, match="event_force"):
        physics.control_step(dm, dict(buf, action=t32(actions[0])), substeps=S, events=(descs, state, t32(u[0]), None))
    for k in range(T):
        buf["action"] = t32(actions[k])
        physics.control_step(dm, buf, substeps=S, events=(descs, state, t32(u[k]), None, force))
    for field in ("qpos", "qvel"):
        want = np.array([np.array(getattr(d, field)) for d in datas])
        assert rel_err(buf[field].cpu().numpy(), want).max() <= TEN_STEP_TOL, field
    got_t, got_f = state.cpu().numpy(), force.cpu().numpy()
    np.testing.assert_allclose(got_t[1], left[1], rtol=0, atol=1e-6)
    for j in (0, 2):
        np.testing.assert_allclose(got_t[j], [fstate[j][e][0] for e in range(N)], rtol=0, atol=1e-6)
        np.testing.assert_allclose(got_f[j, :, 0], [fstate[j][e][1] for e in range(N)], rtol=0, atol=1e-6)
        np.testing.assert_allclose(got_f[j, :, 1:7], [fstate[j][e][2] for e in range(N)], rtol=1e-5, atol=1e-5)
    # a bad body index is refused before any launch
    bad = [kev.ForcePushEvent(body_id=m.nb, **prm[0]).desc(1.0)]
    with pytest.raises(Exception, match="body"):
        physics.control_step(dm, buf, substeps=S, events=(bad, t32(left0[:1]), None, None, t32(force0[:1])))


def test_position_velocity_actuator_steps():
    """PositionVelocityActuator (ksim/actuators.py:241-293): a 2 nu wide action of position and velocity targets, blended
    with the previous action under latency, with noise on both halves and dropped entries."""
    from ksim_amd import physics
    from ksim_amd._lib_dyn import KS_ACT_POSITION_VELOCITY

    m = MODELS["kbot-implicit"]()
    dm = physics.DeviceModel(m)
    N, S, T = 20, 4, 3
    nu = m.nu
    qpos, qvel = random_states(m, N, seed=61, vel_scale=0.2, joint_range=0.3)
    rng = np.random.default_rng(62)
    actions = np.concatenate([rng.uniform(-0.4, 0.4, size=(T, N, nu)), rng.uniform(-1.0, 1.0, size=(T, N, nu))], axis=-1)
    kp, kd, clip = rng.uniform(20, 150, nu), rng.uniform(1, 4, nu), np.full(nu, 45.0)
    latency = rng.uniform(0.0, 1.5, N)
    zero = rng.normal(size=(N, nu)) * 0.02
    an = rng.normal(size=(T, S, N, 2 * nu)) * 0.01
    tn = rng.normal(size=(T, S, N, nu)) * 0.1
    drop = rng.random((T, N, 2 * nu)) < 0.1
    orc = Oracle(m.arrays())
    datas = [orc.data(qpos[e], qvel[e]) for e in range(N)]
    last = np.zeros((N, 2 * nu))
    for k in range(T):
        for e, d in enumerate(datas):
            for s in range(S):
                c = oterms.latency_blend(float(s), latency[e], last[e], actions[k, e], drop[k, e])
                d.ctrl = oterms.position_velocity_actuator_torque(c, np.array(d.qpos[7:]) - zero[e], np.array(d.qvel[6:]), kp, kd, clip,
                                                                  pos_noise=an[k, s, e, :nu], vel_noise=an[k, s, e, nu:], torque_noise=tn[k, s, e])
                orc.step(d)
        last = actions[k].copy()
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=zeros(N, m.nv), time=zeros(N), last_ctrl=zeros(N, 2 * nu),
               latency=t32(latency), zero_offset=t32(zero), kp=t32(kp), kd=t32(kd), ctrl_clip=t32(clip), ctrl_out=zeros(N, nu))
    for k in range(T):
        buf.update(action=t32(actions[k]), action_noise=t32(an[k]), torque_noise=t32(tn[k]),
                   drop=torch.from_numpy(drop[k].astype(np.uint8)).to(DEV))
        physics.control_step(dm, buf, substeps=S, actuator_type=KS_ACT_POSITION_VELOCITY)
    for field, ref in [("qpos", "qpos"), ("qvel", "qvel"), ("ctrl_out", "ctrl")]:
        want = np.array([np.array(getattr(d, ref)) for d in datas])
        assert rel_err(buf[field].cpu().numpy(), want).max() <= TEN_STEP_TOL, field
    assert torch.equal(buf["last_ctrl"], buf["action"])
    with pytest.raises(Exception, match="last_ctrl"):
        physics.control_step(dm, dict(buf, last_ctrl=zeros(N, nu)), substeps=S, actuator_type=KS_ACT_POSITION_VELOCITY)


def test_launch_order_does_not_change_results_and_sorts_heaviest_first():
    """Stepping the envs in a heaviest-first order gives the same bits as the natural order; the order kernel sorts."""
    from ksim_amd import physics

    m = MODELS["kbot-implicit"]()
    dm = physics.DeviceModel(m)
    N, S = 300, 4
    qpos, qvel = random_states(m, N, seed=71, vel_scale=0.2, joint_range=0.3)
    rng = np.random.default_rng(72)
    kp, kd, clip = rng.uniform(20, 150, m.nu), rng.uniform(1, 3, m.nu), np.full(m.nu, 40.0)
    act = rng.uniform(-0.3, 0.3, size=(N, m.nu))
    def run(order):
        buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=zeros(N, m.nv), time=zeros(N), last_ctrl=zeros(N, m.nu),
                   action=t32(act), kp=t32(kp), kd=t32(kd), ctrl_clip=t32(clip), work=zeros(N, dtype=torch.int32),
                   nefc=zeros(N, dtype=torch.int32), solver_niter=zeros(N, dtype=torch.int32), env_order=order)
        for _ in range(3):
            physics.control_step(dm, buf, substeps=S)
        return buf
    a = run(None)
    work = a["work"]
    assert (work >= 4 * 16).all() and work.max() > work.min()          # airborne envs cost the floor, contacts more
    order = torch.empty(N, dtype=torch.int32, device=DEV)
    physics.work_order(dm, work, order)
    o = order.cpu().numpy(); w = work.cpu().numpy()
    assert sorted(o.tolist()) == list(range(N)) and (np.diff(w[o] >> 2) <= 0).all()  # buckets of four work units
    b = run(order)
    for k in ("qpos", "qvel", "qacc_warmstart", "work", "nefc", "solver_niter"):
        assert torch.equal(a[k], b[k]), k
    rev = torch.from_numpy(np.ascontiguousarray(o[::-1])).to(DEV)
    assert torch.equal(run(rev)["qpos"], a["qpos"])
    # a multiple of 8 envs: sorted inside the eight contiguous regions, region r at positions r, r + 8, ...
    N2 = 1024
    w2 = torch.from_numpy(np.random.default_rng(73).integers(64, 900, N2).astype(np.int32)).to(DEV)
    o2 = torch.empty(N2, dtype=torch.int32, device=DEV)
    physics.work_order(dm, w2, o2)
    o2, w2 = o2.cpu().numpy(), w2.cpu().numpy()
    assert sorted(o2.tolist()) == list(range(N2))
    for r in range(8):
        mine = o2[r::8]
        assert mine.min() >= r * N2 // 8 and mine.max() < (r + 1) * N2 // 8 and (np.diff(w2[mine] >> 2) <= 0).all()


def test_joint_limit_and_dry_friction_closed_forms():
    """The kernel itself against the closed forms that pin the oracle's limit and friction rows."""
    from ksim_amd import physics
    from ksim_amd._lib_dyn import KS_ACT_TORQUE

    # dry friction f on a hinge without gravity or damping: a fast joint decelerates at f / I per unit time
    f = 0.4
    m = km.pendulum_chain_model(n_links=1, damping=0.0, frictionloss=f, gravity=(0.0, 0.0, 0.0))
    inertia = float(km.host_mass_matrix(m.arrays(), m.qpos0)[0, 0])
    dm = physics.DeviceModel(m)
    buf = dict(qpos=zeros(2, 1), qvel=t32([[2.0], [-2.0]]), qacc_warmstart=zeros(2, 1), time=zeros(2),
               last_ctrl=zeros(2, 1), action=zeros(2, 1))
    physics.control_step(dm, buf, substeps=10, actuator_type=KS_ACT_TORQUE)
    want = 2.0 - 10 * m.dt * f / inertia
    np.testing.assert_allclose(buf["qvel"].cpu().numpy()[:, 0], [want, -want], rtol=1e-5)
    for _ in range(60):
        physics.control_step(dm, buf, substeps=50, actuator_type=KS_ACT_TORQUE)
    assert buf["qvel"].abs().max().item() < 1e-6  # stopped, and stays stopped

    # a link on a horizontal hinge limited to (0.3, 1.0) settles just below 0.3, where the limit force
    # D k imp |pos| balances the gravity torque m g (L / 2) sin q
    L, mass = 0.5, 1.0
    m = km.pendulum_chain_model(n_links=1, length=L, mass=mass, damping=0.5, joint_range=(0.3, 1.0))
    dm = physics.DeviceModel(m)
    buf = dict(qpos=t32([[0.6]]), qvel=zeros(1, 1), qacc_warmstart=zeros(1, 1), time=zeros(1), last_ctrl=zeros(1, 1),
               action=zeros(1, 1))
    for _ in range(80):
        physics.control_step(dm, buf, substeps=50, actuator_type=KS_ACT_TORQUE)
    q = buf["qpos"].item()
    pos = q - 0.3
    assert abs(buf["qvel"].item()) < 1e-5 and -0.01 < pos < 0
    dmin, dmax, width, mid, power = m.solimp
    x = abs(pos) / width
    y = (1 / mid ** (power - 1)) * x**power if x < mid else 1 - (1 / (1 - mid) ** (power - 1)) * (1 - x) ** power
    imp = dmax if x > 1 else float(np.clip(dmin + y * (dmax - dmin), dmin, dmax))
    k = 1 / (dmax**2 * max(m.solref[0], 2 * m.dt) ** 2 * m.solref[1] ** 2)
    inertia = float(km.host_mass_matrix(m.arrays(), m.qpos0)[0, 0])
    R = (1 / inertia) * (1 - imp) / imp
    # fp32 state: the penetration is ~1e-4 rad on an angle of 0.3, so it is resolved to about three digits
    assert (1 / R) * k * imp * abs(pos) == pytest.approx(mass * 9.81 * (L / 2) * np.sin(q), rel=5e-3)


def test_model_loaded_from_mjcf_matches_oracle():
    """A model read from an MJCF file (welded bodies, capsule feet, limits, dry friction, its own contact and joint
    solref / solimp): forward quantities and ten physics steps against the oracle."""
    import os
    from ksim_amd import physics
    from ksim_amd._lib_dyn import KS_ACT_TORQUE
    from ksim_amd.mjcf import load_mjcf

    m = load_mjcf(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mini_biped.mjcf"), integrator="implicitfast")
    dm = physics.DeviceModel(m)
    N = 40
    rng = np.random.default_rng(61)
    qpos, qvel = random_states(m, N, seed=62, vel_scale=0.3)
    # hips within and slightly beyond their ranges, knees around their lower limit
    qpos[:, 7] = rng.uniform(-1.05, 1.55, N); qpos[:, 9] = rng.uniform(-1.55, 1.05, N)
    qpos[:, 8] = rng.uniform(-0.05, 1.0, N); qpos[:, 10] = rng.uniform(-0.5, 0.5, N)
    ctrl = rng.normal(size=(N, m.nu)) * 3
    warm = np.zeros((N, m.nv))
    want = oracle_forward(m, qpos, qvel, ctrl, None, None, warm)
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=t32(warm), ctrl_in=t32(ctrl), qacc=zeros(N, m.nv),
               xpos=zeros(N, m.nb * 3), nefc=zeros(N, dtype=torch.int32), contact_dist=zeros(N, m.ns))
    physics.forward(dm, buf)
    assert rel_err(buf["xpos"].cpu().numpy(), want["xpos"]).max() < 1e-5
    assert np.array_equal(buf["nefc"].cpu().numpy(), want["nefc"])
    assert (want["nefc"] > 4).sum() >= N // 3  # friction rows always, limit and contact rows in many envs
    assert rel_err(buf["qacc"].cpu().numpy(), want["qacc"]).max() <= ONE_STEP_TOL
    orc = Oracle(m.arrays())
    wq, wv = [], []
    for e in range(N):
        d = orc.data(qpos[e], qvel[e])
        d.ctrl = ctrl[e]
        for _ in range(10):
            orc.step(d)
        wq.append(np.array(d.qpos)); wv.append(np.array(d.qvel))
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=zeros(N, m.nv), time=zeros(N), last_ctrl=t32(ctrl), action=t32(ctrl))
    for _ in range(10):
        physics.control_step(dm, buf, substeps=1, actuator_type=KS_ACT_TORQUE)
    eq, ev = rel_err(buf["qpos"].cpu().numpy(), wq).max(), rel_err(buf["qvel"].cpu().numpy(), wv).max()
    assert eq <= TEN_STEP_TOL and ev <= TEN_STEP_TOL, f"qpos {eq:.2e} qvel {ev:.2e}"


def test_humanoid_file_with_several_hinges_per_body_matches_oracle():
    """A model of the walking example's kind read from an MJCF file: bodies with three hinges (massless bodies in between),
    joint springs, limit rows with their own solimp, feet that collide through explicit pairs; forward quantities and ten
    physics steps against the oracle."""
    import os
    from ksim_amd import physics
    from ksim_amd._lib_dyn import KS_ACT_TORQUE
    from ksim_amd.mjcf import load_mjcf

    m = load_mjcf(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mini_humanoid.mjcf"), integrator="implicitfast")
    dm = physics.DeviceModel(m)
    N = 40
    rng = np.random.default_rng(91)
    qpos, qvel = random_states(m, N, seed=92, vel_scale=0.3, joint_range=0.3)
    # knees from bent to slightly beyond their upper limit of 5 degrees, some hips slightly beyond theirs
    qpos[:, 10] = rng.uniform(-1.2, 0.05, N); qpos[:, 14] = rng.uniform(-1.2, 0.05, N)
    qpos[0::3, 10] = rng.uniform(0.09, 0.14, len(qpos[0::3])); qpos[1::3, 14] = rng.uniform(0.09, 0.12, len(qpos[1::3]))
    qpos[2::4, 7] = rng.uniform(0.35, 0.4, len(qpos[2::4]))
    ctrl = rng.normal(size=(N, m.nu)) * 0.5
    warm = np.zeros((N, m.nv))
    want = oracle_forward(m, qpos, qvel, ctrl, None, None, warm)
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=t32(warm), ctrl_in=t32(ctrl), qacc=zeros(N, m.nv),
               xpos=zeros(N, m.nb * 3), xquat=zeros(N, m.nb * 4), nefc=zeros(N, dtype=torch.int32), contact_dist=zeros(N, m.ns),
               dbg_M=zeros(N, m.nv * m.nv), dbg_qacc_smooth=zeros(N, m.nv))
    physics.forward(dm, buf)
    assert rel_err(buf["xpos"].cpu().numpy(), want["xpos"]).max() < 1e-5
    assert rel_err(buf["xquat"].cpu().numpy(), want["xquat"]).max() < 1e-5
    assert rel_err(buf["dbg_M"].cpu().numpy(), want["M"]).max() < 1e-5
    assert rel_err(buf["dbg_qacc_smooth"].cpu().numpy(), want["qacc_smooth"]).max() <= ONE_STEP_TOL  # springs included
    assert np.array_equal(buf["nefc"].cpu().numpy(), want["nefc"])
    assert (want["nefc"] > 0).sum() >= N // 2
    err = rel_err(buf["qacc"].cpu().numpy(), want["qacc"]).max()
    assert err <= ONE_STEP_TOL, f"qacc {err:.2e}"
    orc = Oracle(m.arrays())
    wq, wv = [], []
    for e in range(N):
        d = orc.data(qpos[e], qvel[e])
        d.ctrl = ctrl[e]  # clipped to the motors' control range and geared inside the model
        for _ in range(10):
            orc.step(d)
        wq.append(np.array(d.qpos)); wv.append(np.array(d.qvel))
    buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=zeros(N, m.nv), time=zeros(N), last_ctrl=t32(ctrl), action=t32(ctrl))
    for _ in range(10):
        physics.control_step(dm, buf, substeps=1, actuator_type=KS_ACT_TORQUE)
    eq, ev = rel_err(buf["qpos"].cpu().numpy(), wq).max(), rel_err(buf["qvel"].cpu().numpy(), wv).max()
    assert eq <= TEN_STEP_TOL and ev <= TEN_STEP_TOL, f"qpos {eq:.2e} qvel {ev:.2e}"


def test_per_env_model_field_overrides_match_oracle():
    """Per-env centres of mass, principal inertias, dry friction and contact spheres (the remaining physics randomisers)
    through the step kernel, two control steps of four substeps against the oracle; dry friction given per env to a model
    that has none of its own selects the kernel variant with dof-lane rows."""
    from ksim_amd import physics
    from ksim_amd._lib_dyn import KS_ACT_TORQUE

    for name, m in (("with friction", km.kbot_scale_model(integrator="implicitfast", frictionloss=0.1, joint_range=(-1.0, 1.0))),
                    ("friction per env only", km.kbot_scale_model(integrator="implicitfast"))):
        dm = physics.DeviceModel(m)
        N = 24
        rng = np.random.default_rng(81)
        qpos, qvel = random_states(m, N, seed=82, vel_scale=0.3)
        ipos = m.body_ipos[None] + rng.uniform(-0.01, 0.01, (N,) + m.body_ipos.shape)
        inertia = m.body_inertia[None] * rng.uniform(0.95, 1.05, (N,) + m.body_inertia.shape)
        floss = np.concatenate([np.zeros((N, 6)), rng.uniform(0.05, 0.3, (N, m.nv - 6))], axis=1)
        spos = m.sph_pos[None] + rng.uniform(-0.002, 0.002, (N,) + m.sph_pos.shape)
        srad = m.sph_radius[None] * rng.uniform(0.95, 1.05, (N, m.ns))
        ctrl = rng.normal(size=(N, m.nu)) * 3
        orc = Oracle(m.arrays())
        wq, wv = [], []
        for e in range(N):
            d = orc.data(qpos[e], qvel[e], body_ipos=ipos[e], body_inertia=inertia[e], dof_frictionloss=floss[e], sph_pos=spos[e],
                         sph_radius=srad[e])
            d.ctrl = ctrl[e]
            for _ in range(8):
                orc.step(d)
            wq.append(np.array(d.qpos)); wv.append(np.array(d.qvel))
        buf = dict(qpos=t32(qpos), qvel=t32(qvel), qacc_warmstart=zeros(N, m.nv), time=zeros(N), last_ctrl=t32(ctrl), action=t32(ctrl),
                   body_ipos=t32(ipos.reshape(N, -1)), body_inertia=t32(inertia.reshape(N, -1)), frictionloss=t32(floss),
                   sph_pos=t32(spos.reshape(N, -1)), sph_radius=t32(srad), nefc=zeros(N, dtype=torch.int32))
        for _ in range(2):
            physics.control_step(dm, buf, substeps=4, actuator_type=KS_ACT_TORQUE)
        eq, ev = rel_err(buf["qpos"].cpu().numpy(), wq).max(), rel_err(buf["qvel"].cpu().numpy(), wv).max()
        assert eq <= TEN_STEP_TOL and ev <= TEN_STEP_TOL, f"{name}: qpos {eq:.2e} qvel {ev:.2e}"
        assert (buf["nefc"] >= m.nv - 6).all()  # a friction row per hinge in every env
    with pytest.raises(Exception, match="come together"):
        physics.control_step(dm, dict(buf, sph_radius=None), substeps=1, actuator_type=KS_ACT_TORQUE)
