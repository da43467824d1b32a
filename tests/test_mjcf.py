"""MJCF loader (CPU): a hand-written fixture with hand-derived expectations, and the reference's K-Bot file when present."""
import os
import re

import numpy as np
import pytest
from scipy.spatial.transform import Rotation

from ksim_amd import model as km
from ksim_amd.mjcf import load_mjcf, mat_to_quat, quat_to_mat
from oracle.dyn import Oracle

HERE = os.path.dirname(os.path.abspath(__file__))
MINI = os.path.join(HERE, "golden", "mini_biped.mjcf")
KBOT = "/root/reference/examples/kbot/robot/kbot-headless/robot.mjcf"


def _rot(q):  # scipy wants xyzw
    return Rotation.from_quat([q[1], q[2], q[3], q[0]])


def test_quaternion_helpers_against_scipy():
    rng = np.random.default_rng(0)
    for _ in range(50):
        q = rng.normal(size=4); q /= np.linalg.norm(q)
        np.testing.assert_allclose(quat_to_mat(q), _rot(q).as_matrix(), atol=1e-12)
        q2 = mat_to_quat(quat_to_mat(q))
        assert min(np.abs(q2 - q).max(), np.abs(q2 + q).max()) < 1e-12


def test_mini_biped_structure_defaults_and_welds():
    m = load_mjcf(MINI)
    assert (m.nb, m.nq, m.nv, m.nu, m.ns) == (6, 11, 10, 4, 4) and m.dt == 0.004
    assert m.body_names == ("world", "base", "hip_l", "knee_l", "hip_r", "knee_r")  # torso and sensor_l are welded away
    # classes: big / small joints and motors; knee_r has no range -> not limited
    assert list(m.jnt_limited) == [0, 0, 1, 1, 1, 0]
    np.testing.assert_allclose(m.jnt_range[2:5], [[-1.0, 1.5], [0.0, 2.4], [-1.5, 1.0]])
    np.testing.assert_allclose(m.dof_frictionloss[6:], [0.2, 0.1, 0.2, 0.1])
    np.testing.assert_allclose(m.dof_armature[6:], [0.03, 0.005, 0.03, 0.005])
    np.testing.assert_allclose(m.dof_damping[6:], [0.5, 0.0, 0.5, 0.0])
    np.testing.assert_allclose(m.act_gear, [1, 2, 1, 2])
    np.testing.assert_allclose(m.act_ctrlrange, [[-40, 40], [-10, 10], [-40, 40], [-10, 10]])
    # contact parameters from the collision class (solimp padded with MuJoCo's defaults), joints keep the defaults
    assert m.friction == 0.7 and tuple(m.solref) == (0.02, 0.8) and tuple(m.solimp) == (0.98, 0.99, 0.1, 0.5, 2.0)
    assert tuple(m.dof_solref) == (0.02, 1.0) and tuple(m.dof_solimp) == (0.9, 0.95, 0.001, 0.5, 2.0)
    # base = marker sphere (density 1000) + welded torso: composite mass, centre of mass and inertia by hand
    ms = 1000 * 4 / 3 * np.pi * 0.05**3
    Rz = _rot([np.sqrt(0.5), 0, 0, np.sqrt(0.5)]).as_matrix()
    ct = np.array([0, 0.02, 0]) + Rz @ np.array([0.01, 0, 0.15])
    assert m.body_mass[1] == pytest.approx(ms + 8)
    com = 8 * ct / (ms + 8)
    np.testing.assert_allclose(m.body_ipos[1], com, atol=1e-12)
    I = np.eye(3) * 0.4 * ms * 0.05**2 + ms * (com @ com * np.eye(3) - np.outer(com, com))
    d = ct - com
    I += Rz @ np.diag([0.2, 0.3, 0.05]) @ Rz.T + 8 * (d @ d * np.eye(3) - np.outer(d, d))
    Ri = quat_to_mat(m.body_iquat[1])
    np.testing.assert_allclose(Ri @ np.diag(m.body_inertia[1]) @ Ri.T, I, atol=1e-12)
    assert np.linalg.det(Ri) == pytest.approx(1.0)
    # knee_l carries the welded sensor body; its inertial has a rotated principal frame
    assert m.body_mass[3] == pytest.approx(1.1) and m.body_mass[5] == pytest.approx(1.0)
    Rk = _rot([0.9238795325112867, 0, 0, 0.3826834323650898]).as_matrix()
    c3 = (1.0 * np.array([0, -0.1, 0.01]) + 0.1 * np.array([0, -0.05, 0.02])) / 1.1
    I3 = np.zeros((3, 3))
    for mass, c, T in ((1.0, np.array([0, -0.1, 0.01]), Rk @ np.diag([0.01, 0.002, 0.011]) @ Rk.T),
                       (0.1, np.array([0, -0.05, 0.02]), np.eye(3) * 1e-4)):
        dd = c - c3
        I3 += T + mass * (dd @ dd * np.eye(3) - np.outer(dd, dd))
    R3 = quat_to_mat(m.body_iquat[3])
    np.testing.assert_allclose(R3 @ np.diag(m.body_inertia[3]) @ R3.T, I3, atol=1e-12)
    np.testing.assert_allclose(m.body_ipos[3], c3, atol=1e-12)


def test_mini_biped_kinematics_by_hand():
    """World positions of the four foot spheres at qpos0, composed by hand through the welded torso."""
    m = load_mjcf(MINI)
    kin = km.host_kinematics(m.arrays(), m.qpos0)
    got = np.array([kin["xpos"][b] + kin["xmat"][b] @ p for b, p in zip(m.sph_body, m.sph_pos)])
    base = np.array([0.1, 0, 0.6])
    Rt = _rot([np.sqrt(0.5), 0, 0, np.sqrt(0.5)])   # torso in base
    Rh = Rt * _rot([np.sqrt(0.5), np.sqrt(0.5), 0, 0])  # hip in base
    want = []
    for sx in (0.1, -0.1):
        hip = np.array([0, 0.02, 0]) + Rt.apply([sx, 0, -0.05])
        knee = hip + Rh.apply([0, -0.25, 0])
        for end in ([-0.06, -0.3, 0.0], [0.09, -0.3, 0.0]):
            want.append(base + knee + Rh.apply(end))
    np.testing.assert_allclose(got, want, atol=1e-12)
    np.testing.assert_allclose(m.sph_radius, 0.02)
    # hinge axes in the world: the two hips turn about opposite axes
    np.testing.assert_allclose(kin["xaxis"][2], Rh.apply([0, 0, 1]), atol=1e-12)
    np.testing.assert_allclose(kin["xaxis"][4], Rh.apply([0, 0, -1]), atol=1e-12)
    # and the loaded model runs: a forward pass with the feet 2 cm in the ground gives finite accelerations and 16 contact
    # rows + 4 friction rows (no joint is beyond its range at qpos0)
    orc = Oracle(m.arrays())
    d = orc.data()
    orc.forward(d)
    assert d.nefc == 16 + 4 and np.isfinite(d.qacc).all()


def test_outside_the_subset_raises(tmp_path):
    text = open(MINI).read()
    for old, new, msg in [('type="hinge" class="big" axis="0 0 1"', 'type="ball" class="big" axis="0 0 1"', "type ball"),
                          ('<geom name="foot_l" type="capsule"', '<geom name="foot_l" type="box"', "colliding box"),
                          ('<motor name="hip_l_m"', '<position name="hip_l_m"', "actuator <position>"),
                          ('<inertial pos="0 -0.1 0" mass="2" diaginertia="0.02 0.004 0.02" />\n          <body name="knee_l"',
                           '<body name="knee_l"', "without mass")]:
        assert old in text
        p = tmp_path / "bad.mjcf"
        p.write_text(text.replace(old, new, 1))
        with pytest.raises(ValueError, match=msg):
            load_mjcf(str(p))


@pytest.mark.skipif(not os.path.exists(KBOT), reason="the reference tree is not present")
def test_kbot_file_from_the_reference():
    """examples/kbot/robot/kbot-headless/robot.mjcf: 20 limited hinges with dry friction on a floating base, the torso and
    IMU bodies welded into the base, 4 collision capsules = 8 contact spheres.  The file puts the base at the height where
    all eight foot spheres sit 2 mm above the ground, which pins every frame composition of both legs."""
    m = load_mjcf(KBOT, dt=0.005, integrator="implicitfast")
    assert (m.nb, m.nq, m.nv, m.nu, m.ns) == (22, 27, 26, 20, 8)
    text = open(KBOT).read()
    masses = [float(x) for x in re.findall(r'<inertial[^>]*mass="([0-9.eE+-]+)"', text)]
    marker = 1000 * 4 / 3 * np.pi * 0.01**3   # the base's only geom: a 1 cm visual sphere
    assert m.body_mass.sum() == pytest.approx(sum(masses) + marker, rel=1e-12)
    assert m.jnt_limited[2:].all() and (m.dof_frictionloss[6:] > 0).all() and (m.dof_armature[6:] > 0).all()
    kin = km.host_kinematics(m.arrays(), m.qpos0)
    low = [kin["xpos"][b][2] + (kin["xmat"][b] @ p)[2] - r for b, p, r in zip(m.sph_body, m.sph_pos, m.sph_radius)]
    np.testing.assert_allclose(low, 0.002, atol=2e-6)
    assert m.friction == 0.64 and tuple(m.solref) == (0.02, 0.8)
    # the model runs in the oracle: standing at qpos0 a few steps under gravity with zero torque stays finite
    orc = Oracle(m.arrays())
    d = orc.data()
    for _ in range(20):
        orc.step(d)
    assert np.isfinite(d.qpos).all() and d.nefc >= 20


def test_sites_and_sensors_are_read_through_the_welds():
    m = load_mjcf(MINI)
    assert set(m.sites) == {"imu_site", "left_foot", "right_foot"}
    body, pos, quat = m.sites["imu_site"]   # on the welded torso: expressed in the base frame
    Rt = _rot([np.sqrt(0.5), 0, 0, np.sqrt(0.5)])
    assert body == 1
    np.testing.assert_allclose(pos, np.array([0, 0.02, 0]) + Rt.apply([0.02, -0.01, 0.3]), atol=1e-12)
    want = (Rt * _rot([0.9238795325112867, 0.3826834323650898, 0, 0])).as_quat()[[3, 0, 1, 2]]
    assert min(np.abs(np.array(quat) - want).max(), np.abs(np.array(quat) + want).max()) < 1e-12
    assert m.sites["left_foot"][0] == 3 and m.sites["right_foot"][0] == 5
    assert m.sensors == {"imu_acc": ("accelerometer", "imu_site"), "imu_gyro": ("gyro", "imu_site"),
                         "left_foot_touch": ("touch", "left_foot"), "right_foot_touch": ("touch", "right_foot"),
                         "imu_quat": ("framequat", "imu_site"), "left_foot_pos": ("framepos", "left_foot"),
                         "left_foot_angvel": ("frameangvel", "left_foot"), "imu_mag": ("magnetometer", "imu_site"),
                         "imu_vel": ("velocimeter", "imu_site")}
    assert m.magnetic == (0.1, -0.4, 0.2)
    from ksim_amd.observation import SensorObservation
    with pytest.raises(ValueError, match="not found"):
        SensorObservation.create(physics_model=m, sensor_name="nope")
    with pytest.raises(ValueError, match="not built"):
        SensorObservation.create(physics_model=m, sensor_name="imu_vel")
    assert SensorObservation.create(physics_model=m, sensor_name="imu_gyro").get_name() == "imu_gyro"


HUMANOID_MINI = os.path.join(HERE, "golden", "mini_humanoid.mjcf")
SCENE = "/root/reference/examples/data/scene.mjcf"


def test_mini_humanoid_several_hinges_on_one_body():
    """A body with three hinges becomes two massless bodies and the body itself; the joints act in file order, so the
    thigh's orientation is R_x(q1) R_z(q2) R_y(q3) about the common anchor, and everything below hangs from that."""
    m = load_mjcf(HUMANOID_MINI)
    assert (m.nb, m.nq, m.nv, m.nu, m.ns) == (10, 15, 14, 8, 2)
    names = list(m.body_names)
    assert names[2:5] == ["thigh_right#hip_x_right", "thigh_right#hip_z_right", "thigh_right"]
    assert m.body_mass[2] == 0 and m.body_mass[3] == 0 and m.body_mass[4] > 0
    # degrees -> radians, class ranges, springs (the knee's class switches its spring off), shared limit-row parameters
    np.testing.assert_allclose(m.jnt_range[2:6], np.deg2rad([[-30, 20], [-50, 40], [-120, 30], [-150, 5]]))
    np.testing.assert_allclose(m.dof_stiffness[6:10], [8, 8, 8, 0])
    np.testing.assert_allclose(m.dof_damping[6:10], [4, 4, 4, 0.3])
    np.testing.assert_allclose(m.dof_armature[6:], 0.02)
    assert tuple(m.dof_solref) == (0.02, 1.0) and tuple(m.dof_solimp) == (0.0, 0.99, 0.01, 0.5, 2.0)
    # the feet collide through their explicit pairs only, with a pair's own defaults (not the geoms' class values)
    assert list(m.sph_names) == ["foot_right", "foot_left"]
    assert m.friction == 1.0 and tuple(m.solref) == (0.02, 1.0) and tuple(m.solimp) == (0.9, 0.95, 0.001, 0.5, 2.0)
    # gears follow the motors to the bodies that carry their joints
    np.testing.assert_allclose(m.arrays()["act_gear"][:8], [40, 40, 120, 80] * 2)
    np.testing.assert_array_equal(m.arrays()["act_dof"][:8], np.arange(6, 14))

    rng = np.random.default_rng(5)
    q = m.qpos0.copy()
    q[7:] = rng.uniform(-0.5, 0.5, 8)
    kin = km.host_kinematics(m.arrays(), q)
    base = np.array([0, 0, 0.83])
    for side, sy, ax in ((0, -1.0, 1.0), (1, 1.0, -1.0)):
        a = q[7 + 4 * side: 11 + 4 * side]
        R = (Rotation.from_rotvec([ax * a[0], 0, 0]) * Rotation.from_rotvec([0, 0, ax * a[1]]) * Rotation.from_rotvec([0, a[2], 0]))
        thigh = 4 + 4 * side
        hip = base + np.array([0, 0.1 * sy, -0.04])
        np.testing.assert_allclose(kin["xpos"][thigh], hip, atol=1e-12)
        np.testing.assert_allclose(kin["xmat"][thigh], R.as_matrix(), atol=1e-12)
        # the knee turns about -y through an anchor 2 cm above the shin's origin
        Rk = R * Rotation.from_rotvec([0, -a[3], 0])
        anchor = hip + R.apply([0, -0.01 * sy, -0.4] + np.array([0, 0, 0.02]))
        shin = anchor - Rk.apply([0, 0, 0.02])
        np.testing.assert_allclose(kin["xpos"][thigh + 1], shin, atol=1e-12)
        foot = kin["xpos"][thigh + 1] + kin["xmat"][thigh + 1] @ m.sph_pos[side]
        np.testing.assert_allclose(foot, shin + Rk.apply([0, 0, -0.35]), atol=1e-12)


def test_mini_humanoid_inertia_from_class_geoms():
    """Masses from the geoms' volumes at the default density (sizes and end points partly from default classes), the
    foot's sphere welded into the shin, and the composite shin's centre of mass by hand."""
    m = load_mjcf(HUMANOID_MINI)
    cap = lambda r, length: 1000 * (np.pi * r * r * length + 4 / 3 * np.pi * r**3)  # noqa: E731
    ball = 1000 * 4 / 3 * np.pi * 0.05**3
    thigh = cap(0.05, np.hypot(0.01, 0.34))
    shin = cap(0.04, 0.3)
    assert m.body_mass[1] == pytest.approx(cap(0.08, 0.16), rel=1e-12)
    assert m.body_mass[4] == pytest.approx(thigh, rel=1e-12) and m.body_mass[8] == pytest.approx(thigh, rel=1e-12)
    assert m.body_mass[5] == pytest.approx(shin + ball, rel=1e-12)
    np.testing.assert_allclose(m.body_ipos[5], [0, 0, (shin * -0.15 + ball * -0.35) / (shin + ball)], atol=1e-12)
    np.testing.assert_allclose(m.body_ipos[4], [0, 0.005, -0.17], atol=1e-12)
    # the shin's inertia about its centre of mass: capsule + sphere through the parallel-axis theorem (z is the long axis)
    r, h = 0.04, 0.3
    mc, mh = 1000 * np.pi * r * r * h, 1000 * 4 / 3 * np.pi * r**3
    izz = mc * r * r / 2 + mh * 2 * r * r / 5
    ixx = mc * (r * r / 4 + h * h / 12) + mh * (2 * r * r / 5 + h * h / 4 + 3 * h * r / 8)
    zc = m.body_ipos[5][2]
    ixx_tot = ixx + shin * (zc + 0.15) ** 2 + ball * 2 / 5 * 0.05**2 + ball * (zc + 0.35) ** 2
    izz_tot = izz + ball * 2 / 5 * 0.05**2
    np.testing.assert_allclose(sorted(m.body_inertia[5]), sorted([ixx_tot, ixx_tot, izz_tot]), rtol=1e-10)


def test_mini_humanoid_runs_and_springs_pull_back():
    """The loaded model steps in the oracle; with gravity off and the base held high, a displaced hip joint accelerates
    back toward its reference angle at -k q / (effective inertia), sign checked per joint."""
    m = load_mjcf(HUMANOID_MINI, gravity=(0, 0, 0))
    orc = Oracle(m.arrays())
    q = m.qpos0.copy()
    q[2] = 3.0
    q[7 + 2] = 0.3    # right hip_y
    d = orc.data(qpos=q)
    orc.forward(d)
    assert d.nefc == 0
    assert d.qfrc_passive[6 + 2] == pytest.approx(-8 * 0.3, rel=1e-12) and d.qacc[6 + 2] < 0
    m = load_mjcf(HUMANOID_MINI)
    orc = Oracle(m.arrays())
    d = orc.data()
    for _ in range(40):
        orc.step(d)
    assert np.isfinite(d.qpos).all()


def test_mini_humanoid_outside_the_subset_raises(tmp_path):
    text = open(HUMANOID_MINI).read()
    for old, new, msg in [('<pair geom1="foot_left" geom2="floor" />', '<pair geom1="foot_left" geom2="foot_right" />', "floor plane"),
                          ('<pair geom1="foot_left" geom2="floor" />', '<pair geom1="foot_left" geom2="floor" condim="1" />', "condim"),
                          ('<joint pos="0 0 .02" axis="0 -1 0" range="-150 5" stiffness="0" />',
                           '<joint pos="0 0 .02" axis="0 -1 0" range="-150 5" stiffness="0" solimplimit=".5 .9 .01" />', "share"),
                          ('<joint name="hip_y_left" class="hip_y" />', '<joint name="hip_y_left" class="hip_y" springref="10" />', "springref")]:
        assert old in text
        p = tmp_path / "bad.mjcf"
        p.write_text(text.replace(old, new, 1))
        with pytest.raises(ValueError, match=msg):
            load_mjcf(str(p))


@pytest.mark.skipif(not os.path.exists(SCENE), reason="the reference tree is not present")
def test_walking_example_scene_from_the_reference():
    """examples/data/scene.mjcf, the humanoid of examples/walking.py: 17 hinges (abdomen 2+1, hips 3, shoulders 2) on a
    floating base, 17 motors, two foot spheres that meet the floor through explicit pairs."""
    m = load_mjcf(SCENE)
    assert (m.nb, m.nq, m.nv, m.nu, m.ns) == (19, 24, 23, 17, 2)
    assert list(m.sph_names) == ["foot_right", "foot_left"] and m.friction == 1.0
    assert m.jnt_limited[2:].all() and tuple(m.dof_solimp[:3]) == (0.0, 0.99, 0.01)
    np.testing.assert_allclose(m.dof_stiffness[6:9], [20, 10, 10])   # abdomen z (stiff class), y, x
    assert sum(n.count("#") for n in m.body_names) == 1 + 2 * 2 + 2 * 1
    kin = km.host_kinematics(m.arrays(), m.qpos0)
    # at qpos0 the feet hang straight below the hips: 1.4 - .26 - .165 - .04 - .4 - .39 above the floor
    for b, p in zip(m.sph_body, m.sph_pos):
        assert (kin["xpos"][b] + kin["xmat"][b] @ p)[2] == pytest.approx(1.4 - 0.26 - 0.165 - 0.04 - 0.4 - 0.39, abs=1e-12)
    orc = Oracle(m.arrays())
    d = orc.data()
    for _ in range(20):
        orc.step(d)
    assert np.isfinite(d.qpos).all()
