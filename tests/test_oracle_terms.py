"""Pins oracle/terms.py against the reference's own known-answer vectors (CPU only)."""
import itertools
import json
import os

import numpy as np
import pytest

from oracle import terms
from oracle import terms as ot

GOLD = os.path.join(os.path.dirname(__file__), "golden")
REWARD_KATS = json.load(open(os.path.join(GOLD, "reward_kats.json")))
TERM_KATS = json.load(open(os.path.join(GOLD, "termination_kats.json")))
FN = {"velocity": terms.action_velocity_penalty, "acceleration": terms.action_acceleration_penalty,
      "jerk": terms.action_jerk_penalty}


@pytest.mark.parametrize("kat", REWARD_KATS, ids=[k["ref"] for k in REWARD_KATS])
def test_reward_kats(kat):
    a = np.array(kat["actions"], dtype=np.float64)
    done = np.zeros(len(a), bool) if kat["done"] is None else np.array(kat["done"])
    got = FN[kat["fn"]](a, done, kat["norm"])
    np.testing.assert_allclose(got, kat["expected"], atol=kat["atol"], rtol=0)


@pytest.mark.parametrize("kat", TERM_KATS, ids=[f'{k["fn"]}-{i}' for i, k in enumerate(TERM_KATS)])
def test_termination_kats(kat):
    if kat["fn"] == "not_upright":
        got = terms.not_upright_termination(np.array(kat["qpos"]), kat["max_radians"])
    elif kat["fn"] == "minimum_height":
        got = terms.minimum_height_termination(np.array(kat["qpos"]), kat["min_height"])
    else:
        got = terms.illegal_contact_termination(kat["ncon"], np.array(kat["geom1"]), np.array(kat["geom2"]),
                                                np.array(kat["dist"]), np.array(kat["illegal"]))
    assert int(got) == kat["expected"]


def _q(x=0.0, y=0.0, z=0.0):
    q = np.zeros(9)
    q[:3] = x, y, z
    q[3] = 1.0
    return q


def test_bad_z_termination_hand_computed():
    """terminations.py:139-146: the bounds move linearly from (min_z, max_z) at level 0 to the final pair at level 1,
    both comparisons are strict, the value is always -1.  Expected values are written out by hand."""
    kw = dict(min_z=-1.0, max_z=2.0, final_min_z=0.0, final_max_z=1.0)
    # level 0: bounds (-1, 2); level 0.5: (-0.5, 1.5); level 1: (0, 1)
    cases = [
        (0.0, -1.25, -1), (0.0, -1.0, 0), (0.0, -0.75, 0), (0.0, 1.75, 0), (0.0, 2.0, 0), (0.0, 2.25, -1),
        (0.5, -0.75, -1), (0.5, -0.5, 0), (0.5, -0.25, 0), (0.5, 1.25, 0), (0.5, 1.5, 0), (0.5, 1.75, -1),
        (1.0, -0.25, -1), (1.0, 0.0, 0), (1.0, 0.25, 0), (1.0, 0.75, 0), (1.0, 1.0, 0), (1.0, 1.25, -1),
    ]
    for level, z, want in cases:
        assert int(ot.bad_z_termination(_q(z=z), level=level, **kw)) == want, (level, z)
    # a point that is healthy at level 0 and unhealthy at level 1 on either side tells the interpolation direction
    assert int(ot.bad_z_termination(_q(z=-0.5), level=0.0, **kw)) == 0 and int(ot.bad_z_termination(_q(z=-0.5), level=1.0, **kw)) == -1
    assert int(ot.bad_z_termination(_q(z=1.5), level=0.0, **kw)) == 0 and int(ot.bad_z_termination(_q(z=1.5), level=1.0, **kw)) == -1
    # without final bounds the level changes nothing; only the z coordinate matters
    for level in (0.0, 0.3, 1.0):
        assert int(ot.bad_z_termination(_q(x=9.0, y=-9.0, z=0.5), -1.0, 2.0, level)) == 0
        assert int(ot.bad_z_termination(_q(z=-1.5), -1.0, 2.0, level)) == -1
        assert int(ot.bad_z_termination(_q(z=2.5), -1.0, 2.0, level)) == -1
    # only one final bound given: the other stays where it was
    assert int(ot.bad_z_termination(_q(z=1.75), -1.0, 2.0, 1.0, final_min_z=0.0)) == 0
    assert int(ot.bad_z_termination(_q(z=-0.5), -1.0, 2.0, 1.0, final_min_z=0.0)) == -1
    got = ot.bad_z_termination(np.stack([_q(z=-2.0), _q(z=0.5), _q(z=3.0)]), -1.0, 2.0)
    assert got.dtype == np.int32 and got.tolist() == [-1, 0, -1]


def test_bad_velocity_termination_hand_computed():
    """terminations.py:155-157: Euclidean norm of the three linear root velocities only, strictly above the limit, -1."""
    v = np.zeros(8)
    v[:3] = 3.0, 4.0, 0.0  # |v| = 5 exactly
    assert int(ot.bad_velocity_termination(v, 5.0)) == 0  # on the limit: strict
    assert int(ot.bad_velocity_termination(v, 4.999)) == -1
    assert int(ot.bad_velocity_termination(v, 5.001)) == 0
    v[:3] = 0.0, -3.0, 4.0  # sign and axis do not matter
    assert int(ot.bad_velocity_termination(v, 4.999)) == -1
    v[:3] = 2.0, 2.0, 1.0  # |v| = 3: a norm, not a sum of magnitudes (5) nor a maximum (2)
    assert int(ot.bad_velocity_termination(v, 2.9)) == -1 and int(ot.bad_velocity_termination(v, 3.1)) == 0
    v[:3] = 0.1, 0.0, 0.0
    v[3:] = 100.0  # angular and joint velocities must not count
    assert int(ot.bad_velocity_termination(v, 1.0)) == 0
    got = ot.bad_velocity_termination(np.array([[3.0, 4.0, 0.0, 0, 0, 0], [3.0, 4.0, 0.1, 0, 0, 0]]), 5.0)
    assert got.dtype == np.int32 and got.tolist() == [0, -1]


def test_far_from_origin_termination_hand_computed():
    """terminations.py:170-172: norm of the root position (x, y, z) strictly above max_dist; +1 by default."""
    q = _q(3.0, 0.0, 4.0)  # distance 5 exactly; z counts
    assert int(ot.far_from_origin_termination(q, 5.0)) == 0
    assert int(ot.far_from_origin_termination(q, 4.999)) == 1  # default is a positive termination
    assert int(ot.far_from_origin_termination(q, 4.999, pos_termination=True)) == 1
    assert int(ot.far_from_origin_termination(q, 4.999, pos_termination=False)) == -1
    assert int(ot.far_from_origin_termination(q, 5.001, pos_termination=False)) == 0
    q = _q(-1.0, -2.0, 2.0)  # distance 3; the quaternion entries (w = 1) must not count
    assert int(ot.far_from_origin_termination(q, 2.9)) == 1 and int(ot.far_from_origin_termination(q, 3.05)) == 0
    got = ot.far_from_origin_termination(np.stack([_q(0.1), _q(0.0, 6.0)]), 5.0, pos_termination=False)
    assert got.dtype == np.int32 and got.tolist() == [0, -1]


def test_episode_length_termination_hand_computed():
    """terminations.py:186-192: time strictly above the limit; +1 by default; with disable_at_curriculum_level the term is
    off while the level is strictly below it."""
    assert int(ot.episode_length_termination(10.0, 10.0)) == 0  # on the limit: strict
    assert int(ot.episode_length_termination(10.005, 10.0)) == 1
    assert int(ot.episode_length_termination(9.995, 10.0)) == 0
    assert int(ot.episode_length_termination(10.005, 10.0, pos_termination=False)) == -1
    assert int(ot.episode_length_termination(9.995, 10.0, pos_termination=False)) == 0
    # disabled below level 2, active from level 2 on (the comparison is level < disable)
    for level, want in ((0.0, 0), (1.0, 0), (1.999, 0), (2.0, 1), (3.0, 1)):
        assert int(ot.episode_length_termination(10.005, 10.0, True, level, 2)) == want, level
        assert int(ot.episode_length_termination(10.005, 10.0, False, level, 2)) == -want, level
        assert int(ot.episode_length_termination(9.0, 10.0, True, level, 2)) == 0
    # a disable level of 0 never disables (no level is below it); None ignores the level altogether
    assert int(ot.episode_length_termination(10.005, 10.0, True, 0.0, 0)) == 1
    assert int(ot.episode_length_termination(10.005, 10.0, True, 0.0, None)) == 1
    got = ot.episode_length_termination(np.array([1.0, 11.0, 11.0]), 10.0, True, np.array([5.0, 5.0, 1.0]), 2)
    assert got.dtype == np.int32 and got.tolist() == [0, 1, 0]


def test_done_success_truth_table():
    for k in (1, 2, 3):
        for combo in itertools.product([-1, 0, 1], repeat=k):
            done, succ = terms.combine_terminations([np.array(c) for c in combo])
            assert bool(done) == any(c != 0 for c in combo)
            assert bool(succ) == (any(c != 0 for c in combo) and all(c != -1 for c in combo))


def test_rotate_vector_by_quat_against_scipy():
    from scipy.spatial.transform import Rotation

    rng = np.random.default_rng(0)
    q = rng.normal(size=(20, 4))
    v = rng.normal(size=(20, 3))
    R = Rotation.from_quat(q[:, [1, 2, 3, 0]])  # scipy is xyzw and normalises
    np.testing.assert_allclose(terms.rotate_vector_by_quat(v, q), R.apply(v), atol=1e-12)
    np.testing.assert_allclose(terms.rotate_vector_by_quat(v, q, inverse=True), R.inv().apply(v), atol=1e-12)


def test_latency_blend_cases():
    last, act = np.array([1.0, 2.0]), np.array([5.0, 6.0])
    nodrop = np.array([False, False])
    # latency 0: substep 0 still applies the previous ctrl, substep >= 1 the new action (engine.py:287-288)
    np.testing.assert_array_equal(terms.latency_blend(0.0, 0.0, last, act, nodrop), last)
    np.testing.assert_array_equal(terms.latency_blend(1.0, 0.0, last, act, nodrop), act)
    # latency >= S: never switches; fractional latency blends linearly
    for s in range(4):
        np.testing.assert_array_equal(terms.latency_blend(float(s), 4.0, last, act, nodrop), last)
    np.testing.assert_allclose(terms.latency_blend(1.0, 0.25, last, act, nodrop), last * 0.25 + act * 0.75)
    np.testing.assert_array_equal(terms.latency_blend(3.0, 0.0, last, act, np.array([True, False])), [1.0, 6.0])


def test_pd_actuator_and_scrub():
    tau = terms.position_actuator_torque(np.array([0.5, -2.0]), np.array([0.1, 0.0]), np.array([1.0, -1.0]),
                                         kp=np.array([20.0, 100.0]), kd=np.array([1.0, 2.0]), ctrl_clip=np.array([np.inf, 50.0]))
    np.testing.assert_allclose(tau, [20 * 0.4 - 1.0, -50.0])
    a = terms.scrub_action(np.array([np.nan, 2e3, -5.0, -1e9]))
    np.testing.assert_array_equal(a, [0.0, 1e3, -5.0, -1e3])


def test_simple_rewards():
    done = np.array([False, True, True]); succ = np.array([False, False, True])
    np.testing.assert_allclose(terms.stay_alive_reward(done, succ), [0.01, -1.0, 0.01])
    np.testing.assert_allclose(terms.stay_alive_reward(done, succ, success_reward=3.0), [0.01, -1.0, 3.0])
    q = np.zeros((2, 9)); q[:, 2] = [1.0, 1.5]; q[:, 3] = 1.0
    np.testing.assert_allclose(terms.base_height_reward(q, 1.0), [1.0, np.exp(-0.25 / (2 * 0.0625))])
    np.testing.assert_allclose(terms.base_height_range_reward(q, 0.8, 1.2, 2.0), [1.0, 0.4])
    up = terms.upright_reward(q, np.zeros((2, 8)))
    np.testing.assert_allclose(up["pose"], [1.0, 1.0])
    tot, comps = terms.total_reward({"a_reward": np.array([1.0, 2.0]), "b_penalty": np.array([4.0, 0.5])},
                                    {"a_reward": 2.0, "b_penalty": 0.5}, {"a_reward": False, "b_penalty": True},
                                    clip_min=0.5)
    np.testing.assert_allclose(tot, [0.5, 3.75])


def test_amp_reward_closed_form():
    # ksim/task/amp.py:111: a parabola with its apex (1) at logit 1, zero at logits -1 and 3, clamped outside
    np.testing.assert_allclose(terms.amp_reward([1.0, 3.0, -1.0, 5.0, -7.0, 0.0, 2.0]), [1.0, 0.0, 0.0, 0.0, 0.0, 0.75, 0.75])
    x = np.linspace(-4, 6, 101)
    np.testing.assert_allclose(terms.amp_reward(x), terms.amp_reward(2.0 - x))  # symmetric about logit 1
    assert (terms.amp_reward(x) >= 0).all() and terms.amp_reward(x).max() == 1.0


def test_velocity_events_closed_forms():
    # timer above dt: nothing happens, the timer runs down by the float32 timestep (events.py:77-78)
    imp, left = terms.velocity_event("linear", dict(linvel=1.0, vel_range=(0.0, 1.0), interval_range=(1.0, 2.0)), 0.5, 0.005, (0.1, 0.2, 0.3), 1.0)
    assert not imp.any() and left == float(np.float32(0.5) - np.float32(0.005))
    # firing: direction theta = 2 pi u0, magnitude linear in u1, next interval linear in u2, curriculum scale on top
    p = dict(linvel=2.0, vel_range=(0.5, 1.5), interval_range=(1.0, 3.0))
    imp, left = terms.velocity_event("linear", p, 0.004, 0.005, (0.25, 0.5, 0.75), 0.5)
    np.testing.assert_allclose(imp, [0.0, 2.0 * 1.0 * 0.5, 0.0, 0.0, 0.0, 0.0], atol=1e-15)   # theta = pi/2
    assert left == 2.5
    # angular push acts on qvel[5] only and is flipped when the Bernoulli(0.5) draw comes out true (u0 < 0.5)
    pa = dict(angvel=3.0, vel_range=(0.0, 1.0), interval_range=(0.0, 1.0))
    assert terms.velocity_event("angular", pa, 0.0, 0.005, (0.4, 1.0, 0.0), 1.0)[0][5] == -3.0
    assert terms.velocity_event("angular", pa, 0.0, 0.005, (0.6, 1.0, 0.0), 1.0)[0][5] == 3.0
    # jump: the impulse that reaches the height, v = sqrt(2 g h)
    pj = dict(jump_height_range=(0.1, 0.3), interval_range=(2.0, 2.0))
    imp, left = terms.velocity_event("jump", pj, 0.001, 0.005, (0.5, 0.0, 0.9), 1.0)
    np.testing.assert_allclose(imp[:3], [0.0, 0.0, np.sqrt(2 * 9.81 * 0.2)])
    v = imp[2]
    assert abs(v * v / (2 * 9.81) - 0.2) < 1e-12 and left == 2.0


def test_force_push_event_state_machine():
    """ForcePushEvent (ksim/events.py:240-365) step by step on hand-computed cases."""
    p = dict(max_force=10.0, max_torque=2.0, force_range=(0.5, 1.0), duration_range=(0.1, 0.3), interval_range=(1.0, 2.0))
    zero = np.zeros(6)
    # nothing held, interval not over: no force, both timers lose dt
    ap, (left, dur, w) = terms.force_push_event(p, (0.5, 0.0, zero), 0.005, np.zeros(10), 1.0)
    assert not ap.any() and not w.any() and left == float(np.float32(0.5) - np.float32(0.005)) and dur == float(-np.float32(0.005))
    # interval over: a new wrench is drawn but not yet applied in this substep; "both" case, unit directions
    u = np.array([1.0, 0.5, 0.5, 1.0, 0.5, 0.5, 0.0, 0.99, 0.5, 0.5])
    ap, (left, dur, w) = terms.force_push_event(p, (0.004, 0.0, zero), 0.005, u, 1.0)
    assert not ap.any()
    np.testing.assert_allclose(w, [10.0, 0, 0, 0, 0, -2.0], atol=1e-12)
    assert (left, dur) == (1.5, pytest.approx(0.2))
    # while the duration lasts the body gets the wrench; the magnitude is the drawn scale times the maximum
    ap, st = terms.force_push_event(p, (left, dur, w), 0.005, np.zeros(10), 1.0)
    np.testing.assert_allclose(ap, w)
    ap, _ = terms.force_push_event(p, (1.0, 0.004, w), 0.005, np.zeros(10), 1.0)
    assert not ap.any()  # duration ran out
    # force-only / torque-only cases and the scale of the magnitude
    for u7, keep in ((0.1, slice(0, 3)), (0.5, slice(3, 6))):
        u = np.array([0.9, 0.2, 0.6, 0.0, 0.3, 0.8, 0.1, u7, 0.0, 0.0])
        _, (_, _, w) = terms.force_push_event(p, (0.0, 0.0, zero), 0.005, u, 1.0)
        other = slice(3, 6) if keep == slice(0, 3) else slice(0, 3)
        assert not w[other].any()
        assert np.linalg.norm(w[keep]) == pytest.approx(0.5 * (10.0 if keep == slice(0, 3) else 2.0))
    # the curriculum scale multiplies the carried wrench every substep and once more when it is applied
    ap, (_, _, w2) = terms.force_push_event(p, (1.0, 0.1, np.ones(6)), 0.005, np.zeros(10), 0.5)
    np.testing.assert_allclose(w2, 0.5 * np.ones(6)); np.testing.assert_allclose(ap, 0.25 * np.ones(6))


def test_stateful_observations_closed_forms():
    from scipy.spatial.transform import Rotation
    # contact flags: negative distance = touching; block is (spheres per foot, 2 feet)
    c = terms.feet_contact_observation([-0.01, 0.2, 0.0, -1e-6], foot_left=(0, 1), foot_right=(2, 3))
    assert c.tolist() == [[1.0, 0.0], [0.0, 1.0]]
    # delay line: after the fill the output at step k is the input at step k - delay
    rng = np.random.default_rng(0)
    xs = rng.normal(size=(9, 4))
    carry = np.tile(xs[0], (3, 1))
    outs = []
    for k in range(1, 9):
        out, carry = terms.delayed_observation(carry, xs[k], zero_offset=np.full(4, 0.5))
        outs.append(out)
    np.testing.assert_allclose(outs[:3], np.tile(xs[0] - 0.5, (3, 1)))
    np.testing.assert_allclose(outs[3:], xs[1:6] - 0.5)
    # roll-pitch-yaw quaternion against scipy's extrinsic xyz composition
    for rpy in rng.uniform(-1, 1, size=(5, 3)):
        q = terms.euler_to_quat(rpy)
        want = Rotation.from_euler("xyz", rpy).as_quat()[[3, 0, 1, 2]]
        np.testing.assert_allclose(q * np.sign(q[0]), want * np.sign(want[0]), atol=1e-12)
    # exponential average of a constant reading: x_k = p (1 - lag^k); p = R_bias R_q^-1 g
    quat = Rotation.from_euler("xyz", [0.3, -0.2, 0.9]).as_quat()[[3, 0, 1, 2]]
    bias = np.array([0.05, -0.02, 0.01])
    p = Rotation.from_euler("xyz", bias).apply(Rotation.from_quat(quat[[1, 2, 3, 0]]).inv().apply([0, 0, -9.81]))
    x = np.zeros(3)
    for k in range(1, 6):
        x = terms.projected_gravity_ema(x, 0.7, bias, quat)
        np.testing.assert_allclose(x, p * (1 - 0.7**k), atol=1e-12)
    np.testing.assert_allclose(terms.projected_gravity_ema(np.ones(3), 0.0, np.zeros(3), [1, 0, 0, 0]), [0, 0, -9.81])


def test_feet_air_time_reward_hand_computed():
    """Two feet, one contact sphere each, air and ground phases of 2 and 3 steps; counters and rewards by hand."""
    #            t:  0  1  2  3  4  5  6
    left = np.array([1, 0, 0, 0, 1, 1, 1])    # left foot: down, three steps up, down
    right = np.ones(7, dtype=int)               # right foot always down
    contact = np.stack([left, right], axis=-1)[:, None, :].astype(float)
    qvel = np.zeros((7, 6)); qvel[:, 0] = 1.0   # moving
    qvel[5, 0] = 0.0                            # standing at t = 5
    done = np.zeros(7, bool); done[6] = True    # a finished step never counts as moving
    zero = (np.zeros(2, int),) * 3
    out, (air, gnd, sta) = terms.feet_air_time_reward(contact, qvel, done, zero, air_steps=2.0, gnd_steps=3.0, bias=0.1,
                                                     ground_penalty=0.25)
    # left air counter 0 1 2 3 0 0 0 -> reward cnt/2 + bias while cnt < 2, else 0; right foot never in the air: bias
    np.testing.assert_allclose(out["air"], [0.1, 0.6, 0.1, 0.1, 0.1, 0.1, 0.1])
    # ground counters: left 1 0 0 0 1 0 0, right 1 2 3 4 5 0 0; cnt/3 + bias while cnt < 3 else -penalty; max over feet
    np.testing.assert_allclose(out["gnd"], [1 / 3 + 0.1, 2 / 3 + 0.1, 0.1, 0.1, 1 / 3 + 0.1, 0.1, 0.1])
    # stationary counters only run while in contact and not moving: t=5 -> 1, t=6 (done) -> 2
    np.testing.assert_allclose(out["stationary_gnd"], [0.1, 0.1, 0.1, 0.1, 0.1, 1 / 3 + 0.1, 2 / 3 + 0.1])
    assert air.tolist() == [0, 0] and gnd.tolist() == [0, 0] and sta.tolist() == [2, 2]
    # the carry continues the count across rollouts; yaw rate alone counts as moving only when positive
    qv = np.zeros((1, 6)); qv[0, 5] = -1.0
    out2, (_, _, sta2) = terms.feet_air_time_reward(contact[:1], qv, np.zeros(1, bool), (air, gnd, sta), air_steps=2.0, gnd_steps=3.0)
    assert sta2.tolist() == [3, 3] and out2["stationary_gnd"][0] == 1.0
    # commands replace the measured velocity when named
    out3, (_, gnd3, _) = terms.feet_air_time_reward(contact[:1], qv, np.zeros(1, bool), zero, air_steps=2.0, gnd_steps=3.0,
                                                    lin_cmd_t=np.array([-0.5]), ang_cmd_t=np.array([0.0]))
    assert gnd3.tolist() == [1, 1]


def test_sparse_target_height_reward_hand_computed():
    #              t:  0    1    2    3    4    5
    z = np.array([0.0, 0.1, 0.3, 0.2, 0.0, 0.5])
    contact = np.array([1, 0, 0, 0, 1, 0])[:, None, None].astype(float)
    pos = np.zeros((6, 1, 3)); pos[:, 0, 2] = z
    qvel = np.zeros((6, 6)); qvel[:, 0] = 1.0
    out, best = terms.sparse_target_height_reward(contact, pos, qvel, np.zeros(6, bool), np.array([0.15]), height=0.25)
    # t=0: touching with a carried maximum of 0.15 -> reward 0.15, maximum reset; t=4: touch-down after a swing that
    # peaked at 0.3 -> capped at 0.25; t=5: in the air again, the maximum restarts from this height
    np.testing.assert_allclose(out, [0.15, 0, 0, 0, 0.25, 0])
    np.testing.assert_allclose(best, [0.5])
    # a robot that is not moving loses the running maximum
    qvel[3, 0] = 0.0
    out, _ = terms.sparse_target_height_reward(contact, pos, qvel, np.zeros(6, bool), np.array([0.0]), height=0.25)
    np.testing.assert_allclose(out, [0, 0, 0, 0, 0.0, 0])


def test_command_tracking_and_rest_rewards_hand_computed():
    k = lambda d, s=0.25, sq=0.1, ab=0.1: -ab * abs(d) - sq * d * d + np.exp(-d * d / (2 * s * s))  # noqa: E731
    # base yawed by 90 degrees: a world velocity of (0, 2, 0) is 2 m/s straight ahead in the robot frame
    q = np.zeros((1, 7)); q[0, 3:7] = [np.cos(np.pi / 4), 0, 0, np.sin(np.pi / 4)]
    v = np.zeros((1, 8)); v[0, :3] = [0.0, 2.0, 0.0]
    out = terms.linear_velocity_reward(q, v, np.array([[1.5, 0.1, 1.5, 0.0]]))
    assert out["vel"][0] == pytest.approx(k(0.5)) and out["x"][0] == pytest.approx(k(0.5))
    assert out["yaw"][0] == pytest.approx(k(-0.1)) and out["y"][0] == pytest.approx(k(0.0), abs=1e-12)
    out = terms.linear_velocity_reward(q, v, np.array([[0.005, 0.1, 1.5, 0.0]]))  # a zero command mutes all but "vel"
    assert (out["yaw"][0], out["x"][0], out["y"][0]) == (0.0, 0.0, 0.0) and out["vel"][0] == pytest.approx(k(1.995))
    v[0, 5] = 0.3
    a = terms.angular_velocity_reward(v, np.array([0.5]))
    assert a["mag"][0] == pytest.approx(k(-0.2)) and a["dir"][0] == 1.0
    assert terms.angular_velocity_reward(v, np.array([-0.5]))["dir"][0] == -1.0
    assert terms.angular_velocity_reward(v, np.array([0.01]))["dir"][0] == -1.0   # command inside the dead band, robot turning
    v[0, 5] = 0.01
    assert terms.angular_velocity_reward(v, np.array([0.02]))["dir"][0] == 1.0    # both inside the dead band
    v[0, 2], v[0, 4], v[0, 5] = 0.25, 0.5, 0.0
    o = terms.off_axis_velocity_reward(v)
    assert o["linz"][0] == pytest.approx(np.exp(-0.5)) and o["angx"][0] == pytest.approx(np.exp(-2.0)) and o["angy"][0] == 1.0
    v[0, :3] = [0.3, 0.0, 0.0]; v[0, 6:] = [3.0, 4.0]
    assert terms.motionless_at_rest_penalty(v)[0] == 5.0
    v[0, 0] = 0.6
    assert terms.motionless_at_rest_penalty(v)[0] == 0.0
    f = np.array([[[3.0, 4.0, 0.0], [0.0, 0.0, 12.0]]])
    assert terms.force_penalty(f, expected_weight=5.0, bias=2.0)[0] == pytest.approx(4.0)   # ((12 - 2) / 5)^2
    assert terms.force_penalty(f * 0.1, expected_weight=5.0, bias=2.0)[0] == 0.0


def test_velocity_commands_hand_computed():
    p = dict(min_vel=0.5, max_vel=1.5, max_yaw=0.4, zero_prob=0.2, backward_prob=0.3, switch_prob=0.1, ctrl_dt=0.02,
             linear_accel=2.0, angular_accel=1.0)
    q = np.zeros(7); q[3:7] = [np.cos(np.pi / 4), 0, 0, np.sin(np.pi / 4)]   # yawed by 90 degrees
    v = np.zeros(8); v[:3] = [0.0, 2.0, 0.0]                                 # 2 m/s straight ahead in the robot frame
    # episode start: measured speed / heading, fresh targets
    c = terms.linear_velocity_command(np.zeros(6), q, v, [0.75, 0.25, 0.9, 0.9, 0.9], True, **p)
    np.testing.assert_allclose(c, [2.0, 0.0, 2.0, 0.0, 1.25, -0.2], atol=1e-12)
    # ordinary step: the current values slew towards the targets, limited by the accelerations
    c2 = terms.linear_velocity_command(c, q, v, [0.0, 0.0, 0.9, 0.9, 0.9], False, **p)
    np.testing.assert_allclose(c2[:2], [2.0 - 0.75 * 0.02, -0.2 * 0.02], atol=1e-12)
    np.testing.assert_allclose(c2[2:4], [c2[0] * np.cos(c2[1]), c2[0] * np.sin(c2[1])])
    assert tuple(c2[4:]) == (1.25, -0.2)
    big = terms.linear_velocity_command([0.0, 0.0, 0.0, 0.0, 9.0, -9.0], q, v, [0, 0, 0, 0, 0.9], False, **p)
    np.testing.assert_allclose(big[:2], [2.0 * 0.02, -1.0 * 0.02])           # clipped slew
    # switch: new targets, current values kept (not measured, not slewed); zero and backward draws
    c3 = terms.linear_velocity_command(c2, q, v, [0.5, 0.5, 0.9, 0.1, 0.05], False, **p)
    np.testing.assert_allclose(c3, [c2[0], c2[1], c2[2], c2[3], -1.0, 0.0], atol=1e-12)
    c4 = terms.linear_velocity_command(c2, q, v, [0.5, 0.9, 0.1, 0.1, 0.05], False, **p)
    assert tuple(c4[4:]) == (0.0, 0.0)
    pa = dict(max_vel=1.0, min_vel=0.2, zero_prob=0.1, switch_prob=0.3, ctrl_dt=0.02, angular_accel=0.5)
    v[5] = 0.3
    a = terms.angular_velocity_command([0.0, 0.0], v, [0.5, 0.4, 0.9, 0.9], True, **pa)
    np.testing.assert_allclose(a, [0.3, -0.6])
    a2 = terms.angular_velocity_command(a, v, [0, 0, 0, 0.9], False, **pa)
    np.testing.assert_allclose(a2, [0.3 - 0.5 * 0.02, -0.6])
    a3 = terms.angular_velocity_command(a2, v, [0.5, 0.6, 0.05, 0.1], False, **pa)   # switch: re-measured, zeroed target
    np.testing.assert_allclose(a3, [0.3, 0.0])


def test_position_velocity_actuator_hand_computed():
    tau = terms.position_velocity_actuator_torque([0.5, -0.2, 1.0, 0.0], np.array([0.1, 0.1]), np.array([0.5, -1.0]),
                                                  kp=[10.0, 20.0], kd=[2.0, 1.0], ctrl_clip=[100.0, 5.5])
    np.testing.assert_allclose(tau, [10 * 0.4 + 2 * 0.5, np.clip(20 * -0.3 + 1 * 1.0, -5.5, 5.5)])
    # zero velocity targets reduce it to the position actuator
    a = terms.position_velocity_actuator_torque([0.5, -0.2, 0.0, 0.0], np.array([0.1, 0.1]), np.array([0.5, -1.0]), [10.0, 20.0], [2.0, 1.0], [100.0, 100.0])
    b = terms.position_actuator_torque(np.array([0.5, -0.2]), np.array([0.1, 0.1]), np.array([0.5, -1.0]), np.array([10.0, 20.0]), np.array([2.0, 1.0]), np.array([100.0, 100.0]))
    np.testing.assert_allclose(a, b)


def test_mixture_head_against_scipy_and_special_cases():
    """The mixture-of-Gaussians head: log-density against scipy, unit mass, component frequencies of the inverse CDF, the
    K = 1 reduction to the Gaussian head, the most probable component when deterministic."""
    from scipy.special import logsumexp, softmax
    from scipy.stats import norm

    rng = np.random.default_rng(31)
    N, nu, K = 40, 5, 3
    raw = rng.normal(size=(N, 3 * nu * K)) * 1.5
    bias = rng.normal(size=nu) * 0.2
    lo, hi = -np.ones(nu) * 0.8, np.ones(nu) * 1.1
    u, z = rng.random((N, nu)), rng.normal(size=(N, nu))
    kw = dict(min_std=0.01, max_std=1.0, var_scale=0.5, mean_bias=bias, clip_lo=lo, clip_hi=hi)
    act, logp, comp = terms.mixture_head(raw, K, uniform=u, normal=z, **kw)
    mean = np.clip(raw[:, :nu * K].reshape(N, nu, K) + bias[None, :, None], lo[None, :, None], hi[None, :, None])
    std = np.minimum((np.log1p(np.exp(raw[:, nu * K:2 * nu * K].reshape(N, nu, K))) + 0.01) * 0.5, 1.0)
    w = softmax(raw[:, 2 * nu * K:].reshape(N, nu, K), axis=-1)
    # component: the interval of the cumulative weights that holds the draw
    cum = np.cumsum(w, -1)
    for e, j in itertools.product(range(N), range(nu)):
        k = int(np.searchsorted(cum[e, j], u[e, j], side="right"))
        assert comp[e, j] == min(k, K - 1)
    sample = np.take_along_axis(mean, comp[..., None], -1)[..., 0] + np.take_along_axis(std, comp[..., None], -1)[..., 0] * z
    np.testing.assert_allclose(act, sample, rtol=1e-12)
    want = logsumexp(np.log(w) + norm.logpdf(sample[..., None], mean, std), axis=-1)
    np.testing.assert_allclose(logp, want, rtol=1e-10, atol=1e-10)
    # the density integrates to one (one env, one joint, fine grid)
    xs = np.linspace(-8, 8, 40001)
    dens = (w[0, 0][None] * norm.pdf(xs[:, None], mean[0, 0][None], std[0, 0][None])).sum(-1)
    assert np.sum(dens) * (xs[1] - xs[0]) == pytest.approx(1.0, abs=1e-6)
    # K = 1: a Gaussian with that mean and deviation, whatever the logit
    raw1 = rng.normal(size=(N, 3 * nu))
    a1, l1, c1 = terms.mixture_head(raw1, 1, uniform=u, normal=z, min_std=0.02, max_std=50.0)
    s1 = np.log1p(np.exp(raw1[:, nu:2 * nu])) + 0.02
    np.testing.assert_allclose(a1, raw1[:, :nu] + s1 * z, rtol=1e-12)
    np.testing.assert_allclose(l1, norm.logpdf(a1, raw1[:, :nu], s1), rtol=1e-10)
    assert (c1 == 0).all()
    # deterministic: the mean of the heaviest component; scrub and clip
    ad, _, cd = terms.mixture_head(raw, K, deterministic=True, **kw)
    assert (cd == np.argmax(w, -1)).all()
    np.testing.assert_allclose(ad, np.take_along_axis(mean, cd[..., None], -1)[..., 0])
    rawn = raw.copy(); rawn[0, 0:K] = np.nan
    an, _, _ = terms.mixture_head(rawn, K, uniform=u, normal=z, clip_max=0.5, **kw)
    assert an[0, 0] == 0.0 and np.abs(an).max() <= 0.5
    # frequencies: many draws pick component k with probability w_k
    big = np.tile(raw[:1], (20000, 1))
    _, _, cb = terms.mixture_head(big, K, uniform=rng.random((20000, nu)), normal=np.zeros((20000, nu)), **kw)
    freq = np.stack([(cb == k).mean(0) for k in range(K)], -1)
    assert np.abs(freq - w[0]).max() < 0.015


def test_action_filters_closed_forms():
    """Low-pass: step response x (1 - (1 - alpha)^k) and the -3 dB meaning of alpha; acceleration clip: reaches a reachable
    target exactly in one step, ramps at the bound otherwise; the integrators against constant-rate kinematics."""
    dt, fc = 0.02, 3.0
    alpha = dt / (1 / (2 * np.pi * fc) + dt)
    y = np.zeros(3)
    for k in range(1, 30):
        y = terms.lowpass_one_pole(np.array([1.0, -2.0, 0.5]), y, dt, fc)
        np.testing.assert_allclose(y, np.array([1.0, -2.0, 0.5]) * (1 - (1 - alpha) ** k), rtol=1e-12)
    assert alpha == pytest.approx(0.2737, abs=1e-4)  # dt / (RC + dt) with RC = 1 / (2 pi 3 Hz) = 53.05 ms
    # acceleration clip: from rest, a target 1 mm away needs a = x / dt^2 = 2.5 <= 10 -> reached exactly, at velocity x / dt
    p, v = terms.clip_acceleration(np.array([0.001]), np.zeros(1), np.zeros(1), 10.0, dt)
    assert p[0] == pytest.approx(0.001) and v[0] == pytest.approx(0.05)
    # a far target: constant acceleration at the bound, p_k = a dt^2 k (k + 1) / 2
    p, v = np.zeros(1), np.zeros(1)
    for k in range(1, 8):
        p, v = terms.clip_acceleration(np.array([5.0]), p, v, 10.0, dt)
        assert v[0] == pytest.approx(10.0 * dt * k) and p[0] == pytest.approx(10.0 * dt * dt * k * (k + 1) / 2)
    # integrators
    p = np.array([0.3])
    for k in range(1, 6):
        p = terms.integrate_velocity(np.array([2.0]), p, dt)
        assert p[0] == pytest.approx(0.3 + 2.0 * dt * k)
    p, v = np.zeros(1), np.zeros(1)
    for k in range(1, 40):
        p, v = terms.integrate_acceleration(np.array([20.0]), p, v, dt, max_velocity=5.0)
        assert v[0] == pytest.approx(min(20.0 * dt * k, 5.0))
    assert v[0] == 5.0
    # ranges: clip, and tanh with its inverse bias
    lo, hi = np.array([-1.0, 0.0]), np.array([2.0, 0.5])
    np.testing.assert_allclose(terms.clip_positions(np.array([[-3.0, 0.2], [5.0, 0.7]]), lo, hi), [[-1.0, 0.2], [2.0, 0.5]])
    zeros = np.array([0.5, 0.1])
    bias = np.arctanh((zeros - lo) / (hi - lo))
    np.testing.assert_allclose(terms.tanh_positions(bias, lo, hi), zeros, rtol=1e-12)


def test_site_sensors_against_rigid_motion():
    """Gyro and accelerometer at a site of a floating base: scipy rotations, the free joint's own body-frame angular
    velocity, the reading at rest, and a central second difference of the site's world position along an analytic rigid
    motion (constant linear acceleration, angular velocity w0 + alpha t in body axes)."""
    from scipy.spatial.transform import Rotation as R

    rng = np.random.default_rng(91)
    q0 = rng.normal(size=4); q0 /= np.linalg.norm(q0)
    qs = rng.normal(size=4); qs /= np.linalg.norm(qs)
    Rb, Rs = R.from_quat(q0[[1, 2, 3, 0]]), R.from_quat(qs[[1, 2, 3, 0]])
    w_l, al_l, a0 = rng.normal(size=3), rng.normal(size=3) * 2, rng.normal(size=3) * 3
    r_s = np.array([0.05, -0.02, 0.4])
    g = np.array([0.0, 0.0, -9.81])
    w_world = Rb.apply(w_l)
    # gyro: body-frame angular velocity (what the free joint's qvel[3:6] holds), turned into the site frame
    np.testing.assert_allclose(terms.site_gyro(q0, w_world, qs), Rs.inv().apply(w_l), atol=1e-12)
    np.testing.assert_allclose(terms.site_gyro(q0, w_world, [1, 0, 0, 0]), w_l, atol=1e-12)
    # at rest the accelerometer reads minus gravity in its own frame
    rest = terms.site_accelerometer(np.zeros(6), q0, np.zeros(3), r_s, qs, g)
    np.testing.assert_allclose(rest, (Rb * Rs).inv().apply([0, 0, 9.81]), atol=1e-12)
    # moving: second difference of p(t) = x(t) + R(t) r_s
    def p(t):
        rot = Rb * R.from_rotvec(w_l * t + 0.5 * al_l * t * t)   # exact to O(t^3)
        return 0.5 * a0 * t * t + rot.apply(r_s)
    h = 1e-4
    acc_fd = (p(h) - 2 * p(0.0) + p(-h)) / h**2
    want = (Rb * Rs).inv().apply(acc_fd - g)
    got = terms.site_accelerometer(np.concatenate([a0, al_l]), q0, w_world, r_s, qs, g)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    # dropped terms would show: centripetal and tangential parts are both far above the tolerance here
    assert np.linalg.norm(np.cross(w_world, np.cross(w_world, Rb.apply(r_s)))) > 0.05 and np.linalg.norm(np.cross(Rb.apply(al_l), Rb.apply(r_s))) > 0.05


def test_joint_and_link_smoothness_hand_computed():
    """Polynomial motions have constant differences: a ramp a constant velocity, a parabola a constant acceleration, a cubic
    a constant jerk; the edge padding makes the first `order` values build up from zero and a done step restarts that."""
    T = 8
    t = np.arange(T, dtype=np.float64)
    base = np.tile([0, 0, 1, 1, 0, 0, 0.0], (T, 1))
    done = np.zeros(T, bool)
    k = lambda x, s=0.25: np.exp(-x * x / (2 * s * s))  # noqa: E731
    ramp = np.concatenate([base, np.stack([0.1 * t, -0.2 * t], axis=1)], axis=1)
    want = np.full(T, (k(0.1) + k(0.2)) / 2); want[0] = 1.0
    np.testing.assert_allclose(ot.small_joint_reward(ramp, done, 1), want, rtol=1e-12)
    par = np.concatenate([base, (0.05 * t * t)[:, None]], axis=1)    # second difference 0.1 from t = 2; at t = 1: v(1) - 0 = 0.05
    want = np.full(T, k(0.1)); want[0] = 1.0; want[1] = k(0.05)
    np.testing.assert_allclose(ot.small_joint_reward(par, done, 2), want, rtol=1e-12)
    cub = np.concatenate([base, (0.01 * t**3)[:, None]], axis=1)    # third difference 0.06 from t = 3
    got = ot.small_joint_reward(cub, done, 3)
    np.testing.assert_allclose(got[3:], k(0.06), rtol=1e-9)
    np.testing.assert_allclose(got[:3], [1.0, k(0.01), k(0.08 - 3 * 0.01)], rtol=1e-9)  # x(1); x(2) - 3 x(1)
    # a done step at t = 3 zeroes the differences taken across it: velocity at t = 4, acceleration at t = 4 (zeroed) and at
    # t = 5 (v(5) - 0)
    done[3] = True
    got = ot.small_joint_reward(ramp, done, 1)
    assert got[4] == 1.0 and got[5] == pytest.approx((k(0.1) + k(0.2)) / 2)
    got = ot.small_joint_reward(par, done, 2)
    v5 = 0.05 * (25 - 16)
    assert got[4] == 1.0 and got[5] == pytest.approx(k(v5)) and got[6] == pytest.approx(k(0.1))
    # links: body 1 moves along a diagonal with quadratic arc length, body 0 (the world) is skipped
    done[:] = False
    s = 0.05 * t * t
    xpos = np.zeros((T, 3, 3))
    xpos[:, 1] = s[:, None] * np.array([0.6, 0.0, 0.8])
    xpos[:, 2] = (0.3 * t)[:, None] * np.array([0.0, 1.0, 0.0])    # constant speed: no acceleration after the build-up
    acc = ot.link_smoothness_penalty(xpos, done, 2, "l1")
    np.testing.assert_allclose(acc[2:], (0.1 + 0.0) / 2, rtol=1e-9)
    np.testing.assert_allclose(acc[:2], [0.0, (0.05 + 0.3) / 2], rtol=1e-9)
    jerk = ot.link_smoothness_penalty(xpos, done, 3, "l2")
    np.testing.assert_allclose(jerk[3:], 0.0, atol=1e-20)
    # t = 1: jerk = acc(1) = speed(1); t = 2: acc(2) - acc(1)
    np.testing.assert_allclose(jerk[:3], [0.0, (0.05**2 + 0.3**2) / 2, ((0.1 - 0.05) ** 2 + (0.0 - 0.3) ** 2) / 2], rtol=1e-9)


def test_joint_space_penalties_hand_computed():
    q = np.array([[0, 0, 1, 1, 0, 0, 0, 0.5, -1.2, 0.0], [0, 0, 1, 1, 0, 0, 0, 1.3, 0.2, -0.4]])
    lim = np.array([[-1.0, 1.0], [-1.0, 1.0], [-np.inf, np.inf]])
    np.testing.assert_allclose(ot.avoid_limits_penalty(q, lim), [0.2 / 3, 0.3 / 3], rtol=1e-12)
    # create: 5 % of the range on each side, unlimited joints never penalised, the free joint's row dropped
    made = ot.avoid_limits_create(np.array([[0, 0], [-1, 1], [0, 2], [0, 0]]), np.array([False, True, True, False]), factor=0.05)
    np.testing.assert_allclose(made, [[-1.1, 1.1], [-0.1, 2.1], [-np.inf, np.inf]])
    ctrl = np.array([[2.0, -1.0, 0.5], [0.0, 4.0, -3.0]])
    np.testing.assert_allclose(ot.torque_penalty(ctrl, (2.0, 1.0, 0.5)), [1.0, (4 + 6) / 3], rtol=1e-12)
    qvel = np.array([[0] * 6 + [1.0, -2.0, 0.0], [0] * 6 + [3.0, 0.5, -1.0]])
    np.testing.assert_allclose(ot.energy_penalty(ctrl, qvel, (2.0, 1.0, 0.5)), [(1 + 2 + 0) / 3, (0 + 2 + 6) / 3], rtol=1e-12)
    np.testing.assert_allclose(ot.joint_deviation_penalty(q, (2, 0), (0.1, 0.0), (2.0, 1.0), "l2"), [0.04 + 0.25, 1.0 + 1.69], rtol=1e-12)
    np.testing.assert_allclose(ot.joint_deviation_penalty(q, (1,), (0.2,), None, "l1"), [1.4, 0.0], atol=1e-15)


def test_body_frame_rewards_hand_computed():
    from scipy.spatial.transform import Rotation

    def wxyz(r):
        x, y, z, w = r.as_quat()
        return np.array([w, x, y, z])

    # a body tilted by angle a about any horizontal axis sees the vertical at cos a
    a, b = 0.4, 1.1
    xquat = np.zeros((1, 3, 4)); xquat[0, 0] = [1, 0, 0, 0]
    xquat[0, 1] = wxyz(Rotation.from_rotvec([a, 0, 0])); xquat[0, 2] = wxyz(Rotation.from_rotvec([0, b, 0]) * Rotation.from_rotvec([0, 0, 0.7]))
    np.testing.assert_allclose(ot.flat_body_reward(xquat, (1, 2)), [(np.cos(a) + np.cos(b)) / 2], rtol=1e-12)
    np.testing.assert_allclose(ot.flat_body_reward(xquat, (0,), plane=(1.0, 0, 0)), [1.0], rtol=1e-12)
    # a base rolled by phi about its x axis: roll = -phi; the yaw before it does not matter
    phi = 0.3
    q = np.zeros((1, 7)); q[0, 3:7] = wxyz(Rotation.from_rotvec([0, 0, 1.0]) * Rotation.from_rotvec([phi, 0, 0]))
    v = np.zeros((1, 6)); v[0, 3] = -0.5
    k = lambda x: np.exp(-x * x / (2 * 0.25**2)) - 0.1 * abs(x) - 0.1 * x * x  # noqa: E731
    ang, pose = ot.no_roll_reward(q, v)
    np.testing.assert_allclose([ang[0], pose[0]], [k(0.5), k(phi)], rtol=1e-12)
    # position tracking: offset (0.3, -0.1, 0.5) against a command (0.2, 0.1, 0.5): l1 error 0.3, l2 "norm" 0.01 + 0.04
    xpos = np.zeros((1, 3, 3)); xpos[0, 1] = [1, 1, 1]; xpos[0, 2] = [1.3, 0.9, 1.5]
    cmd = np.array([[0.2, 0.1, 0.5, 9.0]])
    np.testing.assert_allclose(ot.position_tracking_reward(xpos, cmd, 2, 1, "l1", 0.25), [np.exp(-0.3**2 / (2 * 0.25**2))], rtol=1e-12)
    np.testing.assert_allclose(ot.position_tracking_reward(xpos, cmd, 2, 1, "l2", 0.25), [np.exp(-0.05**2 / (2 * 0.25**2))], rtol=1e-12)
    # feet slip: only the foot with a contact flag set counts
    contact = np.array([[[0.0, 1.0], [0.0, 0.0]]])    # (T, c = 2, n = 2)
    vel = np.array([[[1, 2, 2, 0, 0, 0], [3, 0, 4, 0, 0, 12.0]]])
    np.testing.assert_allclose(ot.feet_slip_penalty(contact, vel), [13.0], rtol=1e-12)


def test_start_pose_and_base_height_commands_hand_computed():
    q = np.array([1.0, 2.0, 3.0, 0.5, 0.5, 0.5, 0.5, 9.0])
    np.testing.assert_array_equal(ot.start_pose_command([0, 0, 0], q, True), [1, 2, 3])
    np.testing.assert_array_equal(ot.start_pose_command([7, 7, 7], q, False), [7, 7, 7])
    np.testing.assert_array_equal(ot.start_pose_command([0] * 4, q, True, quaternion=True), [0.5] * 4)
    kw = dict(min_height=0.5, max_height=1.5, switch_prob=0.1)
    assert ot.base_height_command(0.8, 0.75, True, **kw) == 1.25          # episode start: always a new height
    assert ot.base_height_command(0.8, 0.75, False, **kw) == 0.8          # draw above switch_prob: kept
    assert ot.base_height_command(0.8, 0.04, False, **kw) == pytest.approx(0.54)   # the same draw picks the height


def test_reachability_and_intersection_hand_computed():
    q = np.array([[0, 0, 1, 1, 0, 0, 0, 0.5, -0.2]])
    a = np.array([[0.9, -0.25]])
    np.testing.assert_allclose(ot.reachability_penalty(a, q, (0.1, 0.1)), [0.3**2], rtol=1e-12)
    np.testing.assert_allclose(ot.reachability_penalty(a, q, (0.1, 0.01), squared=False), [0.3 + 0.04], rtol=1e-12)
    pts = np.array([[[0, 0, 0], [0.3, 0, 0], [0, 0.05, 0]], [[0, 0, 0], [0.3, 0, 0], [0, 0.5, 0]]], dtype=float)
    np.testing.assert_array_equal(ot.intersection_penalty(pts, 0.1), [1.0, 0.0])
    np.testing.assert_array_equal(ot.intersection_penalty(pts[:, :1], 0.1), [0.0, 0.0])   # a point is never too close to itself


def test_sinusoidal_gait_command_and_reward_hand_computed():
    kw = dict(gait_period=0.4, ctrl_dt=0.1, max_height=0.2, height_offset=0.01, num_feet=2, stance_ratio=0.5, moving_threshold=0.05)
    v = np.array([0.3, 0.0, 0, 0, 0, 0])
    c = ot.sinusoidal_gait_command(None, v, True, **kw)
    # phase 0: foot 0 in stance, foot 1 at phase 0.5 = start of its swing (sin 0 = 0)
    np.testing.assert_allclose(c, [1, 0, 0.01, 0.01], atol=1e-15)
    c = ot.sinusoidal_gait_command(c, v, False, **kw)
    # phase 0.25: foot 1 at 0.75 = the middle of its swing
    np.testing.assert_allclose(c, [1, 0.25, 0.01, 0.21], atol=1e-15)
    c = ot.sinusoidal_gait_command(c, v, False, **kw)
    c = ot.sinusoidal_gait_command(c, v, False, **kw)
    np.testing.assert_allclose(c, [1, 0.75, 0.21, 0.01], atol=1e-12)      # foot 0 mid-swing, foot 1 back in stance (phase 0.25)
    c = ot.sinusoidal_gait_command(c, v, False, **kw)
    np.testing.assert_allclose(c[:2], [1, 0.0], atol=1e-12)               # wrapped
    c = ot.sinusoidal_gait_command(c, np.array([0.01, 0.02, 0, 0, 0, 0]), False, **kw)
    np.testing.assert_allclose(c, [0, 0, 0.01, 0.01], atol=1e-15)         # standing still: flag and phase drop
    c = ot.sinusoidal_gait_command(c, v, False, **kw)
    np.testing.assert_allclose(c[:2], [0, 0], atol=1e-15)                 # and the flag stays down while the episode lasts
    pos = np.array([[[0, 0, 0.05], [0, 0, 0.2]]])
    np.testing.assert_allclose(ot.sinusoidal_gait_reward(pos, np.array([[0.01, 0.21]]), 0.2), [1 - (0.04 + 0.01) / 0.2], rtol=1e-12)


def test_random_variables_noise_and_bias_hand_computed():
    """ksim/noise.py:74-229 and Observation.add_noise (ksim/observation.py:110-142) on hand-computed numbers."""
    from scipy import stats

    # uniform: U(mean - mag level, mean + mag level); u = +-1 are the ends, u = 0 the mean
    assert ot.random_variable(2.0, 0.5, 0.0, 1.0, 0.0, level=0.5) == pytest.approx(2.25)
    assert ot.random_variable(2.0, 0.5, 0.0, -1.0, 0.0, level=0.5) == pytest.approx(1.75)
    # gaussian: z std level + mean
    assert ot.random_variable(1.0, 0.0, 0.2, 0.7, -1.5, level=0.5) == pytest.approx(1.0 - 0.15)
    # level 0 leaves the mean whatever the draws
    assert ot.random_variable(3.0, 1.0, 1.0, 0.3, 0.4, level=0.0) == pytest.approx(3.0)
    # one key for both parts: the uniform part is 2 Phi(z) - 1 (scipy's normal CDF, not the oracle's erf)
    z = np.array([-2.0, -0.3, 0.0, 1.1])
    np.testing.assert_allclose(ot.same_key_uniform(z), 2 * stats.norm.cdf(z) - 1, rtol=0, atol=1e-15)
    got = ot.random_variable(0.5, 0.2, 0.1, 99.0, z, level=1.0, same_key=True)  # the explicit uniform is ignored
    np.testing.assert_allclose(got, 0.5 + 0.1 * z + 0.2 * (2 * stats.norm.cdf(z) - 1), atol=1e-15)
    # ... and it is uniform on (-1, 1) when z is standard normal
    zz = np.random.default_rng(3).normal(size=20000)
    assert stats.kstest(ot.same_key_uniform(zz), stats.uniform(-1, 2).cdf).pvalue > 1e-3
    # additive / multiplicative noise; multiplicative means default to 1 in the reference (noise.py:201-213)
    assert ot.apply_noise(2.0, "add_gaussian", 0.0, 0.1, 1.5, 0.0, 1.0) == pytest.approx(2.15)
    assert ot.apply_noise(2.0, "mul_uniform", 1.0, 0.1, 0.0, -1.0, 0.5) == pytest.approx(2.0 * 0.95)
    assert ot.apply_noise(2.0, "mul_gaussian", 1.0, 0.1, 2.0, 0.0, 1.0) == pytest.approx(2.4)
    assert ot.apply_noise(2.0, "add_uniform", 0.1, 0.2, 0.0, 0.5, 1.0) == pytest.approx(2.2)
    assert ot.apply_noise(2.0, "add_uniform_gaussian", 0.0, 0.1, 1.0, 0.5, 1.0, 0.4) == pytest.approx(2.0 + 0.1 + 0.2)
    assert ot.apply_noise(2.0, "none", 0.0, 0.0, 1.0, 1.0, 1.0) == 2.0
    # a chain applies its members in order with the same draws, then the bias with the episode's draw:
    # ((2 + 0.1 * 1.5) * (1 + 0.1 * 0.5)) + 0.02 * (-2) = 2.15 * 1.05 - 0.04
    got = ot.add_noise(2.0, [("add_gaussian", 0.0, 0.1), ("mul_uniform", 1.0, 0.1)], ("add_gaussian", 0.0, 0.02), 1.5, 0.5,
                       -2.0, 0.0, 1.0)
    assert got == pytest.approx(2.15 * 1.05 - 0.04)
    # the order matters, which a swapped implementation would fail: (2 * 1.05) + 0.15
    got = ot.add_noise(2.0, [("mul_uniform", 1.0, 0.1), ("add_gaussian", 0.0, 0.1)], None, 1.5, 0.5, 0.0, 0.0, 1.0)
    assert got == pytest.approx(2.0 * 1.05 + 0.15)
    # the bias follows the current level with a fixed draw (observation.py:139 passes curriculum_level every step)
    b1 = ot.add_noise(1.0, [], ("mul_uniform", 1.0, 0.2), 0.0, 0.0, 0.0, 0.5, 1.0)
    b2 = ot.add_noise(1.0, [], ("mul_uniform", 1.0, 0.2), 0.0, 0.0, 0.0, 0.5, 0.5)
    assert b1 == pytest.approx(1.1) and b2 == pytest.approx(1.05)


def test_engine_reset_draws_hand_computed():
    """ksim/engine.py:222-245 and ksim/actuators.py:219-238: ranges, level scaling and layout of the per-episode draws."""
    nu = 2
    u = np.array([0.5, -1.0, 1.0, 0.2, -0.2, 0.0, 0.4, 1.0, -1.0, 0.0])
    z = np.array([9.0, 1.0, -2.0, 0.5, 0.25, -1.0, 2.0, 0.3, 0.1, -0.5])
    out = ot.engine_reset_draws(nu, 0.5, u, z, latency_range=(1.0, 3.0), zero_offset=dict(mean=0.0, mag=0.0, std=0.02),
                                action_bias=dict(mean=0.0, mag=0.1, std=0.0), torque_bias=dict(mean=0.5, mag=0.0, std=2.0),
                                kp_scale=dict(mean=1.0, mag=0.2, std=0.0), kd_scale=None,
                                torque_limit_scale=dict(mean=0.9, mag=0.0, std=0.1))
    # latency ~ U(1 * 0.5, 3 * 0.5): u = 0.5 is three quarters of the way
    assert out["action_latency"] == pytest.approx(0.5 + 0.75 * 1.0)
    np.testing.assert_allclose(out["zero_offset"], [1.0 * 0.02 * 0.5, -2.0 * 0.02 * 0.5])       # scaled by the level
    np.testing.assert_allclose(out["action"], [0.2 * 0.1, -0.2 * 0.1])                          # not scaled by the level
    np.testing.assert_allclose(out["torque"], [0.5 - 2.0, 0.5 + 4.0])
    assert out["kp_scale"] == pytest.approx(1.0 + 0.2) and out["kd_scale"] == pytest.approx(1.0)
    assert out["torque_limit_scale"] == pytest.approx(0.9 - 0.05)
    # defaults: no bias, unit scales, zero latency range gives zero latency whatever the draw
    out = ot.engine_reset_draws(nu, 1.0, u, z, latency_range=(0.0, 0.0), zero_offset=None)
    assert out["action_latency"] == 0.0 and not out["zero_offset"].any() and not out["action"].any()
    assert out["kp_scale"] == 1.0 and out["torque_limit_scale"] == 1.0
    # both zero-offset parts with one key (engine.py:117-124): the uniform part is a function of the normal draw
    out = ot.engine_reset_draws(nu, 1.0, u, z, latency_range=(0.0, 0.0), zero_offset=dict(mean=0.0, mag=0.1, std=0.01, same_key=True))
    np.testing.assert_allclose(out["zero_offset"], 0.01 * z[1:3] + 0.1 * ot.same_key_uniform(z[1:3]))


def test_new_reset_restatements_hand_computed():
    """resets.py:45-120, 284-354 by hand: the cell of a height field, the frame of a motion, and rotations whose effect
    on a vector is known."""
    q0 = np.zeros(10)
    q0[3] = 1.0
    # plane: x = clip(0.5 * 4, -1.5, 1.5) = 1.5, y = -0.25 * 2 = -0.5, z = plane 0.1 + base height 0.9
    q = ot.xy_position_reset(q0, 0.5, -0.25, x_range=4.0, y_range=2.0, padded_bounds=(-1.5, 1.5, -3.0, 3.0), z=0.1,
                             robot_base_height=0.9)
    np.testing.assert_allclose(q[:3], [1.5, -0.5, 1.0])
    # height field 5 x 3 over [-2, 2] x [-1, 1]: x = 1.0 -> (3 / 4) * 4 = 3; y = 0.4 -> (1.4 / 2) * 2 = 1.4 -> 1
    h = np.arange(15.0).reshape(5, 3)
    q = ot.xy_position_reset(q0, 0.25, 0.2, x_range=4.0, y_range=2.0, padded_bounds=(-2, 2, -1, 1), hfield=h,
                             hfield_bounds=(2.0, 1.0, 0.5), robot_base_height=0.25)
    np.testing.assert_allclose(q[:3], [1.0, 0.4, h[3, 1] + 0.75])
    # the far corner clips to the last cell
    q = ot.xy_position_reset(q0, 1.0, 1.0, x_range=9.0, y_range=9.0, padded_bounds=(-2, 2, -1, 1), hfield=h,
                             hfield_bounds=(2.0, 1.0, 0.0))
    assert q[2] == h[4, 2]
    # motion: frame 7 of 5 wraps to 2; joints only unless the free joint is included; time = frame * dt
    motion = np.arange(50.0).reshape(5, 10)
    q, t = ot.initial_motion_state_reset(q0, 7, motion, 0.02, freejoint=False)
    np.testing.assert_allclose(q[:7], q0[:7]); np.testing.assert_allclose(q[7:], motion[2, 7:]); assert t == pytest.approx(0.14)
    q, _ = ot.initial_motion_state_reset(q0, 1, motion, 0.02, freejoint=True)
    np.testing.assert_allclose(q, motion[1])
    # heading u = 0.5 is a quarter turn about z: the body's x axis points along world y
    q = ot.random_heading_reset(q0, 0.5)
    np.testing.assert_allclose(ot.rotate_vector_by_quat(np.array([1.0, 0, 0]), q[3:7]), [0, 1, 0], atol=1e-12)
    # pitch and roll share one draw: u = 0.75 in (-0.2, 0.2) and (0.4, 0.0) gives pitch 0.1, roll 0.1;
    # u = 1/2 in symmetric ranges is no rotation; a pure pitch of pi / 2 turns the body's x axis to world -z
    q = ot.random_pitch_roll_reset(q0, 0.75, (-0.2, 0.2), (0.4, 0.0))
    np.testing.assert_allclose(q[3:7], ot.euler_to_quat([0.1, 0.1, 0.0]))
    np.testing.assert_allclose(ot.random_pitch_roll_reset(q0, 0.5, (-0.3, 0.3), (-0.1, 0.1))[3:7], [1, 0, 0, 0], atol=1e-15)
    q = ot.random_pitch_roll_reset(q0, 1.0, (0.0, np.pi / 2), (0.0, 0.0))
    np.testing.assert_allclose(ot.rotate_vector_by_quat(np.array([1.0, 0, 0]), q[3:7]), [0, 0, -1], atol=1e-12)
    # roll about x then heading: the order matters, quat <- quat * next
    a = ot.random_heading_reset(ot.random_pitch_roll_reset(q0, 1.0, (0.0, 0.0), (0.0, 0.6)), 0.5)
    b = ot.random_pitch_roll_reset(ot.random_heading_reset(q0, 0.5), 1.0, (0.0, 0.0), (0.0, 0.6))
    assert np.abs(a[3:7] - b[3:7]).max() > 0.1


def test_symmetry_and_joint_position_rewards_hand_computed():
    """rewards.py:843-936, 1352-1380 on numbers small enough to do by hand."""
    # two joints (qpos 7 and 9), targets (0.1, -0.2), two steps: x = [[0.4, 0.2], [0.0, 0.6]], mean (0.2, 0.4)
    q = np.zeros((2, 10))
    q[:, 7], q[:, 9] = [0.5, 0.1], [0.0, 0.4]
    r, c = ot.symmetry_reward(q, np.array([1.0, -1.0]), False, (0, 2), (0.1, -0.2), alpha=0.5)
    np.testing.assert_allclose(c, [0.5 + 0.1, -0.5 + 0.2])            # 0.5 carry + 0.5 mean
    np.testing.assert_allclose(r, [-(0.4 * 0.6 + 0.2 * -0.3), -(0.0 * 0.6 + 0.6 * -0.3)])
    _, c2 = ot.symmetry_reward(q, np.array([1.0, -1.0]), True, (0, 2), (0.1, -0.2), alpha=0.5)
    np.testing.assert_allclose(c2, [0.05 + 0.1, -0.1 + 0.2])          # restarts from the targets
    # a pair, right joint flipped: ql = (0.3, 0.1), qr = -(q8 - 0.1) = (0.2, -0.1); difference (0.1, 0.2)
    q = np.zeros((2, 10))
    q[:, 7], q[:, 8] = [0.3, 0.1], [-0.1, 0.2]
    out, c = ot.pairwise_symmetry_reward(q, np.zeros(2), False, 0, 1, 0.0, 0.1, flipped=True, alpha=1.0, kernel_scale=0.5,
                                         sq_scale=0.2, abs_scale=0.3)
    np.testing.assert_allclose(c, [0.2, 0.05])
    np.testing.assert_allclose(out["self"], [-(0.3 * 0.2 + 0.2 * 0.05), -(0.1 * 0.2 - 0.1 * 0.05)])
    d = np.array([0.1, 0.2])
    np.testing.assert_allclose(out["lr"], np.exp(-d**2 / (2 * 0.25)) - 0.2 * d**2 - 0.3 * np.abs(d))
    # joint-position command half way (step 2 of 4) from 0 to 1 over 0.5 s: position 0.5, velocity 2
    q, v = np.zeros((1, 9)), np.zeros((1, 8))
    q[0, 8], v[0, 7] = 0.5, 1.5
    out = ot.joint_position_reward(q, v, np.array([[0.0]]), np.array([[1.0]]), np.array([0.5]), np.array([4.0]), np.array([2.0]), (1,),
                                   pos_scale=0.25, vel_scale=0.5, sq_scale=0.1, abs_scale=0.2)
    assert out["pos"][0] == pytest.approx(1.0)                        # on target: exp(0) and no penalty
    assert out["vel"][0] == pytest.approx(np.exp(-0.25 / 0.5) - 0.1 * 0.25 - 0.2 * 0.5)


def test_imu_offset_site_rotation_and_contact_list_hand_computed():
    # a pure roll error of 0.2 rad: [1, 0.1, 0, 0] normalised; to first order a rotation by 0.2 about x
    q = ot.imu_alignment_offset(0.2, 0.0)
    np.testing.assert_allclose(q, np.array([1, 0.1, 0, 0]) / np.sqrt(1.01))
    v = ot.rotate_vector_by_quat(np.array([0.0, 1.0, 0.0]), q)
    assert v[2] == pytest.approx(np.sin(2 * np.arctan(0.1)))  # the exact angle of [1, t] is 2 atan(t)
    # order: yaw last, i.e. qz on the left; with all three angles the product differs from the reversed order
    a = ot.imu_alignment_offset(0.3, -0.2, 0.5)
    qx, qy, qz = np.array([1, 0.15, 0, 0]), np.array([1, 0, -0.1, 0]), np.array([1, 0, 0, 0.25])
    b = ot.quat_mul(qz, ot.quat_mul(qy, qx))
    np.testing.assert_allclose(a, b / np.linalg.norm(b))
    wrong = ot.quat_mul(qx, ot.quat_mul(qy, qz))
    assert np.abs(a - wrong / np.linalg.norm(wrong)).max() > 1e-2
    # site rotation: body turned a quarter about z, site a quarter about x.  R = Rz(90) Rx(90): rows (0,0,1), (1,0,0)
    s = np.sqrt(0.5)
    np.testing.assert_allclose(ot.site_rotation6d([s, 0, 0, s], [s, s, 0, 0]), [0, 0, 1, 1, 0, 0], atol=1e-12)
    np.testing.assert_allclose(ot.quat_to_matrix([s, 0, 0, s]) @ [1, 0, 0], [0, 1, 0], atol=1e-12)
    # contact list: spheres 0 and 2 with the floor; 0 touches.  Without the floor in the list nothing collides.
    dist = np.array([-0.01, -0.5, 0.02])
    assert ot.contact_observation(dist, (0, -1, 2)).tolist() == [True, True, False]
    assert ot.contact_observation(dist, (0, 1)).tolist() == [False, False]
    assert ot.contact_observation(np.array([0.1, -0.5, 0.02]), (0, -1, 2)).tolist() == [False, False, False]


def test_joint_position_command_reaches_its_target_on_time():
    """What the reference's value type fixes (ksim/commands.py:795-818, 852-893): the commanded position start + (target - start)
    step_id / num_steps moves linearly, is the target exactly when step_id = num_steps = ceil(total_time / ctrl_dt), holds for
    that one step, and the next value starts from where the joints are then; the commanded velocity is (target - start) /
    total_time throughout."""
    rng = np.random.default_rng(3)
    kw = dict(indices=(2, 0), ranges=((-1.0, 1.0), (0.2, 0.4)), ctrl_dt=0.02, min_time=0.1, max_time=0.5)
    qpos = rng.normal(size=12)
    u = np.array([0.25, 0.5, 0.775] + [0.0] * 5)
    v = ot.joint_position_command(np.zeros(7), qpos, u, True, **kw)
    np.testing.assert_allclose(v[:2], qpos[[9, 7]], rtol=1e-6)
    np.testing.assert_allclose(v[2:4], [-0.5, 0.3], rtol=1e-6)
    assert v[4] == pytest.approx(0.41) and v[5] == 21 and v[6] == 0  # ceil(0.41 / 0.02) = 21
    seen = []
    for k in range(1, 22):
        v = ot.joint_position_command(v, rng.normal(size=12), rng.random(8), False, **kw)
        assert v[6] == k
        seen.append(v[:2] + (v[2:4] - v[:2]) * v[6] / v[5])
    np.testing.assert_allclose(np.diff(np.stack(seen), axis=0), np.tile((v[2:4] - v[:2]) / 21, (20, 1)), rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(seen[-1], v[2:4], rtol=1e-6)
    q2, u2 = rng.normal(size=12), rng.random(8)
    w = ot.joint_position_command(v, q2, u2, False, **kw)  # step_id 22 > 21: a new target from the current pose
    assert w[6] == 0
    np.testing.assert_allclose(w[:2], q2[[9, 7]].astype(np.float32), rtol=1e-6)
    assert -1.0 <= w[2] <= 1.0 and 0.2 <= w[3] <= 0.4 and 0.1 <= w[4] <= 0.5 and w[5] == np.ceil(np.float32(w[4]) / np.float32(0.02))


def test_cartesian_coordinate_command_moves_at_its_speed_without_overshoot():
    """ksim/commands.py:556-656: the current point travels straight towards the target at `speed`, lands on it exactly (the
    last stride is cut to the remaining distance), stays there while no switch is drawn, and draws a new target inside the box
    scaled by the curriculum level once it has arrived and the switch draw allows; a jump draw replaces the target at any time."""
    kw = dict(box_min=(-1.0, 0.0, 0.5), box_max=(1.0, 2.0, 1.5), dt=0.05, min_speed=1.0, max_speed=2.0, curriculum_scale=0.5, level=1.0)
    first = ot.cartesian_coordinate_command(np.zeros(7), [0.0, 1.0, 0.5, 0.5, 0.9], True, **kw)
    # the box grows by 1.5 about its centre (0, 1, 1): x in [-1.5, 1.5], y in [-0.5, 2.5], z in [0.25, 1.75]
    np.testing.assert_allclose(first, [-1.5, 2.5, 1.0, -1.5, 2.5, 1.0, 1.5])
    v = first.copy()
    v[3:6] = [-1.5 + 0.3, 2.5, 1.0 + 0.4]  # a target 0.5 away; at 1.5 * 0.05 = 0.075 a step: six full strides and one of 0.05
    path = [v[:3].copy()]
    for k in range(9):
        v = ot.cartesian_coordinate_command(v, [0.1, 0.2, 0.3, 0.4, 0.99], False, switch_prob=0.5, **kw)
        path.append(v[:3].copy())
    strides = np.linalg.norm(np.diff(np.stack(path), axis=0), axis=1)
    np.testing.assert_allclose(strides, [0.075] * 6 + [0.05, 0.0, 0.0], atol=1e-12)
    np.testing.assert_allclose(v[:3], v[3:6], atol=1e-12)
    # arrived and the draw falls under switch_prob: a new target and speed; the point does not move this step (old distance 0)
    w = ot.cartesian_coordinate_command(v, [0.5, 0.5, 0.5, 0.0, 0.2], False, switch_prob=0.5, **kw)
    np.testing.assert_allclose(w, np.concatenate([v[:3], [0.0, 1.0, 1.0, 1.0]]), atol=1e-12)
    # still travelling: the same draw does not switch, a jump does, and the stride of that step is still capped by the old distance
    v[3:6] = v[:3] + [0.0, 0.0, 0.03]
    stay = ot.cartesian_coordinate_command(v, [0.5, 0.5, 0.5, 0.0, 0.2], False, switch_prob=0.0, jump_prob=0.1, **kw)
    np.testing.assert_allclose(stay[3:6], v[3:6]); assert np.linalg.norm(stay[:3] - v[:3]) == pytest.approx(0.03)
    jump = ot.cartesian_coordinate_command(v, [0.5, 0.5, 0.5, 0.0, 0.05], False, switch_prob=0.0, jump_prob=0.1, **kw)
    np.testing.assert_allclose(jump[3:], [0.0, 1.0, 1.0, 1.0]); assert np.linalg.norm(jump[:3] - v[:3]) == pytest.approx(0.03)


def test_site_frame_sensors_against_scipy_rotations():
    """framepos / framequat / magnetometer of a site: composition of the body's pose with the site's, checked with scipy."""
    from scipy.spatial.transform import Rotation

    rng = np.random.default_rng(21)
    for _ in range(5):
        qb, qs = rng.normal(size=4), rng.normal(size=4)
        qb, qs = qb / np.linalg.norm(qb), qs / np.linalg.norm(qs)
        xb, r, field = rng.normal(size=3), rng.normal(size=3), rng.normal(size=3)
        Rb, Rs = Rotation.from_quat(qb[[1, 2, 3, 0]]), Rotation.from_quat(qs[[1, 2, 3, 0]])
        np.testing.assert_allclose(ot.site_frame_position(xb, qb, r), xb + Rb.apply(r), atol=1e-12)
        want = (Rb * Rs).as_quat()[[3, 0, 1, 2]]
        got = ot.site_frame_quaternion(qb, qs)
        assert min(np.abs(got - want).max(), np.abs(got + want).max()) < 1e-12
        np.testing.assert_allclose(ot.site_magnetometer(qb, qs, field), (Rb * Rs).inv().apply(field), atol=1e-12)


def test_lowpass_scan_and_its_backward_sweep():
    """The filter threaded through a trajectory: equal to stepping ksim.lowpass_one_pole (pinned above by its closed form),
    restarted from zero at fresh steps; the written-out reverse sweep against central differences of the forward scan."""
    rng = np.random.default_rng(31)
    Tn, b, n = 9, 4, 3
    dt, fc = 0.02, 7.0
    a = dt / (1.0 / (2 * np.pi * fc) + dt)
    x = rng.normal(size=(Tn, b, n))
    y0 = rng.normal(size=(b, n))
    fresh = np.zeros((Tn, b), bool)
    fresh[4, 1] = fresh[0, 2] = fresh[8, 3] = fresh[5, 3] = True
    y, last = ot.lowpass_scan(x, dt, fc, y0, fresh)
    # env 0 never restarts: the closed form y_t = (1-a)^(t+1) y0 + a sum_s (1-a)^(t-s) x_s
    for t in range(Tn):
        want = (1 - a) ** (t + 1) * y0[0] + a * sum((1 - a) ** (t - s) * x[s, 0] for s in range(t + 1))
        np.testing.assert_allclose(y[t, 0], want, rtol=1e-12)
    # env 1 restarts at step 4: from there on the history before it and y0 are forgotten
    for t in range(4, Tn):
        want = a * sum((1 - a) ** (t - s) * x[s, 1] for s in range(4, t + 1))
        np.testing.assert_allclose(y[t, 1], want, rtol=1e-12)
    np.testing.assert_allclose(y[0, 2], a * x[0, 2], rtol=1e-12)  # fresh at the first step: y0 is not used
    np.testing.assert_allclose(last, y[-1], atol=0)
    # constant input from zero: y_k = x (1 - (1-a)^k)
    c, _ = ot.lowpass_scan(np.full((6, 1, 1), 2.0), dt, fc)
    np.testing.assert_allclose(c[:, 0, 0], 2.0 * (1 - (1 - a) ** np.arange(1, 7)), rtol=1e-12)
    # backward: L = sum(w * y); the recursion is linear, so central differences are exact up to rounding
    w = rng.normal(size=y.shape)
    dx, dy0 = ot.lowpass_scan_backward(w, dt, fc, fresh)
    L = lambda x_, y0_: float((w * ot.lowpass_scan(x_, dt, fc, y0_, fresh)[0]).sum())  # noqa: E731
    eps = 1e-5
    for idx in [(0, 0, 0), (3, 1, 2), (4, 1, 0), (8, 3, 1), (5, 3, 2), (2, 2, 1), (7, 0, 2)]:
        xp, xm = x.copy(), x.copy()
        xp[idx] += eps; xm[idx] -= eps
        assert dx[idx] == pytest.approx((L(xp, y0) - L(xm, y0)) / (2 * eps), rel=1e-7, abs=1e-10), idx
    for idx in [(0, 0), (1, 2), (2, 1), (3, 0)]:
        yp, ym = y0.copy(), y0.copy()
        yp[idx] += eps; ym[idx] -= eps
        assert dy0[idx] == pytest.approx((L(x, yp) - L(x, ym)) / (2 * eps), rel=1e-7, abs=1e-10), idx
    assert np.all(dy0[2] == 0)  # env 2 is fresh at step 0: its y0 reaches nothing
    # the cut: inputs of env 1 before its restart at step 4 reach only the outputs before it
    w_late = np.zeros_like(w); w_late[4:, 1] = 1.0
    assert np.all(ot.lowpass_scan_backward(w_late, dt, fc, fresh)[0][:4, 1] == 0)
    # without any restart dx_s = a sum_{t>=s} (1-a)^(t-s) w_t
    dx_free, _ = ot.lowpass_scan_backward(w, dt, fc)
    s_ = 3
    np.testing.assert_allclose(dx_free[s_, 0], a * sum((1 - a) ** (t - s_) * w[t, 0] for t in range(s_, Tn)), rtol=1e-12)


def test_norm_and_kernel_helpers_hand_computed():
    """`get_norm`, `exp_kernel`, `exp_kernel_with_penalty` (rewards.py:72-88): the values the reference's formulas give at a
    few points worked out by hand."""
    x = np.array([-2.0, 0.0, 0.5])
    np.testing.assert_array_equal(ot.get_norm(x, "l1"), [2.0, 0.0, 0.5])
    np.testing.assert_array_equal(ot.get_norm(x, "l2"), [4.0, 0.0, 0.25])
    with pytest.raises(ValueError):
        ot.get_norm(x, "linf")
    # exp(-x^2 / (2 s^2)): 1 at 0, e^-1/2 one scale away, e^-2 two scales away
    np.testing.assert_allclose(ot.exp_kernel(np.array([0.0, 0.3, -0.6]), 0.3), [1.0, np.exp(-0.5), np.exp(-2.0)], rtol=1e-15)
    # the penalised kernel subtracts |x| abs_scale + x^2 sq_scale from it
    np.testing.assert_allclose(ot.exp_kernel_with_penalty(np.array([0.0, -0.6]), 0.3, 0.5, 0.25),
                               [1.0, np.exp(-2.0) - 0.6 * 0.25 - 0.36 * 0.5], rtol=1e-15)
