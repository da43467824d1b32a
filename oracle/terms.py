"""numpy restatement of the reference's per-env terms (test infrastructure).

Rewards follow ksim/rewards.py, terminations ksim/terminations.py, the PD
actuator ksim/actuators.py:182-217, the latency blend ksim/engine.py:287-288,
the done/success combination ksim/task/rl.py:1049-1050 and the reward total
ksim/task/rl.py:219-239.  Shapes are per env, time leading, like the reference.

Parity unpinned (third-party xax, absent from the reference tree and from this image): the quaternion conventions of
rotate_vector_by_quat / euler_to_quat (Hamilton wxyz assumed) and mixture_head against xax.MixtureOfGaussians (the
textbook mixture is restated and pinned by scipy).
"""

from __future__ import annotations

import numpy as np


# --------------------------------------------------------------------------- quaternions (Hamilton, wxyz)
def quat_mul(a, b):
    aw, ax, ay, az = np.moveaxis(np.asarray(a), -1, 0)
    bw, bx, by, bz = np.moveaxis(np.asarray(b), -1, 0)
    return np.stack(
        [
            aw * bw - ax * bx - ay * by - az * bz,
            aw * bx + ax * bw + ay * bz - az * by,
            aw * by - ax * bz + ay * bw + az * bx,
            aw * bz + ax * by - ay * bx + az * bw,
        ],
        axis=-1,
    )


def rotate_vector_by_quat(v, q, inverse: bool = False):
    """v' = q v q* (inverse: q* v q); the quaternion is normalised first (xax convention assumed)."""
    q = np.asarray(q, dtype=np.float64)
    q = q / np.linalg.norm(q, axis=-1, keepdims=True)
    if inverse:
        q = q * np.array([1.0, -1.0, -1.0, -1.0])
    v = np.asarray(v, dtype=np.float64)
    qv = np.concatenate([np.zeros(v.shape[:-1] + (1,)), v], axis=-1)
    qc = q * np.array([1.0, -1.0, -1.0, -1.0])
    return quat_mul(quat_mul(q, qv), qc)[..., 1:]


# --------------------------------------------------------------------------- norms / kernels
def get_norm(x, norm: str):
    """xax.get_norm as pinned by reference tests/test_rewards.py:95-98,120-123."""
    if norm == "l1":
        return np.abs(x)
    if norm == "l2":
        return np.square(x)
    raise ValueError(norm)


def exp_kernel(x, scale):  # rewards.py:72-73
    return np.exp(-np.square(x) / (2 * scale**2))


def exp_kernel_with_penalty(x, scale, sq_scale, abs_scale):  # rewards.py:84-88
    return np.abs(x) * -abs_scale + np.square(x) * -sq_scale + np.exp(-np.square(x) / (2 * scale**2))


# --------------------------------------------------------------------------- rewards
def _edge_pad_front(x, n):
    return np.concatenate([np.repeat(x[:1], n, axis=0), x], axis=0)


def action_velocity_penalty(action_ta, done_t, norm="l2"):  # rewards.py:410-419
    a = _edge_pad_front(np.asarray(action_ta, dtype=np.float64), 1)
    done = _edge_pad_front(np.asarray(done_t).astype(bool), 1)[:-1, None]
    vel = np.where(done, 0.0, a[1:] - a[:-1])
    pen = get_norm(vel, norm).mean(axis=-1)
    return np.where(np.arange(len(pen)) >= 1, pen, 0.0)


def action_acceleration_penalty(action_ta, done_t, norm="l2"):  # rewards.py:428-440
    a = _edge_pad_front(np.asarray(action_ta, dtype=np.float64), 2)
    done = _edge_pad_front(np.asarray(done_t).astype(bool), 2)[:-1, None]
    vel = np.where(done, 0.0, a[1:] - a[:-1])
    acc = np.where(done[1:], 0.0, vel[1:] - vel[:-1])
    pen = get_norm(acc, norm).mean(axis=-1)
    return np.where(np.arange(len(pen)) >= 2, pen, 0.0)


def action_jerk_penalty(action_ta, done_t, norm="l2"):  # rewards.py:449-460
    a = _edge_pad_front(np.asarray(action_ta, dtype=np.float64), 3)
    done = _edge_pad_front(np.asarray(done_t).astype(bool), 3)[:-1, None]
    vel = np.where(done, 0.0, a[1:] - a[:-1])
    acc = np.where(done[1:], 0.0, vel[1:] - vel[:-1])
    jerk = np.where(done[2:], 0.0, acc[1:] - acc[:-1])
    pen = get_norm(jerk, norm).mean(axis=-1)
    return np.where(np.arange(len(pen)) >= 3, pen, 0.0)


def _padded_differences(x, done_t, order):
    """The differencing shared by the joint and link smoothness terms (rewards.py:469-508, 814-839): pad `order` copies of the
    first row in front, difference `order` times, and zero each difference where the step before it was done."""
    x = _edge_pad_front(np.asarray(x, dtype=np.float64), order)
    done = _edge_pad_front(np.asarray(done_t).astype(bool), order)[:-1]
    done = done.reshape(done.shape + (1,) * (x.ndim - 1))
    return x, done


def small_joint_reward(qpos_tq, done_t, order, kernel_scale=0.25):  # rewards.py:463-508 (order 1, 2, 3 = velocity, acceleration, jerk)
    q, done = _padded_differences(np.asarray(qpos_tq)[:, 7:], done_t, order)
    d = np.where(done, 0.0, q[1:] - q[:-1])
    for k in range(1, order):
        d = np.where(done[k:], 0.0, d[1:] - d[:-1])
    return exp_kernel(d, kernel_scale).mean(axis=-1)


def avoid_limits_penalty(qpos_tq, joint_limits):  # rewards.py:527-533
    q = np.asarray(qpos_tq, dtype=np.float64)[:, 7:]
    lim = np.asarray(joint_limits, dtype=np.float64)
    return (-np.clip(q - lim[:, 0], None, 0.0) + np.clip(q - lim[:, 1], 0.0, None)).mean(axis=-1)


def avoid_limits_create(jnt_range, jnt_limited, factor=0.05):  # rewards.py:535-553 (rows: every joint, the free joint first)
    rng = np.asarray(jnt_range, dtype=np.float64)
    diff = (rng[:, 1] - rng[:, 0]) * factor
    lo = np.where(jnt_limited, rng[:, 0] - diff, -np.inf)
    hi = np.where(jnt_limited, rng[:, 1] + diff, np.inf)
    return np.stack([lo, hi], axis=-1)[1:]


def torque_penalty(ctrl_tu, ctrl_scales):  # rewards.py:567-569
    return np.abs(np.asarray(ctrl_tu, dtype=np.float64) / np.asarray(ctrl_scales, dtype=np.float64)).mean(axis=-1)


def energy_penalty(ctrl_tu, qvel_tv, ctrl_scales):  # rewards.py:588-591
    ctrl_n = np.asarray(ctrl_tu, dtype=np.float64) / np.asarray(ctrl_scales, dtype=np.float64)
    return np.abs(ctrl_n * np.asarray(qvel_tv, dtype=np.float64)[:, 6:]).mean(axis=-1)


def joint_deviation_penalty(qpos_tq, joint_indices, joint_targets, joint_weights=None, norm="l2"):  # rewards.py:629-639
    diff = np.asarray(qpos_tq, dtype=np.float64)[:, np.asarray(joint_indices) + 7] - np.asarray(joint_targets, dtype=np.float64)
    if joint_weights is not None:
        diff = diff * np.asarray(joint_weights, dtype=np.float64)
    return get_norm(diff, norm).sum(axis=-1)


def flat_body_reward(xquat_tb4, body_indices, plane=(0.0, 0.0, 1.0)):  # rewards.py:678-682
    quat = np.asarray(xquat_tb4, dtype=np.float64)[:, list(body_indices), :]
    plane = np.asarray(plane, dtype=np.float64)
    unit = rotate_vector_by_quat(np.broadcast_to(plane, quat.shape[:-1] + (3,)), quat, inverse=True)
    return (unit * plane).sum(axis=-1).mean(axis=-1)


def position_tracking_reward(xpos_tb3, cmd_t3, tracked, base, norm="l1", kernel_scale=0.25):  # rewards.py:713-719
    x = np.asarray(xpos_tb3, dtype=np.float64)
    err = get_norm((x[:, tracked] - x[:, base]) - np.asarray(cmd_t3, dtype=np.float64)[:, :3], norm).sum(-1)
    return exp_kernel(err, kernel_scale)


def no_roll_reward(qpos_tq, qvel_tv, s=0.25, sq=0.1, ab=0.1):  # rewards.py:789-804 (defaults); returns (angvel, pose)
    q, v = np.asarray(qpos_tq, dtype=np.float64), np.asarray(qvel_tv, dtype=np.float64)
    zb = rotate_vector_by_quat(np.broadcast_to(np.array([0.0, 0.0, 1.0]), q.shape[:-1] + (3,)), q[:, 3:7], inverse=True)
    roll = -np.arctan2(zb[:, 1], zb[:, 2])
    return exp_kernel_with_penalty(v[:, 3], s, sq, ab), exp_kernel_with_penalty(roll, s, sq, ab)


def link_smoothness_penalty(xpos_tb3, done_t, order, norm="l2"):  # rewards.py:813-821 (order 2), 830-840 (order 3)
    p, done = _padded_differences(np.asarray(xpos_tb3)[:, 1:], done_t, order)
    done = done[..., 0]
    d = np.where(done, 0.0, np.linalg.norm(p[1:] - p[:-1], axis=-1))
    for k in range(1, order):
        d = np.where(done[k:], 0.0, d[1:] - d[:-1])
    return get_norm(d, norm).mean(axis=-1)


def feet_slip_penalty(contact_tcn, velocity_tn6):  # rewards.py:1095-1105
    touching = (np.asarray(contact_tcn) > 0.5).any(axis=-2)
    speed = np.linalg.norm(np.asarray(velocity_tn6, dtype=np.float64), axis=-1)
    return np.where(touching, speed, 0.0).sum(axis=-1)


def reachability_penalty(action_tj, qpos_tq, delta_max_j, squared=True):  # rewards.py:1119-1129
    excess = np.maximum(0.0, np.abs(np.asarray(action_tj, dtype=np.float64) - np.asarray(qpos_tq, dtype=np.float64)[:, 7:])
                        - np.asarray(delta_max_j, dtype=np.float64))
    return (excess**2 if squared else excess).sum(axis=-1)


def intersection_penalty(position_tn3, min_distance):  # rewards.py:1424-1430
    p = np.asarray(position_tn3, dtype=np.float64)
    dist = np.linalg.norm(p[:, :, None, :] - p[:, None, :, :], axis=-1)
    dist = dist + np.triu(np.ones_like(dist)) * min_distance * 2
    return np.where((dist < min_distance).any(axis=(-2, -1)), 1.0, 0.0)


def stay_alive_reward(done_t, success_t, balance=100.0, success_reward=None):  # rewards.py:178-188
    alive = 1.0 / balance
    return np.where(done_t, np.where(success_t, alive if success_reward is None else success_reward, -1.0), alive)


def base_height_reward(qpos_tq, height_target, kernel_scale=0.25):  # rewards.py:382-385
    return exp_kernel(np.asarray(qpos_tq)[..., 2] - height_target, kernel_scale)


def base_height_range_reward(qpos_tq, z_lower, z_upper, dropoff):  # rewards.py:396-401
    z = np.asarray(qpos_tq)[..., 2]
    return np.clip(1.0 - np.clip(np.maximum(z_lower - z, z - z_upper), 0.0, None) * dropoff, 0.0, None)


def amp_reward(discriminator_logits):  # ksim/task/amp.py:109-111
    d = np.asarray(discriminator_logits, dtype=np.float64)
    return np.maximum(0.0, 1.0 - 0.25 * np.square(d - 1.0))


def upright_reward(qpos_tq, qvel_tv, s=0.25, sq=0.1, ab=0.1):  # rewards.py:760-777 (defaults)
    qpos = np.asarray(qpos_tq, dtype=np.float64)
    qvel = np.asarray(qvel_tv, dtype=np.float64)
    z_b = rotate_vector_by_quat(np.broadcast_to([0.0, 0.0, 1.0], qpos.shape[:-1] + (3,)), qpos[..., 3:7], inverse=True)
    pitch = np.arctan2(z_b[..., 0], z_b[..., 2])
    return {
        "angvel": exp_kernel_with_penalty(qvel[..., 4], s, sq, ab),
        "linvel": exp_kernel_with_penalty(qvel[..., 2], s, sq, ab),
        "pose": exp_kernel_with_penalty(pitch, s, sq, ab),
    }


def total_reward(components, scales, is_penalty, clip_min=None, clip_max=None):
    """rl.py:219-239: each term * (+/-)scale, summed in insertion order, optional clip."""
    total = None
    out = {}
    for name, val in components.items():
        s = -scales[name] if is_penalty[name] else scales[name]
        out[name] = np.asarray(val) * s
        total = out[name] if total is None else total + out[name]
    if clip_min is not None:
        total = np.maximum(total, clip_min)
    if clip_max is not None:
        total = np.minimum(total, clip_max)
    return total, out


# --------------------------------------------------------------------------- terminations (int32 in {-1, 0, +1})
def minimum_height_termination(qpos, min_height):  # terminations.py:79-80
    return np.where(np.asarray(qpos)[..., 2] < min_height, -1, 0).astype(np.int32)


def bad_z_termination(qpos, min_z, max_z, level=0.0, final_min_z=None, final_max_z=None):  # terminations.py:140-146
    z = np.asarray(qpos)[..., 2]
    fmin = min_z if final_min_z is None else final_min_z
    fmax = max_z if final_max_z is None else final_max_z
    lo = (fmin - min_z) * level + min_z
    hi = (fmax - max_z) * level + max_z
    return np.where((z < lo) | (z > hi), -1, 0).astype(np.int32)


def not_upright_termination(qpos, max_radians):  # terminations.py:66-70
    qpos = np.asarray(qpos, dtype=np.float64)
    g = rotate_vector_by_quat(np.broadcast_to([0.0, 0.0, 1.0], qpos.shape[:-1] + (3,)), qpos[..., 3:7], inverse=True)
    return np.where(np.arccos(np.clip(g[..., 2], -1.0, 1.0)) > max_radians, -1, 0).astype(np.int32)


def bad_velocity_termination(qvel, max_vel):  # terminations.py:155-157
    return np.where(np.linalg.norm(np.asarray(qvel)[..., 0:3], axis=-1) > max_vel, -1, 0).astype(np.int32)


def far_from_origin_termination(qpos, max_dist, pos_termination=True):  # terminations.py:170-172
    val = 1 if pos_termination else -1
    return np.where(np.linalg.norm(np.asarray(qpos)[..., :3], axis=-1) > max_dist, val, 0).astype(np.int32)


def episode_length_termination(time, max_length_sec, pos_termination=True, level=0.0,
                               disable_at_curriculum_level=None):  # terminations.py:186-192
    val = 1 if pos_termination else -1
    long_episodes = np.where(np.asarray(time) > max_length_sec, val, 0).astype(np.int32)
    if disable_at_curriculum_level is not None:  # terminations.py:188-190: off below that curriculum level
        return np.where(np.asarray(level) < disable_at_curriculum_level, 0, long_episodes).astype(np.int32)
    return long_episodes


def illegal_contact_termination(ncon, geom1, geom2, dist, illegal_geom_idxs, contact_eps=-1e-3):  # terminations.py:90-99
    if ncon == 0:
        return np.int32(0)
    bad = np.isin(geom1, illegal_geom_idxs) | np.isin(geom2, illegal_geom_idxs)
    return np.int32(-1 if np.any(np.where(bad, np.asarray(dist) < contact_eps, False)) else 0)


def combine_terminations(terms):
    """rl.py:1049-1050: done = OR(t != 0); success = AND(t != -1) & done."""
    terms = [np.asarray(t) for t in terms]
    done = np.zeros(terms[0].shape, dtype=bool)
    succ = np.ones(terms[0].shape, dtype=bool)
    for t in terms:
        done |= t != 0
        succ &= t != -1
    return done, succ & done


# --------------------------------------------------------------------------- actuator / engine sub-step helpers
def position_actuator_torque(
    action, qpos_j, qvel_j, kp, kd, ctrl_clip,
    action_scale=1.0, action_noise=0.0, action_bias=0.0, torque_noise=0.0, torque_bias=0.0,
    kp_scale=1.0, kd_scale=1.0, torque_limit_scale=1.0,
):
    """actuators.py:198-217 with the noise draws passed in as explicit arrays."""
    target = action * action_scale + action_noise + action_bias
    ctrl = (kp * kp_scale) * (target - qpos_j) + (kd * kd_scale) * (0.0 - qvel_j)
    ctrl = ctrl + torque_noise + torque_bias
    lim = ctrl_clip * torque_limit_scale
    return np.clip(ctrl, -lim, lim)


def latency_blend(step_num, latency, last_ctrl, action, drop):
    """engine.py:287-288."""
    prct = np.clip(step_num - latency, 0.0, 1.0)
    return np.where(drop, last_ctrl, last_ctrl * (1.0 - prct) + action * prct)


# --------------------------------------------------------------------------- random variables, noise, bias
def same_key_uniform(z):
    """The U(-1, 1) draw that the random bits behind the standard normal draw z give: jax.random builds a normal as
    sqrt(2) erfinv(u) of the uniform u in (-1, 1) those bits give, so u = erf(z / sqrt 2) = 2 Phi(z) - 1.  This is what
    'both drawn with the same key' (ksim/noise.py:106-121, 222-229) means for explicit draws.  jax is third-party and
    absent here: the construction is restated, parity unpinned; that the result is uniform when z is normal is a theorem
    (probability integral transform) and is tested."""
    from math import erf, sqrt

    return np.vectorize(lambda x: erf(x / sqrt(2.0)))(np.asarray(z, dtype=np.float64))


def random_variable(mean, mag, std, u, z, level=1.0, same_key=False):
    """ksim/noise.py:74-121 with explicit standard draws u ~ U(-1,1), z ~ N(0,1): Uniform (std 0), Gaussian (mag 0),
    UniformGaussian (both, same_key) and Zero (all 0) random variables."""
    w = same_key_uniform(z) if same_key else np.asarray(u, dtype=np.float64)
    return mean + np.asarray(z, dtype=np.float64) * (std * level) + w * (mag * level)


def apply_noise(obs, kind, mean, scale, z, w, level, scale2=0.0):
    """One Noise or Bias of ksim/noise.py:129-213 on an observation.  kind: 'add_gaussian', 'add_uniform', 'mul_gaussian',
    'mul_uniform', 'add_uniform_gaussian', 'mul_uniform_gaussian' or 'none'."""
    if kind == "none":
        return np.asarray(obs, dtype=np.float64)
    op, dist = kind.split("_", 1)
    if dist == "gaussian":
        rv = random_variable(mean, 0.0, scale, 0.0, z, level)
    elif dist == "uniform":
        rv = random_variable(mean, scale, 0.0, w, 0.0, level)
    else:
        rv = random_variable(mean, scale2, scale, w, z, level)
    return obs + rv if op == "add" else obs * rv


def add_noise(obs, noises, bias, z, w, bias_z, bias_w, level):
    """Observation.add_noise (ksim/observation.py:110-142): the noise (a chain applies every member with the same key,
    noise.py:222-229, hence the same z and w), then the per-episode bias, whose draw (bias_z, bias_w) is fixed over the
    episode while its scale follows the current level.  noises: list of (kind, mean, scale[, scale2]); bias: one or None."""
    out = np.asarray(obs, dtype=np.float64)
    for st in noises:
        out = apply_noise(out, st[0], st[1], st[2], z, w, level, *(st[3:4]))
    if bias is not None:
        out = apply_noise(out, bias[0], bias[1], bias[2], bias_z, bias_w, level, *(bias[3:4]))
    return out


def engine_reset_draws(nu, level, u, z, *, latency_range, zero_offset, action_bias=None, torque_bias=None, kp_scale=None,
                       kd_scale=None, torque_limit_scale=None):
    """What MjxEngine.reset draws besides the state (ksim/engine.py:222-245) with PositionActuators.get_initial_state
    (ksim/actuators.py:219-238), from explicit standard draws u ~ U(-1,1), z ~ N(0,1) of length 3 nu + 4 laid out as
    [latency, zero offset (nu), action bias (nu), torque bias (nu), kp scale, kd scale, torque limit scale].
    latency_range is in physics steps; the random variables are dicts(mean, mag, std[, same_key]); None means the
    reference's default (zero bias, unit scale).  Latency and zero offset scale with the curriculum level, the actuator
    state does not (get_random_variable is called without a level there)."""
    u, z = np.asarray(u, dtype=np.float64), np.asarray(z, dtype=np.float64)

    def rv(spec, sl, lvl, default_mean):
        spec = spec or dict(mean=default_mean, mag=0.0, std=0.0)
        return random_variable(spec["mean"], spec.get("mag", 0.0), spec.get("std", 0.0), u[sl], z[sl], lvl, spec.get("same_key", False))

    lo, hi = latency_range[0] * level, latency_range[1] * level
    return {
        "action_latency": lo + 0.5 * (u[0] + 1.0) * (hi - lo),  # uniform(minval, maxval), engine.py:233-237
        "zero_offset": rv(zero_offset, slice(1, 1 + nu), level, 0.0),
        "action": rv(action_bias, slice(1 + nu, 1 + 2 * nu), 1.0, 0.0),
        "torque": rv(torque_bias, slice(1 + 2 * nu, 1 + 3 * nu), 1.0, 0.0),
        "kp_scale": rv(kp_scale, 3 * nu + 1, 1.0, 1.0),
        "kd_scale": rv(kd_scale, 3 * nu + 2, 1.0, 1.0),
        "torque_limit_scale": rv(torque_limit_scale, 3 * nu + 3, 1.0, 1.0),
    }


def scrub_action(action, clip_max=1e3):
    """rl.py:998-1001: NaN -> 0, then clip."""
    a = np.where(np.isnan(action), 0.0, action)
    return np.clip(a, -clip_max, clip_max)


def velocity_event(kind, params, time_remaining, dt, u, level_scale, gravity=(0.0, 0.0, -9.81)):
    """One physics substep of a velocity event for one env (ksim/events.py:58-237): returns (impulse on qvel[0:6],
    new time remaining).  `u` = U[0,1) draws, the first three used (direction / sign / height, magnitude, next interval).
    kind: "linear" (linvel, vel_range), "angular" (angvel, vel_range), "jump" (jump_height_range)."""
    f32 = np.float32
    left = f32(time_remaining) - f32(dt)  # events.py:77-78: float32 timestep
    imp = np.zeros(6)
    if left > 0.0:
        return imp, float(left)
    u0, u1, u2 = (float(x) for x in u[:3])
    if kind == "linear":  # events.py:153-171
        theta = 2.0 * np.pi * u0
        mag = (params["vel_range"][0] + u1 * (params["vel_range"][1] - params["vel_range"][0])) * params["linvel"]
        imp[:3] = np.array([np.cos(theta), np.sin(theta), 0.0]) * mag * level_scale
    elif kind == "angular":  # events.py:92-108: flipped when the Bernoulli(0.5) draw is true
        mag = (params["vel_range"][0] + u1 * (params["vel_range"][1] - params["vel_range"][0])) * params["angvel"]
        imp[5] = (-mag if u0 < 0.5 else mag) * level_scale
    elif kind == "jump":  # events.py:204-231
        lo, hi = params["jump_height_range"]
        h = (lo + u0 * (hi - lo)) * level_scale
        imp[:3] = np.sqrt(2.0 * -np.asarray(gravity, dtype=np.float64) * h)
    else:
        raise ValueError(kind)
    lo, hi = params["interval_range"]
    return imp, lo + u2 * (hi - lo)


def force_push_event(params, state, dt, u, level_scale):
    """One physics substep of ForcePushEvent for one env (ksim/events.py:279-365).  `state` = (time remaining,
    force duration left, wrench(6) = force then torque); `u` = ten U[0,1) draws (force direction 3, magnitude,
    torque direction 3, case, interval, duration).  Returns (wrench applied to the body this substep, new state).
    Float32 timers like the reference (events.py:293-295)."""
    f32 = np.float32
    left, dur, wrench = state
    left, dur = f32(left) - f32(dt), f32(dur) - f32(dt)           # events.py:293-295
    wrench = np.asarray(wrench, dtype=np.float64) * level_scale   # events.py:296: rebinds the carried value
    applied = wrench * level_scale if dur > 0.0 else np.zeros(6)  # events.py:297-299
    if left <= 0.0:                                                # events.py:310-315 -> _sample_force 320-358
        u = [float(x) for x in u]
        d0, d1 = 2.0 * np.array(u[0:3]) - 1.0, 2.0 * np.array(u[4:7]) - 1.0
        s = params["force_range"][0] + u[3] * (params["force_range"][1] - params["force_range"][0])
        force = d0 / np.linalg.norm(d0) * s * params["max_force"]
        torque = d1 / np.linalg.norm(d1) * s * params["max_torque"]
        which = min(2, int(3.0 * u[7]))                            # randint(0, 3)
        wrench = np.concatenate([force if which != 1 else np.zeros(3), torque if which != 0 else np.zeros(3)])
        left = params["interval_range"][0] + u[8] * (params["interval_range"][1] - params["interval_range"][0])
        dur = params["duration_range"][0] + u[9] * (params["duration_range"][1] - params["duration_range"][0])
    return applied, (float(left), float(dur), wrench)


# ------------------------------------------------------------------ stateful observations, contact observations
def feet_contact_observation(contact_dist, foot_left, foot_right):
    """FeetContactObservation (ksim/observation.py:481-521) on sphere-floor contacts: geoms_colliding
    (ksim/utils/mujoco.py:175-217) is "a contact of the pair exists with negative distance".  Returns (c, 2)."""
    d = np.asarray(contact_dist)
    return np.stack([d[list(foot_left)] < 0.0, d[list(foot_right)] < 0.0], axis=-1).astype(np.float64)


def delayed_observation(carry, current, zero_offset=None):
    """Delayed joint observation (observation.py:228-283): emits the oldest slot, rolls, appends the current value.
    carry (delay, n).  The initial carry is the current value tiled (observation.py:231-236)."""
    carry = np.asarray(carry, dtype=np.float64)
    out = carry[0] - (0.0 if zero_offset is None else np.asarray(zero_offset))
    new = np.roll(carry, -1, axis=0)
    new[-1] = current
    return out, new


def euler_to_quat(rpy):
    """Roll-pitch-yaw to a wxyz quaternion, yaw applied last (R = Rz Ry Rx)."""
    r, p, y = (0.5 * float(a) for a in rpy)
    cr, sr, cp, sp, cy, sy = np.cos(r), np.sin(r), np.cos(p), np.sin(p), np.cos(y), np.sin(y)
    return np.array([cr * cp * cy + sr * sp * sy, sr * cp * cy - cr * sp * sy, cr * sp * cy + sr * cp * sy,
                     cr * cp * sy - sr * sp * cy])


def projected_gravity_ema(x, lag, bias, quat, gravity=(0.0, 0.0, -9.81)):
    """ProjectedGravityObservation.observe_stateful (observation.py:421-442): gravity in the sensor frame, rotated by
    the bias quaternion, averaged exponentially."""
    g = rotate_vector_by_quat(np.asarray(gravity, dtype=np.float64)[None], np.asarray(quat, dtype=np.float64)[None], inverse=True)
    g = rotate_vector_by_quat(g, euler_to_quat(bias)[None])[0]
    return np.asarray(x) * lag + g * (1.0 - lag)


# ------------------------------------------------------------------ stateful rewards
def feet_air_time_reward(contact_tcn, qvel_t, done_t, carry, *, air_steps, gnd_steps, bias=0.0, ground_penalty=0.1,
                         linvel_threshold=0.1, angvel_threshold=np.radians(10), lin_cmd_t=None, ang_cmd_t=None):
    """FeetAirTimeReward.get_reward_stateful for one env (ksim/rewards.py:1020-1085).  contact (T, c, n) of 0/1 values,
    carry = (air, gnd, stationary) integer counters per foot.  Returns ({air, gnd, stationary_gnd}: (T,), carry)."""
    contact_tn = (np.asarray(contact_tcn) > 0.5).any(axis=-2)
    T_ = contact_tn.shape[0]
    lin = (np.linalg.norm(qvel_t[:, :2], axis=-1) > linvel_threshold) if lin_cmd_t is None else np.abs(lin_cmd_t) > linvel_threshold
    ang = (qvel_t[:, 5] > angvel_threshold) if ang_cmd_t is None else np.abs(ang_cmd_t) > angvel_threshold
    moving = (lin | ang) & ~np.asarray(done_t, dtype=bool)
    air, gnd, sta = (np.asarray(c, dtype=np.int64).copy() for c in carry)
    out = {"air": np.zeros(T_), "gnd": np.zeros(T_), "stationary_gnd": np.zeros(T_)}
    for t in range(T_):
        c, mv = contact_tn[t], moving[t]
        air = np.where(~c & mv, air + 1, 0)
        gnd = np.where(c & mv, gnd + 1, 0)
        sta = np.where(c & ~mv, sta + 1, 0)
        out["air"][t] = np.where(air < air_steps, air / air_steps + bias, 0.0).max()
        out["gnd"][t] = np.where(gnd < gnd_steps, gnd / gnd_steps + bias, -ground_penalty).max()
        out["stationary_gnd"][t] = (np.clip(sta / gnd_steps, 0.0, 1.0) + bias).max()
    return out, (air, gnd, sta)


def sparse_target_height_reward(contact_tcn, position_tn3, qvel_t, done_t, carry, *, height, linvel_threshold=0.5,
                                angvel_threshold=np.radians(30)):
    """SparseTargetHeightReward.get_reward_stateful for one env (ksim/rewards.py:1160-1192): on touch-down a body earns
    the greatest height it reached since its last contact, capped at `height`."""
    contact_tn = (np.asarray(contact_tcn) > 0.5).any(axis=-2)
    still = ((np.linalg.norm(qvel_t[:, :2], axis=-1) < linvel_threshold) & (qvel_t[:, 5] < angvel_threshold)) | np.asarray(done_t, dtype=bool)
    best = np.asarray(carry, dtype=np.float64).copy()
    out = np.zeros(contact_tn.shape[0])
    for t in range(contact_tn.shape[0]):
        rew = np.minimum(np.where(contact_tn[t], best, 0.0), height)
        best = np.maximum(best, position_tn3[t][:, 2])
        best = np.where(still[t] | contact_tn[t], 0.0, best)
        out[t] = rew.max()
    return out, best


# ------------------------------------------------------------------ command tracking and rest / force penalties
def linear_velocity_reward(qpos_tq, qvel_tv, cmd_t4, vel_length_scale=0.25, yaw_length_scale=0.25, zero_threshold=0.01,
                           sq_scale=0.1, abs_scale=0.1):
    """LinearVelocityReward (ksim/rewards.py:248-272); cmd columns = (vel, yaw, xvel, yvel)."""
    lin = rotate_vector_by_quat(qvel_tv[..., :3], qpos_tq[..., 3:7], inverse=True)
    x, y = lin[..., 0], lin[..., 1]
    vel, yaw = np.hypot(x, y), np.arctan2(y, x)
    zero = np.abs(cmd_t4[..., 0]) < zero_threshold
    k = lambda d, s: exp_kernel_with_penalty(d, s, sq_scale, abs_scale)  # noqa: E731
    return {"vel": k(vel - cmd_t4[..., 0], vel_length_scale),
            "yaw": np.where(zero, 0.0, k(yaw - cmd_t4[..., 1], yaw_length_scale)),
            "x": np.where(zero, 0.0, k(x - cmd_t4[..., 2], vel_length_scale)),
            "y": np.where(zero, 0.0, k(y - cmd_t4[..., 3], vel_length_scale))}


def angular_velocity_reward(qvel_tv, cmd_t, angvel_length_scale=0.25, sq_scale=0.1, abs_scale=0.1,
                            zero_threshold=np.radians(5.0)):
    """AngularVelocityReward (rewards.py:332-347)."""
    w = qvel_tv[..., 5]
    real = np.where(np.abs(w) < zero_threshold, 0.0, np.sign(w))
    want = np.where(np.abs(cmd_t) < zero_threshold, 0.0, np.sign(cmd_t))
    return {"mag": exp_kernel_with_penalty(w - cmd_t, angvel_length_scale, sq_scale, abs_scale),
            "dir": np.where(real == want, 1.0, -1.0)}


def off_axis_velocity_reward(qvel_tv, lin_length_scale=0.25, ang_length_scale=0.25):  # rewards.py:360-372
    g = lambda v, s: np.exp(-np.square(v) / (2 * s**2))  # noqa: E731
    return {"linz": g(qvel_tv[..., 2], lin_length_scale), "angx": g(qvel_tv[..., 4], ang_length_scale),
            "angy": g(qvel_tv[..., 5], ang_length_scale)}


def motionless_at_rest_penalty(qvel_tv, linvel_moving_threshold=0.5, angvel_moving_threshold=np.radians(30)):  # rewards.py:1213-1221
    still = (np.linalg.norm(qvel_tv[..., :2], axis=-1) < linvel_moving_threshold) & (qvel_tv[..., 5] < angvel_moving_threshold)
    return np.where(still, np.linalg.norm(qvel_tv[..., 6:], axis=-1), 0.0)


def force_penalty(force_tn3, expected_weight, bias=0.0):  # rewards.py:1237-1240
    obs = np.clip(np.linalg.norm(force_tn3, axis=-1) - bias, 0.0, None)
    return np.square(obs / expected_weight).max(axis=-1)


# ------------------------------------------------------------------ commands
def linear_velocity_command(prev, qpos, qvel, u, fresh, *, min_vel, max_vel, max_yaw=0.0, zero_prob=0.0, backward_prob=0.0,
                            switch_prob=0.0, ctrl_dt, linear_accel, angular_accel):
    """One control step of LinearVelocityCommand for one env (ksim/commands.py:301-391).  prev / result =
    (vel, yaw, xvel, yvel, target_vel, target_yaw); u = draws (target speed, target yaw, zero, backward, switch);
    `fresh` = the env starts an episode (initial_command without a previous command)."""
    vel, yaw, _, _, tv, ty = (float(x) for x in prev)
    redraw = fresh or u[4] < switch_prob
    if fresh:
        lv = rotate_vector_by_quat(np.asarray(qvel[:3], dtype=np.float64)[None], np.asarray(qpos[3:7], dtype=np.float64)[None], inverse=True)[0]
        vel, yaw = float(np.hypot(lv[0], lv[1])), float(np.arctan2(lv[1], lv[0]))
    if redraw:
        tv = min_vel + u[0] * (max_vel - min_vel)
        ty = -max_yaw + u[1] * (2.0 * max_yaw)
        zero, back = u[2] < zero_prob, u[3] < backward_prob
        tv = 0.0 if zero else (-tv if back else tv)
        ty = 0.0 if zero else ty
    else:
        vel = vel + float(np.clip(tv - vel, -linear_accel, linear_accel)) * ctrl_dt
        yaw = yaw + float(np.clip(ty - yaw, -angular_accel, angular_accel)) * ctrl_dt
    return np.array([vel, yaw, vel * np.cos(yaw), vel * np.sin(yaw), tv, ty])


def angular_velocity_command(prev, qvel, u, fresh, *, max_vel, min_vel=0.0, zero_prob=0.0, switch_prob=0.0, ctrl_dt, angular_accel):
    """One control step of AngularVelocityCommand for one env (commands.py:460-507); prev / result = (vel, target_vel);
    u = draws (target speed, flip, zero, switch)."""
    vel, tv = float(prev[0]), float(prev[1])
    if fresh or u[3] < switch_prob:
        tv = min_vel + u[0] * (max_vel - min_vel)
        tv = -tv if u[1] < 0.5 else tv
        tv = 0.0 if u[2] < zero_prob else tv
        vel = float(qvel[5])
    else:
        vel = vel + float(np.clip(tv - vel, -angular_accel, angular_accel)) * ctrl_dt
    return np.array([vel, tv])


def start_pose_command(prev, qpos, fresh, quaternion=False):  # commands.py:173-215
    return np.array(qpos[3:7] if quaternion else qpos[:3], dtype=np.float64) if fresh else np.asarray(prev, dtype=np.float64)


def base_height_command(prev, u, fresh, *, min_height, max_height, switch_prob=0.005):  # commands.py:773-796
    """`u` is the single uniform draw of the step: the reference hands the same key to jax.random.uniform and to
    jax.random.bernoulli (which compares a uniform draw of that key with p), so the new height and the decision to switch
    come from one number."""
    new = min_height + u * (max_height - min_height)
    return new if (fresh or u < switch_prob) else prev


def sinusoidal_gait_command(prev, qvel, fresh, *, gait_period, ctrl_dt, max_height, height_offset=0.0, num_feet=2, stance_ratio=0.6,
                            moving_threshold=0.05):  # commands.py:696-770; the value is (moving_flag, phase, heights...)
    def heights(phase):
        per_foot = (phase + np.linspace(0.0, 1.0, num_feet, endpoint=False)) % 1.0
        progress = np.clip((per_foot - stance_ratio) / (1.0 - stance_ratio), 0.0, 1.0)
        return np.where(per_foot >= stance_ratio, max_height * np.sin(np.pi * progress), 0.0) + height_offset

    if fresh:
        return np.concatenate([[1.0, 0.0], heights(0.0)])
    flag, phase = prev[0], prev[1]
    new_phase = (phase + ctrl_dt / gait_period) % 1.0 if flag else 0.0
    moving = np.linalg.norm(qvel[:2]) > moving_threshold
    flag = flag if moving else 0.0
    new_phase = new_phase if moving else 0.0
    return np.concatenate([[flag, new_phase], heights(new_phase)])


def joint_position_command(prev, qpos, u, fresh, *, indices, ranges, ctrl_dt, min_time, max_time):
    """One control step of JointPositionCommand for one env (ksim/commands.py:852-893), in float32 like the reference.
    prev / result = start (n), target (n), total_time, num_steps, step_id; u = draws (one per target, then the time)."""
    f = np.float32
    n = len(indices)
    prev = np.asarray(prev, dtype=f)
    step_id = prev[2 * n + 2] + f(1)
    if fresh or step_id > prev[2 * n + 1]:
        lo, hi = np.asarray(ranges, dtype=f).T
        target = lo + np.asarray(u[:n], dtype=f) * (hi - lo)
        start = np.asarray(qpos, dtype=f)[7 + np.asarray(indices)]
        total = f(min_time) + f(u[n]) * (f(max_time) - f(min_time))
        return np.concatenate([start, target, [total, np.ceil(total / f(ctrl_dt)), f(0)]]).astype(f)
    out = prev.copy()
    out[2 * n + 2] = step_id
    return out


def cartesian_coordinate_command(prev, u, fresh, *, box_min, box_max, dt, min_speed=0.5, max_speed=3.0, switch_prob=0.0, jump_prob=0.0,
                                 curriculum_scale=0.1, level=1.0):
    """One control step of CartesianCoordinateCommand for one env (ksim/commands.py:556-656).  prev / result = current (3),
    target (3), speed; u = draws (box point x, y, z; speed; switch / jump, which share one key in the reference)."""
    lo, hi = np.asarray(box_min, dtype=np.float64), np.asarray(box_max, dtype=np.float64)
    centre, half = (lo + hi) / 2.0, (hi - lo) / 2.0 * (curriculum_scale * level + 1.0)
    point = (centre - half) + np.asarray(u[:3], dtype=np.float64) * (2.0 * half)
    new_speed = min_speed + u[3] * (max_speed - min_speed)
    if fresh:
        return np.concatenate([point, point, [new_speed]])
    prev = np.asarray(prev, dtype=np.float64)
    current, target, speed = prev[:3], prev[3:6], prev[6]
    distance = np.linalg.norm(target - current)
    reached = distance < dt * speed * 0.5
    if (reached and u[4] < switch_prob) or u[4] < jump_prob:
        target, speed = point, new_speed
    direction = target - current
    norm = np.linalg.norm(direction)
    direction = direction / norm if norm > 0 else direction
    return np.concatenate([current + direction * min(speed * dt, distance), target, [speed]])


def sinusoidal_gait_reward(position_tn3, height_tn, max_height):  # rewards.py:1331-1335
    return 1.0 - np.abs(np.asarray(position_tn3, dtype=np.float64)[..., 2] - np.asarray(height_tn, dtype=np.float64)).sum(axis=-1) / max_height


def position_velocity_actuator_torque(action, qpos, qvel, kp, kd, ctrl_clip, pos_noise=0.0, vel_noise=0.0, torque_noise=0.0):
    """PositionVelocityActuator.get_ctrl (ksim/actuators.py:261-293): action = (position targets, velocity targets)."""
    n = len(qpos)
    action = np.asarray(action, dtype=np.float64)
    target_pos, target_vel = action[:n] + pos_noise, action[n:] + vel_noise
    ctrl = np.asarray(kp) * (target_pos - qpos) + np.asarray(kd) * (target_vel - qvel)
    return np.clip(ctrl + torque_noise, -np.asarray(ctrl_clip), np.asarray(ctrl_clip))


def mixture_head(raw, num_mixtures, *, min_std, max_std, var_scale=1.0, mean_bias=None, clip_lo=None, clip_hi=None,
                 uniform=None, normal=None, deterministic=False, clip_max=1e3):
    """Mixture-of-Gaussians actor head (examples/walking.py:127-144): raw (N, 3 nu K) -> component means (zero bias, joint
    range clip), deviations (softplus, floor, scale, cap) and logits, each (N, nu, K).  One component per action dimension
    by inverse CDF of softmax(logits) at the uniform draw, action = mean_k + std_k z; log-probability of the sample under
    the mixture; NaN scrub and clip (ksim/task/rl.py:998-1001).  xax.MixtureOfGaussians is third-party and absent: this is
    the textbook mixture, pinned by scipy (logsumexp of norm.logpdf), unit mass and the K = 1 reduction to a Gaussian.
    Returns (action, log_prob, component)."""
    raw = np.asarray(raw, np.float64)
    K = int(num_mixtures)
    N, nu = raw.shape[0], raw.shape[1] // (3 * K)
    mean = raw[:, : nu * K].reshape(N, nu, K)
    rstd = raw[:, nu * K: 2 * nu * K].reshape(N, nu, K)
    logit = raw[:, 2 * nu * K:].reshape(N, nu, K)
    if mean_bias is not None:
        mean = mean + np.asarray(mean_bias, np.float64)[None, :, None]
    if clip_lo is not None:
        mean = np.clip(mean, np.asarray(clip_lo, np.float64)[None, :, None], np.asarray(clip_hi, np.float64)[None, :, None])
    std = np.minimum((np.logaddexp(0.0, rstd) + min_std) * var_scale, max_std)
    logw = logit - np.logaddexp.reduce(logit, axis=-1, keepdims=True)
    if deterministic:
        comp = np.argmax(logit, axis=-1)
        action = np.take_along_axis(mean, comp[..., None], -1)[..., 0]
    else:
        cum = np.cumsum(np.exp(logw), axis=-1)
        comp = np.minimum((cum <= np.asarray(uniform, np.float64)[..., None]).sum(-1), K - 1)
        pm = np.take_along_axis(mean, comp[..., None], -1)[..., 0]
        ps = np.take_along_axis(std, comp[..., None], -1)[..., 0]
        action = pm + ps * np.asarray(normal, np.float64)
    d = (action[..., None] - mean) / std
    logp = np.logaddexp.reduce(logw - 0.5 * d * d - np.log(std) - 0.5 * np.log(2 * np.pi), axis=-1)
    action = np.clip(np.where(np.isnan(action), 0.0, action), -clip_max, clip_max)
    return action, logp, comp


# --------------------------------------------------------------------------- action filters (ksim/actions.py)
def lowpass_one_pole(x, y_last, ctrl_dt, fc):  # actions.py:248-257
    alpha = ctrl_dt / (1.0 / (2.0 * np.pi * fc) + ctrl_dt)
    return np.asarray(y_last, np.float64) + alpha * (np.asarray(x, np.float64) - y_last)


def lowpass_scan(x, ctrl_dt, fc, y0=None, fresh=None):
    """The filter threaded through a trajectory as the K-Bot task's scan does (examples/kbot/train.py:1439-1451, 1506-1533):
    x (T, ..., n); the state starts at y0 (zeros when None) and is the initial one, zero, at the steps flagged in `fresh`
    (T, ...) (the step after a done one: the carry was replaced by the initial carry).  Returns (y (T, ..., n), last state)."""
    x = np.asarray(x, np.float64)
    last = np.zeros(x.shape[1:]) if y0 is None else np.array(y0, dtype=np.float64)
    out = np.empty_like(x)
    for t in range(x.shape[0]):
        if fresh is not None:
            last = np.where(np.asarray(fresh[t], bool)[..., None], 0.0, last)
        last = lowpass_one_pole(x[t], last, ctrl_dt, fc)
        out[t] = last
    return out, last


def lowpass_scan_backward(dy, ctrl_dt, fc, fresh=None):
    """Reverse-mode derivative of `lowpass_scan`, written out: from dL/dy (T, ..., n) to (dL/dx, dL/dy0).
    y_t = (1 - a) y_{t-1} + a x_t, so the gradient reaching y_t is G_t = dy_t + (1 - a) G_{t+1} unless step t + 1 is fresh
    (its y_{t} input was replaced by zero), and dL/dx_t = a G_t; dL/dy0 = (1 - a) G_0 unless step 0 is fresh."""
    dy = np.asarray(dy, np.float64)
    a = ctrl_dt / (1.0 / (2.0 * np.pi * fc) + ctrl_dt)
    dx = np.empty_like(dy)
    carry = np.zeros(dy.shape[1:])
    for t in range(dy.shape[0] - 1, -1, -1):
        G = dy[t] + carry
        dx[t] = a * G
        carry = (1.0 - a) * G
        if fresh is not None:
            carry = np.where(np.asarray(fresh[t], bool)[..., None], 0.0, carry)
    return dx, carry


def clip_acceleration(target, position, velocity, max_acceleration, ctrl_dt):  # actions.py:54-80: (position, velocity)
    target, position, velocity = (np.asarray(a, np.float64) for a in (target, position, velocity))
    cur_v = (target - position) / ctrl_dt
    acc = np.clip((cur_v - velocity) / ctrl_dt, -max_acceleration, max_acceleration)
    nv = velocity + acc * ctrl_dt
    return position + nv * ctrl_dt, nv


def integrate_velocity(velocity, position, ctrl_dt):  # actions.py:108-133
    return np.asarray(position, np.float64) + np.asarray(velocity, np.float64) * ctrl_dt


def integrate_acceleration(acceleration, position, velocity, ctrl_dt, max_velocity=10.0):  # actions.py:162-191
    nv = np.clip(np.asarray(velocity, np.float64) + np.asarray(acceleration, np.float64) * ctrl_dt, -max_velocity, max_velocity)
    return np.asarray(position, np.float64) + nv * ctrl_dt, nv


def clip_positions(x, lo, hi):  # actions.py:211-213
    return np.clip(np.asarray(x, np.float64), lo, hi)


def tanh_positions(x, lo, hi):  # actions.py:234-237 (the image is lo + (hi - lo) tanh x, as written there)
    return np.tanh(np.asarray(x, np.float64)) * (np.asarray(hi) - np.asarray(lo)) + np.asarray(lo)


# --------------------------------------------------------------------------- site sensors (MuJoCo gyro / accelerometer)
def site_gyro(xquat_body, omega_world, site_quat):
    """MuJoCo's gyro: the body's angular velocity in the site frame, (q_body q_site)^-1 w (what SensorObservation reads
    from sensordata, ksim/observation.py:307-340)."""
    in_body = rotate_vector_by_quat(np.asarray(omega_world, np.float64), np.asarray(xquat_body, np.float64), inverse=True)
    return rotate_vector_by_quat(in_body, np.asarray(site_quat, np.float64), inverse=True)


def site_accelerometer(qacc6, xquat_body, omega_world, site_pos, site_quat, gravity):
    """MuJoCo's accelerometer for a site on the floating base: the site's acceleration minus gravity, in the site frame.
    qacc6 = the free joint's accelerations (origin acceleration in world axes, angular acceleration in body axes)."""
    qacc6, q = np.asarray(qacc6, np.float64), np.asarray(xquat_body, np.float64)
    w = np.asarray(omega_world, np.float64)
    r = rotate_vector_by_quat(np.asarray(site_pos, np.float64), q)
    alpha = rotate_vector_by_quat(qacc6[..., 3:6], q)
    a = qacc6[..., :3] + np.cross(alpha, r) + np.cross(w, np.cross(w, r)) - np.asarray(gravity, np.float64)
    return rotate_vector_by_quat(rotate_vector_by_quat(a, q, inverse=True), np.asarray(site_quat, np.float64), inverse=True)


def site_frame_position(xpos_body, xquat_body, site_pos):
    """MuJoCo's framepos sensor of a site: the site's origin in world coordinates, x_body + R_body r."""
    return np.asarray(xpos_body, np.float64) + rotate_vector_by_quat(np.asarray(site_pos, np.float64), np.asarray(xquat_body, np.float64))


def site_frame_quaternion(xquat_body, site_quat):
    """MuJoCo's framequat sensor of a site: its world orientation q_body q_site (w, x, y, z)."""
    return quat_mul(np.asarray(xquat_body, np.float64), np.asarray(site_quat, np.float64))


def site_magnetometer(xquat_body, site_quat, magnetic):
    """MuJoCo's magnetometer: the model's (constant, world-frame) magnetic field seen in the site frame."""
    in_body = rotate_vector_by_quat(np.asarray(magnetic, np.float64), np.asarray(xquat_body, np.float64), inverse=True)
    return rotate_vector_by_quat(in_body, np.asarray(site_quat, np.float64), inverse=True)


# ------------------------------------------------------------------ resets (ksim/resets.py), one env, explicit draws
def xy_position_reset(qpos, ux, uy, *, x_range, y_range, padded_bounds, z=None, hfield=None, hfield_bounds=None,
                      robot_base_height=0.0):
    """PlaneXYPositionReset (resets.py:93-120) with `z` = the plane's height, or HFieldXYPositionReset (resets.py:45-90)
    with `hfield` (nx, ny) and `hfield_bounds` = (x_bound, y_bound, z_top).  ux, uy in [-1, 1)."""
    lower_x, upper_x, lower_y, upper_y = padded_bounds
    q = np.array(qpos, dtype=np.float64)
    q[0] = np.clip(ux * x_range, lower_x, upper_x)
    q[1] = np.clip(uy * y_range, lower_y, upper_y)
    if hfield is None:
        q[2] = z + robot_base_height
        return q
    x_bound, y_bound, z_top = hfield_bounds
    nx, ny = hfield.shape
    ix = int(np.clip(np.int32(((q[0] + x_bound) / (2 * x_bound)) * (nx - 1)), 0, nx - 1))
    iy = int(np.clip(np.int32(((q[1] + y_bound) / (2 * y_bound)) * (ny - 1)), 0, ny - 1))
    q[2] = hfield[ix, iy] + z_top + robot_base_height
    return q


def initial_motion_state_reset(qpos, frame, motion_qpos, ctrl_dt, freejoint):
    """InitialMotionStateReset (resets.py:284-306): returns (qpos, time)."""
    q = np.array(qpos, dtype=np.float64)
    ref = np.asarray(motion_qpos, dtype=np.float64)[frame % len(motion_qpos)]
    if freejoint:
        q[:] = ref
    else:
        q[7:] = ref[7:]
    return q, frame * ctrl_dt


def random_heading_reset(qpos, u):
    """RandomHeadingReset (resets.py:309-320): quat <- quat * yaw, yaw = pi u, u in [-1, 1)."""
    q = np.array(qpos, dtype=np.float64)
    q[3:7] = quat_mul(q[3:7], euler_to_quat(np.array([0.0, 0.0, np.pi * u])))
    return q


def random_pitch_roll_reset(qpos, u01, pitch_range, roll_range):
    """RandomPitchRollReset (resets.py:338-354): both angles come from the SAME key, hence from one uniform number
    u01 in [0, 1): pitch = min_p + u (max_p - min_p), roll = min_r + u (max_r - min_r); quat <- quat * euler(roll, pitch, 0)."""
    q = np.array(qpos, dtype=np.float64)
    pitch = pitch_range[0] + u01 * (pitch_range[1] - pitch_range[0])
    roll = roll_range[0] + u01 * (roll_range[1] - roll_range[0])
    q[3:7] = quat_mul(q[3:7], euler_to_quat(np.array([roll, pitch, 0.0])))
    return q


# ------------------------------------------------------------------ symmetry and joint-position rewards
def symmetry_reward(qpos_tq, carry, done_last, joint_indices, joint_targets, alpha=0.1):
    """SymmetryReward.get_reward_stateful (rewards.py:868-877) with the carry restart of get_rewards (rl.py:206-214):
    returns (reward (T,), new carry)."""
    targets = np.asarray(joint_targets, dtype=np.float64)
    carry = targets.copy() if done_last else np.asarray(carry, dtype=np.float64)
    q = np.asarray(qpos_tq, dtype=np.float64)[:, np.asarray(joint_indices) + 7] - targets
    new = carry * (1.0 - alpha) + q.mean(axis=0) * alpha
    return (q * -new[None, :]).sum(axis=-1), new


def pairwise_symmetry_reward(qpos_tq, carry, done_last, left, right, left_zero=0.0, right_zero=0.0, flipped=False, alpha=0.1,
                             kernel_scale=0.25, sq_scale=0.1, abs_scale=0.1):
    """PairwiseSymmetryReward.get_reward_stateful (rewards.py:916-936): returns ({"lr", "self"} each (T,), new carry)."""
    carry = np.array([left_zero, right_zero], dtype=np.float64) if done_last else np.asarray(carry, dtype=np.float64)
    q = np.asarray(qpos_tq, dtype=np.float64)
    ql, qr = q[:, left + 7] - left_zero, q[:, right + 7] - right_zero
    if flipped:
        qr = -qr
    lr = exp_kernel_with_penalty(ql - qr, kernel_scale, sq_scale, abs_scale)
    pair = np.stack([ql, qr], axis=-1)
    new = carry * (1.0 - alpha) + pair.mean(axis=0) * alpha
    return {"lr": lr, "self": (pair * -new[None, :]).sum(axis=-1)}, new


def joint_position_reward(qpos_tq, qvel_tv, start, target, total_time, num_steps, step_id, indices, pos_scale=0.25,
                          vel_scale=0.25, sq_scale=0.1, abs_scale=0.1):
    """JointPositionReward.get_reward (rewards.py:1366-1380) with JointPositionCommandValue.current_position / velocity
    (commands.py:803-818).  start, target: (T, n); total_time, num_steps, step_id: (T,)."""
    idx = np.asarray(indices)
    cur_pos = start + (target - start) * (step_id / num_steps)[:, None]
    cur_vel = (target - start) / total_time[:, None]
    pos = exp_kernel_with_penalty(cur_pos - np.asarray(qpos_tq)[:, idx + 7], pos_scale, sq_scale, abs_scale)
    vel = exp_kernel_with_penalty(cur_vel - np.asarray(qvel_tv)[:, idx + 6], vel_scale, sq_scale, abs_scale)
    return {"pos": pos.mean(axis=-1), "vel": vel.mean(axis=-1)}


# ------------------------------------------------------------------ IMU mounting error, site orientation, contact list
def imu_alignment_offset(rx, ry, rz=0.0):
    """IMUAlignmentRandomizer's rotation offset (ksim/randomization.py:262-271): small-angle quaternions [1, angle / 2]
    about x, y, z composed as qz * (qy * qx), normalised."""
    qx, qy, qz = np.array([1.0, 0.5 * rx, 0.0, 0.0]), np.array([1.0, 0.0, 0.5 * ry, 0.0]), np.array([1.0, 0.0, 0.0, 0.5 * rz])
    q = quat_mul(qz, quat_mul(qy, qx))
    return q / np.linalg.norm(q)


def quat_to_matrix(q):
    w, x, y, z = (float(v) for v in np.asarray(q, dtype=np.float64) / np.linalg.norm(q))
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


def site_rotation6d(xquat_body, site_quat):
    """SiteOrientationObservation (ksim/observation.py:664-669): site_xmat = R(q_body q_site), then its 6-D form, taken
    here as the first two rows, row-major."""
    return quat_to_matrix(quat_mul(np.asarray(xquat_body, np.float64), np.asarray(site_quat, np.float64)))[:2].reshape(6)


def contact_observation(contact_dist, geom_idxs, floor=-1):
    """ContactObservation (ksim/observation.py:452-478) for sphere-against-floor collisions: entry i says whether geom i
    touches another geom of the list.  Spheres never touch each other."""
    dist = np.asarray(contact_dist)
    has_floor = floor in geom_idxs
    spheres = [g for g in geom_idxs if g != floor]
    out = []
    for g in geom_idxs:
        if g == floor:
            out.append(any(dist[s] < 0 for s in spheres))
        else:
            out.append(bool(has_floor and dist[g] < 0))
    return np.array(out)
