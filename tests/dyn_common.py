"""Shared helpers of the dynamics parity tests: seeded env states and oracle drivers."""
import numpy as np

from ksim_amd import model as km
from oracle.dyn import Oracle


def random_states(m, N, seed, contact_fraction=0.5, vel_scale=0.5, joint_range=0.6):
    """Seeded env states; a fraction of the free-root envs is sunk so that contact spheres penetrate."""
    rng = np.random.default_rng(seed)
    qpos = np.tile(m.qpos0, (N, 1))
    qvel = rng.normal(size=(N, m.nv)) * vel_scale
    a = m.arrays()
    for e in range(N):
        for b in range(1, m.nb):
            qa = m.body_qadr[b]
            if m.body_jtype[b] == km.JNT_FREE:
                qpos[e, qa:qa + 2] += rng.normal(size=2) * 0.3
                q = np.array([1.0, 0, 0, 0]) + rng.normal(size=4) * 0.15
                qpos[e, qa + 3:qa + 7] = q / np.linalg.norm(q)
            else:
                qpos[e, qa] = rng.uniform(-joint_range, joint_range)
        if m.ns and m.has_free_root and rng.random() < contact_fraction:
            kin = km.host_kinematics(a, qpos[e])
            low = min(kin["xpos"][b][2] + (kin["xmat"][b] @ p)[2] - r
                      for b, p, r in zip(m.sph_body, m.sph_pos, m.sph_radius))
            qpos[e, 2] -= low + rng.uniform(0.0, 0.01)
    return qpos, qvel


def oracle_forward(m, qpos, qvel, ctrl=None, friction=None, mass_scale=None, warm=None, dtype=np.float64, steps=0):
    """Runs the oracle env by env; returns a dict of stacked arrays (after `steps` full steps, then a forward)."""
    orc = Oracle(m.arrays(), dtype)
    N = qpos.shape[0]
    keys = ("qpos", "qvel", "qacc", "qacc_smooth", "qfrc_bias", "M", "con_dist", "xpos", "xquat", "cvel",
            "qacc_warmstart", "cinert", "cfrc_ext")
    out = {k: [] for k in keys}
    out["nefc"], out["niter"] = [], []
    for e in range(N):
        d = orc.data(qpos[e], qvel[e], friction=None if friction is None else friction[e],
                     mass_scale=None if mass_scale is None else mass_scale[e])
        if ctrl is not None:
            d.ctrl = ctrl[e]
        if warm is not None:
            d.qacc_warmstart = warm[e]
        for _ in range(steps):
            orc.step(d)
        orc.forward(d)
        for k in keys:
            out[k].append(np.array(getattr(d, k), dtype=np.float64).reshape(-1))
        out["nefc"].append(d.nefc)
        out["niter"].append(d.solver_niter)
    return {k: np.array(v) for k, v in out.items()}


def rel_err(got, want, floor=1e-3):
    """Per-env max abs error relative to the env's max magnitude (floored)."""
    got = np.asarray(got, dtype=np.float64).reshape(len(want), -1)
    want = np.asarray(want, dtype=np.float64).reshape(len(want), -1)
    scale = np.maximum(np.abs(want).max(axis=1), floor)
    return np.abs(got - want).max(axis=1) / scale
