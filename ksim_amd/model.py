"""Kinematic-tree physics model (the subset of MuJoCo's MjModel the rollout hot path needs).

The reference hands ``mjx.Model`` objects built by ``mjx.put_model`` (ksim/utils/mujoco.py:388-391)
to its engine (ksim/engine.py:205-361).  MuJoCo is not a dependency here: models are described
with :class:`ModelBuilder` (bodies in depth-first order, one free or hinge joint per body, motor
actuators, contact spheres against the ground plane z = 0) and frozen into a
:class:`KinematicModel` of flat numpy arrays that is uploaded once to the GPU.

The constants MuJoCo derives at compile time (``body_invweight0``, ``stat.meaninertia``) are
computed here on the host in float64 at ``qpos0`` from brute-force Jacobians.
"""
from __future__ import annotations

from dataclasses import dataclass, field, fields
from typing import Sequence

import numpy as np

JNT_NONE, JNT_FREE, JNT_HINGE = 0, 1, 2

MAX_BODIES = 32
MAX_QPOS = 40
MAX_DOFS = 32
MAX_ACTUATORS = 32
MAX_SPHERES = 16


# --------------------------------------------------------------------------- small math (host, float64)
def quat_mul(a, b):
    aw, ax, ay, az = a
    bw, bx, by, bz = b
    return np.array([
        aw * bw - ax * bx - ay * by - az * bz,
        aw * bx + ax * bw + ay * bz - az * by,
        aw * by - ax * bz + ay * bw + az * bx,
        aw * bz + ax * by - ay * bx + az * bw,
    ])


def quat_to_mat(q):
    w, x, y, z = q
    return np.array([
        [w * w + x * x - y * y - z * z, 2 * (x * y - w * z), 2 * (x * z + w * y)],
        [2 * (x * y + w * z), w * w - x * x + y * y - z * z, 2 * (y * z - w * x)],
        [2 * (x * z - w * y), 2 * (y * z + w * x), w * w - x * x - y * y + z * z],
    ])


def axis_angle_quat(axis, angle):
    axis = np.asarray(axis, dtype=np.float64)
    return np.concatenate([[np.cos(angle / 2)], axis * np.sin(angle / 2)])


def quat_z_to(direction):
    """Shortest-arc quaternion rotating +z onto ``direction``."""
    d = np.asarray(direction, dtype=np.float64)
    d = d / np.linalg.norm(d)
    z = np.array([0.0, 0.0, 1.0])
    c = float(z @ d)
    if c > 1 - 1e-12:
        return np.array([1.0, 0.0, 0.0, 0.0])
    if c < -1 + 1e-12:
        return np.array([0.0, 1.0, 0.0, 0.0])
    axis = np.cross(z, d)
    axis /= np.linalg.norm(axis)
    return axis_angle_quat(axis, np.arccos(c))


def capsule_inertia(mass: float, radius: float, length: float):
    """Principal inertia (about the centre, axis = z) of a capsule with cylinder ``length``."""
    r, h = radius, length
    v_cyl = np.pi * r * r * h
    v_sph = 4.0 / 3.0 * np.pi * r**3
    m_cyl = mass * v_cyl / (v_cyl + v_sph)
    m_sph = mass - m_cyl
    izz = m_cyl * r * r / 2 + m_sph * 2 * r * r / 5
    ixx = m_cyl * (h * h / 12 + r * r / 4) + m_sph * (2 * r * r / 5 + h * h / 4 + 3 * h * r / 8)
    return np.array([ixx, ixx, izz])


# --------------------------------------------------------------------------- frozen model
@dataclass(frozen=True, eq=False)
class KinematicModel:
    nb: int
    nq: int
    nv: int
    nu: int
    ns: int
    # options (ksim/task/rl.py:555-578,717-748 sets the same MuJoCo options)
    dt: float
    gravity: np.ndarray
    iterations: int
    ls_iterations: int
    tolerance: float
    ls_tolerance: float
    impratio: float
    eulerdamp: bool
    condim: int  # 3: friction pyramid; 1: frictionless contacts (MuJoCo condim of every sphere-floor pair)
    solref: np.ndarray
    solimp: np.ndarray
    friction: float
    # bodies
    body_parent: np.ndarray
    body_jtype: np.ndarray
    body_qadr: np.ndarray
    body_dofadr: np.ndarray
    body_subtree_end: np.ndarray
    body_pos: np.ndarray
    body_quat: np.ndarray
    body_mass: np.ndarray
    body_ipos: np.ndarray
    body_iquat: np.ndarray
    body_inertia: np.ndarray
    jnt_axis: np.ndarray
    jnt_pos: np.ndarray
    qpos0: np.ndarray
    # dofs
    dof_body: np.ndarray
    dof_parent: np.ndarray
    dof_damping: np.ndarray
    dof_armature: np.ndarray
    # joint limits of hinges, by body (MuJoCo jnt_limited / jnt_range), and dry joint friction (dof_frictionloss)
    jnt_limited: np.ndarray
    jnt_range: np.ndarray
    dof_frictionloss: np.ndarray
    # solref / solimp of the limit and friction rows (MuJoCo: per joint, its defaults here unless given)
    dof_solref: np.ndarray
    dof_solimp: np.ndarray
    dof_stiffness: np.ndarray  # joint springs of hinges about qpos0
    # actuators (motors: force = gear * clip(ctrl, ctrlrange))
    act_dof: np.ndarray
    act_gear: np.ndarray
    act_ctrlrange: np.ndarray
    # contact spheres against the plane z = 0
    sph_body: np.ndarray
    sph_pos: np.ndarray
    sph_radius: np.ndarray
    # derived constants
    body_invweight0: np.ndarray
    dof_invweight0: np.ndarray
    meaninertia: float
    body_names: tuple = field(default=())
    sph_names: tuple = field(default=())  # collision geom of each contact sphere (both ends of a capsule carry its name)
    sites: dict = field(default_factory=dict)    # name -> (body, position (3), orientation wxyz (4)) in the body frame
    sensors: dict = field(default_factory=dict)  # name -> (MuJoCo sensor type, site name)
    magnetic: tuple = (0.0, -0.5, 0.0)           # the magnetic field a magnetometer reads (MuJoCo option `magnetic`, its default)

    @property
    def has_free_root(self) -> bool:
        return self.nb > 1 and int(self.body_jtype[1]) == JNT_FREE

    @property
    def max_depth(self) -> int:
        depth = np.zeros(self.nb, dtype=int)
        for b in range(1, self.nb):
            depth[b] = depth[self.body_parent[b]] + 1
        return int(depth.max())

    def arrays(self) -> dict:
        """All fields as plain python / numpy values (for checkers and serialisation)."""
        return {f.name: getattr(self, f.name) for f in fields(self)}

    def __hash__(self) -> int:  # engines holding a model must stay hashable like the reference's
        return id(self)


class ModelBuilder:
    """Incrementally describes a kinematic tree; bodies must be added in depth-first order."""

    def __init__(self, dt=0.005, gravity=(0.0, 0.0, -9.81), iterations=8, ls_iterations=8, tolerance=1e-10,
                 ls_tolerance=0.01, impratio=1.0, eulerdamp=False, solref=(0.02, 1.0),
                 solimp=(0.9, 0.95, 0.001, 0.5, 2.0), friction=1.0, integrator=None, dof_solref=None, dof_solimp=None,
                 condim=3, magnetic=(0.0, -0.5, 0.0)):
        # integrator: "euler" (explicit joint damping unless `eulerdamp`) or "implicitfast", the one ksim sets
        # (ksim/task/rl.py:555-578).  With torque motors the only velocity-dependent smooth force is joint damping, so
        # implicitfast is the damping-implicit velocity update, (M + dt diag(damping)) a = M qacc.
        if integrator not in (None, "euler", "implicitfast"):
            raise ValueError(f"unknown integrator {integrator!r}")
        eulerdamp = bool(eulerdamp) or integrator == "implicitfast"
        if int(condim) not in (1, 3):
            raise ValueError(f"condim {condim}: contacts are frictionless (1) or pyramidal (3)")
        self.opt = dict(dt=float(dt), gravity=np.array(gravity, dtype=np.float64), iterations=int(iterations),
                        ls_iterations=int(ls_iterations), tolerance=float(tolerance),
                        ls_tolerance=float(ls_tolerance), impratio=float(impratio), eulerdamp=bool(eulerdamp),
                        solref=np.array(solref, dtype=np.float64), solimp=np.array(solimp, dtype=np.float64),
                        friction=float(friction), condim=int(condim),
                        dof_solref=np.array(solref if dof_solref is None else dof_solref, dtype=np.float64),
                        dof_solimp=np.array(solimp if dof_solimp is None else dof_solimp, dtype=np.float64))
        self.magnetic = tuple(float(x) for x in magnetic)
        self.bodies = [dict(parent=-1, jtype=JNT_NONE, pos=np.zeros(3), quat=np.array([1.0, 0, 0, 0]), mass=0.0,
                            ipos=np.zeros(3), iquat=np.array([1.0, 0, 0, 0]), inertia=np.zeros(3),
                            axis=np.array([0.0, 0, 1]), jpos=np.zeros(3), damping=0.0, armature=0.0, qpos0=0.0,
                            range=None, frictionloss=0.0, stiffness=0.0, name="world")]
        self.actuators: list[dict] = []
        self.spheres: list[dict] = []
        self.sites: dict = {}
        self.sensors: dict = {}

    def add_body(self, parent: int, pos, *, joint: str | None = "hinge", axis=(0.0, 1.0, 0.0),
                 joint_pos=(0.0, 0.0, 0.0), quat=(1.0, 0.0, 0.0, 0.0), mass: float, ipos=(0.0, 0.0, 0.0),
                 iquat=(1.0, 0.0, 0.0, 0.0), inertia, damping=0.0, armature=0.0, range=None, frictionloss=0.0,
                 stiffness=0.0, name: str | None = None) -> int:
        b = len(self.bodies)
        if not (0 <= parent < b):
            raise ValueError(f"parent {parent} does not exist")
        # depth-first order: the parent must be the previous body or one of its ancestors
        anc = b - 1
        while anc != parent and anc > 0:
            anc = self.bodies[anc]["parent"]
        if anc != parent and parent != 0:
            raise ValueError("bodies must be added in depth-first order (parent on the current path)")
        jtype = {None: JNT_NONE, "none": JNT_NONE, "free": JNT_FREE, "hinge": JNT_HINGE}[joint]
        if jtype == JNT_FREE and parent != 0:
            raise ValueError("a free joint must attach to the world")
        if jtype == JNT_NONE:
            raise ValueError("every body needs a free or hinge joint in this model subset")
        if range is not None:
            if jtype != JNT_HINGE:
                raise ValueError("joint limits apply to hinge joints")
            if not (float(range[0]) < float(range[1])):
                raise ValueError(f"joint range {range} is empty")
            range = (float(range[0]), float(range[1]))
        if frictionloss < 0 or (frictionloss > 0 and jtype != JNT_HINGE):
            raise ValueError("frictionloss is a non-negative property of hinge joints")
        ax = np.array(axis, dtype=np.float64)
        ax /= np.linalg.norm(ax)
        q = np.array(quat, dtype=np.float64)
        iq = np.array(iquat, dtype=np.float64)
        self.bodies.append(dict(parent=parent, jtype=jtype, pos=np.array(pos, dtype=np.float64),
                                quat=q / np.linalg.norm(q), mass=float(mass), ipos=np.array(ipos, dtype=np.float64),
                                iquat=iq / np.linalg.norm(iq), inertia=np.array(inertia, dtype=np.float64), axis=ax,
                                jpos=np.array(joint_pos, dtype=np.float64), damping=float(damping),
                                armature=float(armature), qpos0=0.0, range=range, frictionloss=float(frictionloss),
                                stiffness=float(stiffness), name=name or f"body{b}"))
        return b

    def add_capsule_body(self, parent: int, pos, direction, length: float, radius: float, mass: float, **kw) -> int:
        """Body whose mass is a capsule from its origin along ``direction`` (body frame)."""
        d = np.asarray(direction, dtype=np.float64)
        d = d / np.linalg.norm(d)
        return self.add_body(parent, pos, mass=mass, ipos=d * (length / 2), iquat=quat_z_to(d),
                             inertia=capsule_inertia(mass, radius, length), **kw)

    def add_actuator(self, body: int, gear: float = 1.0, ctrlrange: tuple[float, float] | None = None) -> int:
        if self.bodies[body]["jtype"] != JNT_HINGE:
            raise ValueError("actuators drive hinge joints")
        lo, hi = (-np.inf, np.inf) if ctrlrange is None else ctrlrange
        self.actuators.append(dict(body=body, gear=float(gear), lo=float(lo), hi=float(hi)))
        return len(self.actuators) - 1

    def add_contact_sphere(self, body: int, pos, radius: float, name: str | None = None) -> int:
        """`name`: the collision geom the sphere comes from; the two end spheres of a capsule share their geom's name."""
        self.spheres.append(dict(body=body, pos=np.array(pos, dtype=np.float64), radius=float(radius),
                                 name=name or f"sphere{len(self.spheres)}"))
        return len(self.spheres) - 1

    def add_site(self, name: str, body: int, pos=(0.0, 0.0, 0.0), quat=(1.0, 0.0, 0.0, 0.0)) -> None:
        q = np.array(quat, dtype=np.float64)
        self.sites[name] = (int(body), tuple(float(v) for v in pos), tuple(q / np.linalg.norm(q)))

    def add_sensor(self, name: str, kind: str, site: str) -> None:
        if site not in self.sites:
            raise ValueError(f"sensor {name!r} refers to the unknown site {site!r}")
        self.sensors[name] = (kind, site)

    def build(self) -> KinematicModel:
        nb = len(self.bodies)
        qadr, dofadr = np.full(nb, -1, np.int32), np.full(nb, -1, np.int32)
        nq = nv = 0
        for b, body in enumerate(self.bodies):
            if body["jtype"] == JNT_FREE:
                qadr[b], dofadr[b] = nq, nv
                nq, nv = nq + 7, nv + 6
            elif body["jtype"] == JNT_HINGE:
                qadr[b], dofadr[b] = nq, nv
                nq, nv = nq + 1, nv + 1
        nu, ns = len(self.actuators), len(self.spheres)
        if nb > MAX_BODIES or nq > MAX_QPOS or nv > MAX_DOFS or nu > MAX_ACTUATORS or ns > MAX_SPHERES:
            raise ValueError(f"model too large: nb={nb} nq={nq} nv={nv} nu={nu} ns={ns}")
        parent = np.array([b["parent"] for b in self.bodies], np.int32)
        subtree_end = np.arange(1, nb + 1, dtype=np.int32)
        for b in range(nb - 1, 0, -1):
            subtree_end[parent[b]] = max(subtree_end[parent[b]], subtree_end[b])
        dof_body, dof_parent = np.zeros(nv, np.int32), np.full(nv, -1, np.int32)
        damping, armature, frictionloss, stiffness = np.zeros(nv), np.zeros(nv), np.zeros(nv), np.zeros(nv)
        limited, jrange = np.zeros(nb, np.int32), np.zeros((nb, 2))

        def last_dof_of(body: int) -> int:
            while body > 0:
                if self.bodies[body]["jtype"] == JNT_FREE:
                    return int(dofadr[body]) + 5
                if self.bodies[body]["jtype"] == JNT_HINGE:
                    return int(dofadr[body])
                body = int(parent[body])
            return -1

        for b, body in enumerate(self.bodies):
            if body["jtype"] == JNT_FREE:
                for k in range(6):
                    i = dofadr[b] + k
                    dof_body[i] = b
                    dof_parent[i] = i - 1 if k else last_dof_of(int(parent[b]))
                    damping[i], armature[i] = 0.0, 0.0
            elif body["jtype"] == JNT_HINGE:
                i = dofadr[b]
                dof_body[i] = b
                dof_parent[i] = last_dof_of(int(parent[b]))
                damping[i], armature[i] = body["damping"], body["armature"]
                frictionloss[i] = body["frictionloss"]
                stiffness[i] = body["stiffness"]
                if body["range"] is not None:
                    limited[b], jrange[b] = 1, body["range"]
        qpos0 = np.zeros(nq)
        for b, body in enumerate(self.bodies):
            if body["jtype"] == JNT_FREE:
                qpos0[qadr[b]:qadr[b] + 3] = body["pos"]
                qpos0[qadr[b] + 3:qadr[b] + 7] = body["quat"]
            elif body["jtype"] == JNT_HINGE:
                qpos0[qadr[b]] = body["qpos0"]
        stack = lambda key: np.array([b[key] for b in self.bodies], dtype=np.float64)  # noqa: E731
        partial = dict(
            nb=nb, nq=nq, nv=nv, nu=nu, ns=ns, **self.opt,
            body_parent=parent, body_jtype=np.array([b["jtype"] for b in self.bodies], np.int32), body_qadr=qadr,
            body_dofadr=dofadr, body_subtree_end=subtree_end, body_pos=stack("pos"), body_quat=stack("quat"),
            body_mass=stack("mass"), body_ipos=stack("ipos"), body_iquat=stack("iquat"),
            body_inertia=stack("inertia"), jnt_axis=stack("axis"), jnt_pos=stack("jpos"), qpos0=qpos0,
            dof_body=dof_body, dof_parent=dof_parent, dof_damping=damping, dof_armature=armature,
            jnt_limited=limited, jnt_range=jrange, dof_frictionloss=frictionloss, dof_stiffness=stiffness,
            act_dof=np.array([dofadr[a["body"]] for a in self.actuators], np.int32).reshape(nu),
            act_gear=np.array([a["gear"] for a in self.actuators], np.float64).reshape(nu),
            act_ctrlrange=np.array([[a["lo"], a["hi"]] for a in self.actuators], np.float64).reshape(nu, 2),
            sph_body=np.array([s["body"] for s in self.spheres], np.int32).reshape(ns),
            sph_pos=np.array([s["pos"] for s in self.spheres], np.float64).reshape(ns, 3),
            sph_radius=np.array([s["radius"] for s in self.spheres], np.float64).reshape(ns),
            body_names=tuple(b["name"] for b in self.bodies), sph_names=tuple(s["name"] for s in self.spheres),
        )
        inv_b, inv_d, mean_inertia = _compile_constants(partial)
        return KinematicModel(**partial, body_invweight0=inv_b, dof_invweight0=inv_d, meaninertia=mean_inertia,
                              sites=dict(self.sites), sensors=dict(self.sensors), magnetic=self.magnetic)


# --------------------------------------------------------------------------- host kinematics (float64, init-time only)
def host_kinematics(m: dict, qpos: np.ndarray):
    """World poses of every body frame, inertial frame and joint (brute-force chain composition)."""
    nb = m["nb"]
    xpos, xquat = np.zeros((nb, 3)), np.zeros((nb, 4))
    xquat[0, 0] = 1.0
    xanchor, xaxis = np.zeros((nb, 3)), np.zeros((nb, 3))
    for b in range(1, nb):
        p = m["body_parent"][b]
        if m["body_jtype"][b] == JNT_FREE:
            qa = m["body_qadr"][b]
            xpos[b] = qpos[qa:qa + 3]
            q = qpos[qa + 3:qa + 7]
            xquat[b] = q / np.linalg.norm(q)
            xanchor[b] = xpos[b]
        else:
            pos = xpos[p] + quat_to_mat(xquat[p]) @ m["body_pos"][b]
            quat = quat_mul(xquat[p], m["body_quat"][b])
            if m["body_jtype"][b] == JNT_HINGE:
                anchor = pos + quat_to_mat(quat) @ m["jnt_pos"][b]
                xaxis[b] = quat_to_mat(quat) @ m["jnt_axis"][b]
                ang = qpos[m["body_qadr"][b]] - m["qpos0"][m["body_qadr"][b]]
                quat = quat_mul(quat, axis_angle_quat(m["jnt_axis"][b], ang))
                pos = anchor - quat_to_mat(quat) @ m["jnt_pos"][b]
                xanchor[b] = anchor
            xpos[b], xquat[b] = pos, quat / np.linalg.norm(quat)
    xmat = np.stack([quat_to_mat(q) for q in xquat])
    xipos = xpos + np.einsum("bij,bj->bi", xmat, m["body_ipos"])
    ximat = np.stack([quat_to_mat(quat_mul(xquat[b], m["body_iquat"][b])) for b in range(nb)])
    return dict(xpos=xpos, xquat=xquat, xmat=xmat, xipos=xipos, ximat=ximat, xanchor=xanchor, xaxis=xaxis)


def host_jacobian(m: dict, kin: dict, point: np.ndarray, body: int):
    """Translational and rotational Jacobians (3 x nv each) of a world point fixed to ``body``."""
    nv = m["nv"]
    jp, jr = np.zeros((3, nv)), np.zeros((3, nv))
    b = body
    while b > 0:
        da = m["body_dofadr"][b]
        if m["body_jtype"][b] == JNT_FREE:
            jp[:, da:da + 3] = np.eye(3)
            for k in range(3):
                ax = kin["xmat"][b][:, k]
                jr[:, da + 3 + k] = ax
                jp[:, da + 3 + k] = np.cross(ax, point - kin["xpos"][b])
        elif m["body_jtype"][b] == JNT_HINGE:
            ax = kin["xaxis"][b]
            jr[:, da] = ax
            jp[:, da] = np.cross(ax, point - kin["xanchor"][b])
        b = m["body_parent"][b]
    return jp, jr


def host_mass_matrix(m: dict, qpos: np.ndarray, mass_scale: np.ndarray | None = None) -> np.ndarray:
    """M = sum_b m_b Jp^T Jp + Jr^T (R I R^T) Jr + diag(armature), from brute-force Jacobians."""
    kin = host_kinematics(m, qpos)
    nv = m["nv"]
    M = np.diag(np.asarray(m["dof_armature"], dtype=np.float64)).reshape(nv, nv).copy()
    for b in range(1, m["nb"]):
        jp, jr = host_jacobian(m, kin, kin["xipos"][b], b)
        mass = m["body_mass"][b] * (1.0 if mass_scale is None else mass_scale[b])
        Iw = kin["ximat"][b] @ np.diag(m["body_inertia"][b]) @ kin["ximat"][b].T
        M += mass * jp.T @ jp + jr.T @ Iw @ jr
    return M


def _compile_constants(m: dict):
    """body_invweight0 / dof_invweight0 / meaninertia at qpos0, as MuJoCo's compiler derives them."""
    nv, nb = m["nv"], m["nb"]
    if nv == 0:
        return np.zeros((nb, 2)), np.zeros(0), 1.0
    M = host_mass_matrix(m, m["qpos0"])
    Minv = np.linalg.inv(M)
    kin = host_kinematics(m, m["qpos0"])
    inv_b = np.zeros((nb, 2))
    for b in range(1, nb):
        jp, jr = host_jacobian(m, kin, kin["xipos"][b], b)
        inv_b[b, 0] = np.trace(jp @ Minv @ jp.T) / 3.0
        inv_b[b, 1] = np.trace(jr @ Minv @ jr.T) / 3.0
    inv_d = np.diag(Minv).copy()
    for b in range(1, nb):
        if m["body_jtype"][b] == JNT_FREE:
            da = m["body_dofadr"][b]
            inv_d[da:da + 3] = inv_d[da:da + 3].mean()
            inv_d[da + 3:da + 6] = inv_d[da + 3:da + 6].mean()
    return inv_b, inv_d, float(np.trace(M) / nv)


# --------------------------------------------------------------------------- procedural models of the benchmark configs
def pendulum_chain_model(n_links: int = 3, length: float = 0.5, radius: float = 0.05, mass: float = 1.0,
                         damping: float = 0.1, dt: float = 0.005, joint_range=None, frictionloss: float = 0.0,
                         stiffness: float = 0.0, **opts) -> KinematicModel:
    """Planar hinge chain hanging from the world origin along -z, hinge axes along y, no contacts."""
    mb = ModelBuilder(dt=dt, **opts)
    parent = 0
    for i in range(n_links):
        pos = (0.0, 0.0, 0.0) if i == 0 else (0.0, 0.0, -length)
        parent = mb.add_capsule_body(parent, pos, (0.0, 0.0, -1.0), length, radius, mass, joint="hinge",
                                     axis=(0.0, 1.0, 0.0), damping=damping, range=joint_range,
                                     frictionloss=frictionloss, stiffness=stiffness, name=f"link{i}")
        mb.add_actuator(parent)
    return mb.build()


def _limb(mb: ModelBuilder, rng, parent: int, attach, axes: Sequence, direction, seg_len: Sequence[float],
          radius: float, mass_range, damping: float, armature_range, name: str, joint_range=None,
          frictionloss: float = 0.0) -> list[int]:
    ids = []
    pos = np.array(attach, dtype=np.float64)
    for k, (axis, ln) in enumerate(zip(axes, seg_len)):
        ln = float(ln * rng.uniform(0.9, 1.1))
        arm = float(rng.uniform(*armature_range)) if armature_range else 0.0
        b = mb.add_capsule_body(parent, pos, direction, ln, radius, float(rng.uniform(*mass_range)), joint="hinge",
                                axis=axis, damping=damping, armature=arm, range=joint_range, frictionloss=frictionloss,
                                name=f"{name}{k}")
        mb.add_actuator(b)
        ids.append(b)
        parent = b
        pos = np.asarray(direction, dtype=np.float64) / np.linalg.norm(direction) * ln
    return ids


def humanoid_model(seed: int = 1003, dt: float = 0.005, friction: float = 1.0, joint_range=None,
                   frictionloss: float = 0.0, **opts) -> KinematicModel:
    """Free root + 21 hinges in a seeded 5-limb tree (4+4+4+4+5), 4 foot spheres, 21 motors.

    ``joint_range`` limits every hinge to that interval and ``frictionloss`` gives every hinge that much dry friction
    (both off by default)."""
    rng = np.random.default_rng(seed)
    jl = dict(joint_range=joint_range, frictionloss=frictionloss)
    mb = ModelBuilder(dt=dt, friction=friction, **opts)
    mr = (0.5, 5.0)
    root = mb.add_capsule_body(0, (0.0, 0.0, 1.3), (0.0, 0.0, 1.0), 0.3, 0.1, float(rng.uniform(*mr)), joint="free",
                               name="torso")
    X, Y, Z = (1.0, 0, 0), (0, 1.0, 0), (0, 0, 1.0)
    feet = []
    for side, sy in (("l", 0.1), ("r", -0.1)):
        ids = _limb(mb, rng, root, (0.0, sy, -0.05), [X, Y, Y, Y], (0.0, 0.0, -1.0), [0.06, 0.4, 0.4, 0.06], 0.05, mr,
                    0.2, (0.01, 0.01), f"leg_{side}", **jl)
        feet.append(ids[-1])
    for side, sy in (("l", 0.2), ("r", -0.2)):
        _limb(mb, rng, root, (0.0, sy, 0.3), [X, Y, Y, X], (0.0, float(np.sign(sy)) * 0.3, -1.0),
              [0.05, 0.28, 0.25, 0.05], 0.04, mr, 0.2, (0.01, 0.01), f"arm_{side}", **jl)
    _limb(mb, rng, root, (0.0, 0.0, 0.32), [Z, Y, X, Y, Z], (0.0, 0.0, 1.0), [0.05, 0.1, 0.15, 0.05, 0.12], 0.07, mr,
          0.2, (0.01, 0.01), "spine", **jl)
    for f in feet:
        tip = mb.bodies[f]["ipos"] * 2
        mb.add_contact_sphere(f, tip + np.array([0.08, 0.0, 0.0]), 0.04)
        mb.add_contact_sphere(f, tip + np.array([-0.05, 0.0, 0.0]), 0.04)
    return mb.build()


def kbot_scale_model(seed: int = 1004, dt: float = 0.005, joint_range=None, frictionloss: float = 0.0,
                     **opts) -> KinematicModel:
    """K-Bot-scale biped: free root + 20 hinges (legs 5+5, arms 5+5), 8 foot spheres, armature ~U(0.01,0.05).

    ``joint_range`` / ``frictionloss``: limits and dry friction on every hinge, as the real K-Bot's joints have
    (examples/kbot/robot/kbot-headless/robot.mjcf:5-18); off by default."""
    rng = np.random.default_rng(seed)
    jl = dict(joint_range=joint_range, frictionloss=frictionloss)
    mb = ModelBuilder(dt=dt, **opts)
    root = mb.add_capsule_body(0, (0.0, 0.0, 1.05), (0.0, 0.0, 1.0), 0.35, 0.1, 12.0, joint="free", name="torso")
    X, Y, Z = (1.0, 0, 0), (0, 1.0, 0), (0, 0, 1.0)
    arm_r = (0.01, 0.05)
    feet = []
    for side, sy in (("l", 0.09), ("r", -0.09)):
        ids = _limb(mb, rng, root, (0.0, sy, -0.02), [Y, X, Z, Y, Y], (0.0, 0.0, -1.0),
                    [0.05, 0.05, 0.35, 0.35, 0.05], 0.04, (0.8, 3.0), 0.2, arm_r, f"leg_{side}", **jl)
        feet.append(ids[-1])
    for side, sy in (("l", 0.18), ("r", -0.18)):
        _limb(mb, rng, root, (0.0, sy, 0.33), [Y, X, Z, Y, X], (0.0, float(np.sign(sy)) * 0.15, -1.0),
              [0.04, 0.04, 0.22, 0.2, 0.06], 0.03, (0.3, 1.2), 0.2, arm_r, f"arm_{side}", **jl)
    for f in feet:
        tip = mb.bodies[f]["ipos"] * 2
        for dx in (0.1, -0.06):
            for dy in (0.035, -0.035):
                mb.add_contact_sphere(f, tip + np.array([dx, dy, 0.0]), 0.02)
    return mb.build()
