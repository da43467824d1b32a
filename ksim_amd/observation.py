"""Observations with the reference's class names (ksim/observation.py:184-352,705-713).

Each class compiles to per-element descriptors that the fused observation kernel evaluates
(`ks_observe`); ``noise`` / ``bias`` follow ksim/observation.py:89-145 (a float noise is additive
Gaussian).  Stateful observations (delay buffers, the lag filter and bias of ProjectedGravityObservation) own a
slice of a per-env carry row (`carry_size`); the kernel advances it in place every control step and initialises
it for the envs that start an episode.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from . import _lib_terms as T
from .model import KinematicModel
from .noise import Bias, Noise, convert_to_bias, convert_to_noise


@dataclass(frozen=True)
class ObsElem:
    kind: int
    src: int
    index: int = 0
    comp: int = 0
    const: tuple = (0.0, 0.0, 0.0)
    carry: int = 0      # offset inside the observation's own carry block
    stride: int = 0
    q: tuple = (0.0, 0.0, 0.0)
    e: tuple = (1.0, 0.0, 0.0, 0.0)  # site kinds: the site's orientation in its body
    env_site: int = 0   # site kinds: 1 = the site's pose comes per env (IMUAlignmentRandomizer)


@dataclass(frozen=True)
class Observation:
    noise: Noise | float | None = None
    bias: Bias | float | None = None  # per-episode bias; a float is the std of an additive Gaussian one (observation.py:79-86)

    def elements(self, model: KinematicModel, command_dim: int) -> list[ObsElem]:  # pragma: no cover
        raise NotImplementedError

    def carry_size(self, model: KinematicModel) -> int:
        """Floats of per-env carry (StatefulObservation.initial_carry, observation.py:148-181); 0 when stateless."""
        return 0

    def get_name(self) -> str:
        name = type(self).__name__
        out = "".join("_" + c.lower() if c.isupper() else c for c in name).lstrip("_")
        return out

    @property
    def observation_name(self) -> str:
        return self.get_name()

    def _noise(self) -> Noise | None:
        return convert_to_noise(self.noise)

    def _bias(self) -> Bias | None:
        return convert_to_bias(self.bias)


def _copy(src, start, n):
    return [ObsElem(T.OBS_COPY, src, start + i) for i in range(n)]


def _rot(src, start, const=(0.0, 0.0, 0.0)):
    return [ObsElem(T.OBS_ROT_INV, src, start, c, const) for c in range(3)]


@dataclass(frozen=True)
class BasePositionObservation(Observation):  # observation.py:185-188
    def elements(self, m, command_dim):
        return _copy(T.SRC_QPOS, 0, 3)


@dataclass(frozen=True)
class BaseOrientationObservation(Observation):  # observation.py:192-195
    def elements(self, m, command_dim):
        return _copy(T.SRC_QPOS, 3, 4)


@dataclass(frozen=True)
class BaseLinearVelocityObservation(Observation):  # observation.py:199-206
    in_robot_frame: bool = False

    def elements(self, m, command_dim):
        return _rot(T.SRC_QVEL, 0) if self.in_robot_frame else _copy(T.SRC_QVEL, 0, 3)


@dataclass(frozen=True)
class BaseAngularVelocityObservation(Observation):  # observation.py:210-217
    in_robot_frame: bool = False

    def elements(self, m, command_dim):
        return _rot(T.SRC_QVEL, 3) if self.in_robot_frame else _copy(T.SRC_QVEL, 3, 3)


@dataclass(frozen=True)
class JointPositionObservation(Observation):  # observation.py:221-225 (qpos[7:] - zero_offset)
    def elements(self, m, command_dim):
        return [ObsElem(T.OBS_JOINT_POS, T.SRC_QPOS, 7 + i) for i in range(m.nq - 7)]


@dataclass(frozen=True)
class JointVelocityObservation(Observation):  # observation.py:255-257
    def elements(self, m, command_dim):
        return _copy(T.SRC_QVEL, 6, m.nv - 6)


@dataclass(frozen=True)
class ActuatorForceObservation(Observation):  # observation.py:300-303 (unit-gear motors: force = ctrl)
    def elements(self, m, command_dim):
        return _copy(T.SRC_CTRL, 0, m.nu)


@dataclass(frozen=True)
class BaseLinearAccelerationObservation(Observation):  # observation.py:343-346
    def elements(self, m, command_dim):
        return _copy(T.SRC_QACC, 0, 3)


@dataclass(frozen=True)
class BaseAngularAccelerationObservation(Observation):  # observation.py:349-352
    def elements(self, m, command_dim):
        return _copy(T.SRC_QACC, 3, 3)


@dataclass(frozen=True)
class ActuatorAccelerationObservation(Observation):  # observation.py:445-448
    def elements(self, m, command_dim):
        return _copy(T.SRC_QACC, 6, m.nv - 6)


@dataclass(frozen=True)
class CenterOfMassVelocityObservation(Observation):  # observation.py:293-297 (cvel[1:].ravel())
    def elements(self, m, command_dim):
        return _copy(T.SRC_CVEL, 6, (m.nb - 1) * 6)


@dataclass(frozen=True)
class CenterOfMassInertiaObservation(Observation):  # observation.py:285-290 (cinert[1:].ravel())
    def elements(self, m, command_dim):
        return _copy(T.SRC_CINERT, 10, (m.nb - 1) * 10)


@dataclass(frozen=True)
class BodyVelocityObservation(Observation):  # observation.py:544-560 (cvel of chosen bodies: angular, then linear)
    body_idxs: tuple = ()

    def elements(self, m, command_dim):
        return [e for b in self.body_idxs for e in _copy(T.SRC_CVEL, 6 * b, 6)]


@dataclass(frozen=True)
class FeetForceObservation(Observation):
    """cfrc_ext[foot][:3] of the left and right foot, stacked (2, 3) (observation.py:563-588).  MuJoCo orders cfrc_ext
    torque first, so these three numbers are the contact torque about the tree's centre of mass; the reference's class
    name notwithstanding, the slice is kept as it is there."""
    foot_left: int = 0
    foot_right: int = 0

    def elements(self, m, command_dim):
        return _copy(T.SRC_CFRC_EXT, 6 * self.foot_left, 3) + _copy(T.SRC_CFRC_EXT, 6 * self.foot_right, 3)


@dataclass(frozen=True)
class FeetTorqueObservation(Observation):
    """cfrc_ext[foot][3:] of both feet, (2, 3) (observation.py:591-616): the linear contact force, see FeetForceObservation."""
    foot_left: int = 0
    foot_right: int = 0

    def elements(self, m, command_dim):
        return _copy(T.SRC_CFRC_EXT, 6 * self.foot_left + 3, 3) + _copy(T.SRC_CFRC_EXT, 6 * self.foot_right + 3, 3)


@dataclass(frozen=True)
class ActPosObservation(Observation):  # observation.py:717-750: (last action, joint position) of one joint, for debugging
    ctrl_idx: int = 0
    qpos_idx: int = 7

    def elements(self, m, command_dim):
        return _copy(T.SRC_LAST_ACTION, self.ctrl_idx, 1) + _copy(T.SRC_QPOS, self.qpos_idx, 1)


@dataclass(frozen=True)
class BodyPositionObservation(Observation):  # observation.py:524-559 (xpos of chosen bodies)
    body_ids: tuple = ()

    def elements(self, m, command_dim):
        return [e for b in self.body_ids for e in _copy(T.SRC_XPOS, 3 * b, 3)]


@dataclass(frozen=True)
class BodyOrientationObservation(Observation):  # observation.py:618-641
    body_ids: tuple = ()

    def elements(self, m, command_dim):
        return [e for b in self.body_ids for e in _copy(T.SRC_XQUAT, 4 * b, 4)]


@dataclass(frozen=True)
class FeetOrientationObservation(BodyOrientationObservation):  # observation.py:672-703: exactly the two feet
    def __post_init__(self):
        if len(self.body_ids) != 2:
            raise ValueError("FeetOrientationObservation expects exactly two bodies (left and right foot).")


@dataclass(frozen=True)
class TimestepObservation(Observation):  # observation.py:705-713
    def elements(self, m, command_dim):
        return _copy(T.SRC_TIME, 0, 1)


@dataclass(frozen=True)
class ProjectedGravityObservation(Observation):
    """Gravity in the base frame, rot(q_base)^-1 g (observation.py:355-442; the base quaternion stands for the
    framequat sensor).  With a lag range or an IMU bias the reading is the exponential average
    x <- x lag + g_body (1 - lag) of the biased vector, lag and bias drawn per episode; without them it is stateless."""
    gravity: tuple = (0.0, 0.0, -9.81)
    min_lag: float = 0.0
    max_lag: float = 0.0
    imu_bias: float = 0.0

    def __post_init__(self):
        for name in ("min_lag", "max_lag"):  # observation.py:372-373
            if not 0.0 <= getattr(self, name) < 1.0:
                raise ValueError(f"{name} must be in [0, 1)")
        if self.imu_bias < 0.0:
            raise ValueError("imu_bias must be non-negative")

    @property
    def stateful(self) -> bool:
        return self.min_lag > 0.0 or self.max_lag > 0.0 or self.imu_bias > 0.0

    def carry_size(self, m):
        return 7 if self.stateful else 0  # x(3), lag, bias(3): ProjectedGravityCarry

    def elements(self, m, command_dim):
        g = tuple(float(x) for x in self.gravity)
        if not self.stateful:
            return _rot(T.SRC_CONST, 0, g)
        return [ObsElem(T.OBS_GRAVITY_EMA, T.SRC_CONST, 0, c, g, 0, 0, (self.min_lag, self.max_lag, self.imu_bias))
                for c in range(3)]


@dataclass(frozen=True)
class _Delayed(Observation):
    delay_steps: int = 1

    def __post_init__(self):
        if self.delay_steps < 1:  # observation.py:230
            raise ValueError("delay_steps must be >= 1")

    def _source(self, m):  # pragma: no cover
        raise NotImplementedError

    def carry_size(self, m):
        return self.delay_steps * self._source(m)[2]

    def elements(self, m, command_dim):
        src, start, n = self._source(m)
        return [ObsElem(T.OBS_DELAYED, src, start + i, self.delay_steps, carry=i, stride=n) for i in range(n)]


@dataclass(frozen=True)
class DelayedJointPositionObservation(_Delayed):  # observation.py:228-252 (minus zero_offset, like the live one)
    def _source(self, m):
        return T.SRC_QPOS, 7, m.nq - 7


@dataclass(frozen=True)
class DelayedJointVelocityObservation(_Delayed):  # observation.py:260-283
    def _source(self, m):
        return T.SRC_QVEL, 6, m.nv - 6


@dataclass(frozen=True)
class FeetContactObservation(Observation):
    """1.0 where a foot's contact sphere touches the floor (observation.py:481-521 over geoms_colliding,
    utils/mujoco.py:175-217).  `foot_left` / `foot_right` list contact-sphere indices of the model, equally many;
    the output is the (n_spheres_per_foot, 2) block the reference emits, row-major."""
    foot_left: tuple = ()
    foot_right: tuple = ()

    def __post_init__(self):
        if len(self.foot_left) != len(self.foot_right) or not self.foot_left:
            raise ValueError("foot_left and foot_right need the same, non-zero number of contact spheres")

    @classmethod
    def create(cls, *, physics_model, foot_left_body_names, foot_right_body_names, noise=None):
        """Feet given by body name: every contact sphere attached to the named bodies."""
        def spheres(names):
            names = [names] if isinstance(names, str) else list(names)
            ids = []
            for n in names:
                if n not in physics_model.body_names:
                    raise ValueError(f"Body name {n} not found in model")
                b = list(physics_model.body_names).index(n)
                ids += [i for i, sb in enumerate(physics_model.sph_body) if int(sb) == b]
            return tuple(ids)
        return cls(foot_left=spheres(foot_left_body_names), foot_right=spheres(foot_right_body_names), noise=noise)

    def elements(self, m, command_dim):
        out = []
        for l_, r_ in zip(self.foot_left, self.foot_right):
            out += [ObsElem(T.OBS_CONTACT, T.SRC_CONTACT_DIST, int(l_)), ObsElem(T.OBS_CONTACT, T.SRC_CONTACT_DIST, int(r_))]
        return out


FLOOR_GEOM = -1  # the floor plane in a list of geoms; contact spheres go by their index


@dataclass(frozen=True)
class ContactObservation(Observation):  # observation.py:452-478
    """For each listed geom, whether it touches another listed geom (geoms_colliding of the list with itself, any over the
    partners).  The collision model here is contact spheres against the floor plane, so a sphere's entry is its own floor
    contact when `FLOOR_GEOM` is in the list (otherwise 0: spheres do not collide with each other) and the floor's entry
    is whether any listed sphere touches it."""
    geom_idxs: tuple = ()
    contact_group: str | None = None

    @classmethod
    def create(cls, *, physics_model, geom_names, contact_group=None, noise=None):
        """Geoms by name: "floor", or a body's name for all of its contact spheres."""
        names = [geom_names] if isinstance(geom_names, str) else list(geom_names)
        idx = []
        for n in names:
            if n == "floor":
                idx.append(FLOOR_GEOM)
                continue
            if n not in physics_model.body_names:
                raise ValueError(f"Geom name {n} not found in model")
            b = list(physics_model.body_names).index(n)
            idx += [i for i, sb in enumerate(physics_model.sph_body) if int(sb) == b]
        return cls(geom_idxs=tuple(idx), contact_group=contact_group, noise=noise)

    def elements(self, m, command_dim):
        spheres = [int(g) for g in self.geom_idxs if g != FLOOR_GEOM]
        if any(g < 0 or g >= m.ns for g in spheres):
            raise ValueError(f"contact spheres are numbered 0..{m.ns - 1}")
        if spheres and m.ns > 31:
            raise ValueError(f"a contact list covers at most 31 spheres (one bit each of an int32 mask); the model has {m.ns}")
        has_floor = FLOOR_GEOM in self.geom_idxs
        mask = sum(1 << g for g in set(spheres))
        out = []
        for g in self.geom_idxs:
            if g == FLOOR_GEOM:
                out.append(ObsElem(T.OBS_CONTACT_ANY, T.SRC_CONTACT_DIST, mask) if mask else ObsElem(T.OBS_COPY, T.SRC_CONST, 0))
            elif has_floor:
                out.append(ObsElem(T.OBS_CONTACT, T.SRC_CONTACT_DIST, int(g)))
            else:
                out.append(ObsElem(T.OBS_COPY, T.SRC_CONST, 0))
        return out


@dataclass(frozen=True)
class SiteOrientationObservation(Observation):  # observation.py:645-669
    """6-D rotation of each named site in the world frame: the first two rows of its rotation matrix, row-major.  (The
    reference calls xax.rotation_matrix_to_rotation6d, whose entry order is not stated in the reference's own files.)"""
    site_names: tuple = ()
    name: str = "site_orientation"
    site_pose_per_env: bool = False  # the site's pose is randomised per env (IMUAlignmentRandomizer): read it from `site_pose`

    @classmethod
    def create(cls, *, physics_model, site_names, noise=None):
        for n in site_names:
            if n not in physics_model.sites:
                raise ValueError(f"site {n!r} not found in model. Available: {sorted(physics_model.sites)}")
        return cls(site_names=tuple(site_names), name="site_orientation_observation_" + "_".join(site_names), noise=noise)

    def elements(self, m, command_dim):
        out = []
        for n in self.site_names:
            body, pos, quat = m.sites[n]
            env = int(self.site_pose_per_env)
            out += [ObsElem(T.OBS_SITE_ROT6D, T.SRC_XQUAT, body, c, e=tuple(quat), env_site=env) for c in range(6)]
        return out

    def get_name(self) -> str:
        return self.name


@dataclass(frozen=True)
class LastActionObservation(Observation):
    """The previous control step's action (PhysicsState.last_ctrl, ksim/types.py:33-43)."""

    action_dim: int | None = None  # 2 nu for position-velocity actuators; None = nu

    def elements(self, m, command_dim):
        return _copy(T.SRC_LAST_ACTION, 0, m.nu if self.action_dim is None else int(self.action_dim))


@dataclass(frozen=True)
class CommandObservation(Observation):
    """The env's command vector (ksim/observation.py:61-66 ObservationInput.commands), passed through."""

    def elements(self, m, command_dim):
        return _copy(T.SRC_COMMAND, 0, command_dim)


@dataclass(frozen=True)
class SensorObservation(Observation):
    """A sensor of the model by name (observation.py:307-340 reads its slice of `sensordata`).  Built sensor types:
    `gyro` (angular velocity in the site frame), `accelerometer` (acceleration minus gravity in the site frame; the site
    must sit on the floating base, where an IMU does), `touch` (the normal contact force on the site's body: every
    contact sphere of that body is taken to lie inside the site's volume, which holds for the feet of the shipped robots),
    `framepos`, `framequat`, `frameangvel` of a site in world axes and `magnetometer` (the model's magnetic field in the site
    frame).  Like `sensordata`, they describe the state the last substep started from."""
    sensor_name: str = ""
    site_pose_per_env: bool = False  # the sensor's site is randomised per env (IMUAlignmentRandomizer, randomization.py:245-284)
    BUILT = ("gyro", "accelerometer", "touch", "framepos", "framequat", "frameangvel", "magnetometer")

    @classmethod
    def create(cls, *, physics_model: KinematicModel, sensor_name: str, noise=None):
        if sensor_name not in physics_model.sensors:
            options = "\n".join(sorted(physics_model.sensors))
            raise ValueError(f"{sensor_name} not found in model. Available:\n{options}")
        kind = physics_model.sensors[sensor_name][0]
        if kind not in cls.BUILT:
            raise ValueError(f"sensor {sensor_name!r} of type {kind} is not built ({', '.join(cls.BUILT)} are)")
        return cls(sensor_name=sensor_name, noise=noise)

    def elements(self, m, command_dim):
        kind, site = m.sensors[self.sensor_name]
        body, pos, quat = m.sites[site]
        if kind == "touch":
            return [ObsElem(T.OBS_COPY, T.SRC_CFRC_EXT, 6 * body + 5)]
        env = int(self.site_pose_per_env)
        if kind == "gyro":
            return [ObsElem(T.OBS_SITE_GYRO, T.SRC_CVEL, body, c, e=tuple(quat), env_site=env) for c in range(3)]
        if kind == "frameangvel":  # the body's angular velocity in world axes, wherever on the body the site sits
            return [ObsElem(T.OBS_COPY, T.SRC_CVEL, 6 * body + c) for c in range(3)]
        if kind == "framepos":
            return [ObsElem(T.OBS_SITE_POS, T.SRC_XPOS, body, c, const=tuple(pos), e=tuple(quat), env_site=env) for c in range(3)]
        if kind == "framequat":
            return [ObsElem(T.OBS_SITE_QUAT, T.SRC_XQUAT, body, c, e=tuple(quat), env_site=env) for c in range(4)]
        if kind == "magnetometer":
            return [ObsElem(T.OBS_SITE_MAGNETOMETER, T.SRC_XQUAT, body, c, q=tuple(m.magnetic), e=tuple(quat), env_site=env) for c in range(3)]
        if body != 1 or not m.has_free_root:
            raise ValueError(f"accelerometer {self.sensor_name!r}: its site must sit on the floating base")
        return [ObsElem(T.OBS_SITE_ACCEL, T.SRC_CVEL, body, c, const=tuple(pos), q=tuple(m.gravity), e=tuple(quat), env_site=env)
                for c in range(3)]

    def get_name(self) -> str:
        return self.sensor_name
