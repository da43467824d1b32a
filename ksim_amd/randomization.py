"""Per-env physics randomisers with the reference's names (ksim/randomization.py:39-243).

Each returns ``{field: (N, ...) tensor}`` sampled once per env at initialisation (ksim/task/rl.py:2231-2243);
the step kernel reads ``friction`` (N), ``mass_scale`` (N, nb), ``armature_scale``, ``damping_scale`` and
``frictionloss`` (N, nv), ``body_ipos`` / ``body_inertia`` (N, nb*3), ``sph_pos`` (N, ns*3) and ``sph_radius`` (N, ns) every
step (rl.py:1182).
"""
from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class PhysicsRandomizer:
    def __call__(self, model, num_envs: int, gen) -> dict:  # pragma: no cover
        raise NotImplementedError


@dataclass(frozen=True)
class FloorFrictionRandomizer(PhysicsRandomizer):  # randomization.py:74-104: absolute value U(lo, hi)
    scale_lower: float = 0.4
    scale_upper: float = 1.0

    def __call__(self, model, num_envs, gen):
        u = torch.rand(num_envs, generator=gen, device=gen.device)
        return {"friction": self.scale_lower + (self.scale_upper - self.scale_lower) * u}


@dataclass(frozen=True)
class AllBodiesMassMultiplicationRandomizer(PhysicsRandomizer):  # randomization.py:207-222: body_mass *= U
    scale_lower: float = 0.95
    scale_upper: float = 1.05

    def __call__(self, model, num_envs, gen):
        u = torch.rand(num_envs, model.nb, generator=gen, device=gen.device)
        return {"mass_scale": self.scale_lower + (self.scale_upper - self.scale_lower) * u}


def _joint_scale(model, num_envs, gen, lo, hi):
    """A factor per dof: U(lo, hi) on the joints, 1 on the six dofs of the floating base (randomization.py:115-122)."""
    s = torch.ones(num_envs, model.nv, device=gen.device)
    first = 6 if model.has_free_root else 0
    s[:, first:] = lo + (hi - lo) * torch.rand(num_envs, model.nv - first, generator=gen, device=gen.device)
    return s


@dataclass(frozen=True)
class ArmatureRandomizer(PhysicsRandomizer):  # randomization.py:108-123: dof_armature[6:] *= U
    scale_lower: float = 0.95
    scale_upper: float = 1.05

    def __call__(self, model, num_envs, gen):
        return {"armature_scale": _joint_scale(model, num_envs, gen, self.scale_lower, self.scale_upper)}


@dataclass(frozen=True)
class JointDampingRandomizer(PhysicsRandomizer):  # randomization.py:226-243: dof_damping[6:] *= U
    scale_lower: float = 0.9
    scale_upper: float = 1.1

    def __call__(self, model, num_envs, gen):
        return {"damping_scale": _joint_scale(model, num_envs, gen, self.scale_lower, self.scale_upper)}


@dataclass(frozen=True)
class MassMultiplicationRandomizer(PhysicsRandomizer):  # randomization.py:166-204: one body's mass *= U
    body_id: int = 1
    scale_lower: float = 0.95
    scale_upper: float = 1.05

    @classmethod
    def from_body_name(cls, model, body_name: str, scale_lower: float = 0.0, scale_upper: float = 1.0):
        if body_name not in model.body_names:
            raise ValueError(f"Body name {body_name} not found in model")
        return cls(body_id=list(model.body_names).index(body_name), scale_lower=scale_lower, scale_upper=scale_upper)

    def __call__(self, model, num_envs, gen):
        s = torch.ones(num_envs, model.nb, device=gen.device)
        s[:, self.body_id] = self.scale_lower + (self.scale_upper - self.scale_lower) * torch.rand(num_envs, generator=gen, device=gen.device)
        return {"mass_scale": s}


@dataclass(frozen=True)
class MassAdditionRandomizer(PhysicsRandomizer):  # randomization.py:126-163: one body's mass += U(lo, hi), as a factor
    body_id: int = 1
    scale_lower: float = 0.0
    scale_upper: float = 1.0

    def __call__(self, model, num_envs, gen):
        s = torch.ones(num_envs, model.nb, device=gen.device)
        add = self.scale_lower + (self.scale_upper - self.scale_lower) * torch.rand(num_envs, generator=gen, device=gen.device)
        s[:, self.body_id] = (float(model.body_mass[self.body_id]) + add) / float(model.body_mass[self.body_id])
        return {"mass_scale": s}


@dataclass(frozen=True)
class StaticFrictionRandomizer(PhysicsRandomizer):  # randomization.py:56-71: dof_frictionloss[6:] *= U
    scale_lower: float = 0.5
    scale_upper: float = 2.0

    def __call__(self, model, num_envs, gen):
        base = torch.tensor(model.dof_frictionloss, dtype=torch.float32, device=gen.device)
        return {"frictionloss": base[None, :] * _joint_scale(model, num_envs, gen, self.scale_lower, self.scale_upper)}


def _ipos(model, device):
    return torch.tensor(model.body_ipos, dtype=torch.float32, device=device)


@dataclass(frozen=True)
class COMRandomizer(PhysicsRandomizer):  # randomization.py:290-333: one body's centre of mass += U(-scale, scale)^3
    body_id: int = 1
    scale: float = 0.01

    @classmethod
    def from_body_name(cls, model, body_name: str, scale: float = 0.01):
        if body_name not in model.body_names:
            raise ValueError(f"Body name {body_name} not found in model")
        return cls(body_id=list(model.body_names).index(body_name), scale=scale)

    def __call__(self, model, num_envs, gen):
        ipos = _ipos(model, gen.device)[None].repeat(num_envs, 1, 1)
        ipos[:, self.body_id] += (2 * torch.rand(num_envs, 3, generator=gen, device=gen.device) - 1) * self.scale
        return {"body_ipos": ipos.reshape(num_envs, -1)}


@dataclass(frozen=True)
class AllBodiesCOMRandomizer(PhysicsRandomizer):  # randomization.py:336-356
    scale: float = 0.01

    def __call__(self, model, num_envs, gen):
        off = (2 * torch.rand(num_envs, model.nb, 3, generator=gen, device=gen.device) - 1) * self.scale
        return {"body_ipos": (_ipos(model, gen.device)[None] + off).reshape(num_envs, -1)}


@dataclass(frozen=True)
class AllBodiesInertiaRandomizer(PhysicsRandomizer):
    """body_mass *= s, body_inertia *= s * shape with s ~ 1 + U(-scale, scale) per body and shape ~ 1 + U(-scale, scale) per
    principal axis (randomization.py:359-383; the inverse weights stay as they are, as there)."""
    scale: float = 0.02

    def __call__(self, model, num_envs, gen):
        s = 1 + (2 * torch.rand(num_envs, model.nb, generator=gen, device=gen.device) - 1) * self.scale
        shape = 1 + (2 * torch.rand(num_envs, model.nb, 3, generator=gen, device=gen.device) - 1) * self.scale
        inertia = torch.tensor(model.body_inertia, dtype=torch.float32, device=gen.device)[None] * s[..., None] * shape
        return {"mass_scale": s, "body_inertia": inertia.reshape(num_envs, -1)}


@dataclass(frozen=True)
class CollisionBodyRandomizer(PhysicsRandomizer):
    """Jitters collision capsules (randomization.py:386-487): radius and half-length scaled by 1 + U(-s, s), the centre moved
    by U(-j, j) per axis.  A capsule is the pair of contact spheres at its ends, `capsules` lists those pairs: the radius
    scale applies to both spheres, the length scale moves them symmetrically about the centre."""
    capsules: tuple = ()
    radius_scale: float = 0.05
    length_scale: float = 0.05
    position_jitter_x: float = 0.001
    position_jitter_y: float = 0.001
    position_jitter_z: float = 0.001

    @classmethod
    def from_geom_names(cls, model, geom_names, **kw):
        pairs = []
        for name in geom_names:
            idx = [i for i, n in enumerate(model.sph_names) if n == name]
            if len(idx) != 2:
                raise ValueError(f"Geom name '{name}' is not a collision capsule of the model. Available geoms: {sorted(set(model.sph_names))}")
            pairs.append(tuple(idx))
        return cls(capsules=tuple(pairs), **kw)

    def __call__(self, model, num_envs, gen):
        dev = gen.device
        pos = torch.tensor(model.sph_pos, dtype=torch.float32, device=dev)[None].repeat(num_envs, 1, 1)
        rad = torch.tensor(model.sph_radius, dtype=torch.float32, device=dev)[None].repeat(num_envs, 1)
        n = len(self.capsules)
        u = lambda *shape: 2 * torch.rand(*shape, generator=gen, device=dev) - 1  # noqa: E731
        rs, ls = 1 + u(num_envs, n) * self.radius_scale, 1 + u(num_envs, n) * self.length_scale
        jit = u(num_envs, n, 3) * torch.tensor([self.position_jitter_x, self.position_jitter_y, self.position_jitter_z], device=dev)
        for k, (i, j) in enumerate(self.capsules):
            centre, half = 0.5 * (pos[:, i] + pos[:, j]), 0.5 * (pos[:, j] - pos[:, i])
            pos[:, i] = centre + jit[:, k] - half * ls[:, k, None]
            pos[:, j] = centre + jit[:, k] + half * ls[:, k, None]
            rad[:, i] *= rs[:, k]
            rad[:, j] *= rs[:, k]
        return {"sph_pos": pos.reshape(num_envs, -1), "sph_radius": rad}


@dataclass(frozen=True)
class IMUAlignmentRandomizer(PhysicsRandomizer):  # randomization.py:245-284
    """Mounting error of the IMU site: small roll and pitch ~ N(0, tilt_std_rad), optionally yaw and a translation.  The
    offset is the normalised product of the small-angle quaternions [1, angle / 2] about z, y, x, applied on the left of
    the site's orientation.  Returns `site_pose` (N, 7): orientation (wxyz) then position of the site in its body, which the
    observations built with `site_pose_per_env=True` read."""
    site_name: str = "imu_site"
    tilt_std_rad: float = 0.03490658503988659
    yaw_std_rad: float | None = None
    translate_std_m: float | None = None

    def __call__(self, model, num_envs, gen, normal=None):
        """`normal` (N, 6): explicit standard normal draws (rx, ry, rz, dx, dy, dz) instead of the generator's."""
        if self.site_name not in model.sites:
            raise ValueError(f"site {self.site_name!r} not found in model. Available: {sorted(model.sites)}")
        dev = gen.device
        z = torch.randn(num_envs, 6, generator=gen, device=dev) if normal is None else normal.to(dev)
        body, pos, quat = model.sites[self.site_name]
        h = 0.5
        rx, ry = z[:, 0] * self.tilt_std_rad, z[:, 1] * self.tilt_std_rad
        rz = z[:, 2] * self.yaw_std_rad if self.yaw_std_rad is not None else torch.zeros(num_envs, device=dev)
        one, zero = torch.ones(num_envs, device=dev), torch.zeros(num_envs, device=dev)

        def mul(a, b):  # Hamilton product, wxyz
            aw, ax, ay, az = a
            bw, bx, by, bz = b
            return (aw * bw - ax * bx - ay * by - az * bz, aw * bx + ax * bw + ay * bz - az * by,
                    aw * by - ax * bz + ay * bw + az * bx, aw * bz + ax * by - ay * bx + az * bw)

        qx, qy, qz = (one, rx * h, zero, zero), (one, zero, ry * h, zero), (one, zero, zero, rz * h)
        off = torch.stack(mul(qz, mul(qy, qx)), dim=-1)
        off = off / off.norm(dim=-1, keepdim=True)
        site = tuple(torch.full((num_envs,), float(v), device=dev) for v in quat)
        new_quat = torch.stack(mul(tuple(off[:, k] for k in range(4)), site), dim=-1)
        new_pos = torch.tensor(pos, dtype=torch.float32, device=dev)[None].repeat(num_envs, 1)
        if self.translate_std_m is not None and self.translate_std_m > 0.0:
            new_pos = new_pos + z[:, 3:6] * self.translate_std_m
        return {"site_pose": torch.cat([new_quat, new_pos], dim=-1).float()}


def get_physics_randomizers(model, randomizers: dict, num_envs: int, gen) -> dict:
    """Merges the randomisers' fields; duplicate fields raise (ksim/task/rl.py:343-346)."""
    out: dict = {}
    for name, r in randomizers.items():
        for k, v in r(model, num_envs, gen).items():
            if k in out:
                raise ValueError(f"Found duplicate randomization keys: {k}")
            out[k] = v.contiguous()
    return out
