"""MJCF -> KinematicModel for the model subset the step kernel runs.

The reference compiles its robot files with MuJoCo (`mujoco.MjModel.from_xml_path`, ksim/task/rl.py:717-748,
ksim/utils/mujoco.py:388-391) and hands the result to MJX.  This loader reads the same files for robots of the K-Bot's
kind (examples/kbot/robot/kbot-headless/robot.mjcf) and for the humanoid of the walking example
(examples/data/scene.mjcf): a floating base, hinge joints, `<inertial>` elements or inertia from sphere / capsule geoms,
`<motor>` actuators, and sphere or capsule collision geoms against the ground plane.  What MuJoCo's compiler does
for such a file is restated here:

* `<default>` classes nest and inherit; `childclass` on a body applies to everything below it;
* a body without a joint is welded to its parent: its inertia, geoms and children move into the parent's frame, and the
  parent's inertial becomes the composite (mass, centre of mass, inertia tensor by the parallel-axis theorem, principal
  axes by an eigendecomposition);
* a body without `<inertial>` takes its inertia from its sphere / capsule geoms at the default density of 1000;
* a capsule touches the plane with its two end spheres, so each collision capsule becomes two contact spheres;
* a joint with a `range` is limited (autolimits); `armature`, `damping`, `frictionloss`, `stiffness` (a spring about the
  joint's reference angle) come from the joint or its class;
* several hinges on one body act in the order they are listed: the body becomes a chain of massless bodies, one per
  joint but the last, at the same place, and the last joint carries the body itself;
* collisions come from `contype` / `conaffinity` or from explicit `<contact><pair>` elements against the floor plane.

Anything else (ball or slide joints, meshes or boxes as collision geoms or as the only source of inertia, tendons,
equality constraints, position actuators, contact dimensions other than 3) raises ValueError: the file needs MuJoCo's
full compiler.
"""
from __future__ import annotations

import xml.etree.ElementTree as ET

import numpy as np

from .model import KinematicModel, ModelBuilder

_DENSITY = 1000.0


def _vec(text, n=None, default=None):
    if text is None:
        return None if default is None else np.array(default, dtype=np.float64)
    v = np.array([float(t) for t in text.split()], dtype=np.float64)
    if n is not None and v.size != n:
        raise ValueError(f"expected {n} numbers, got {text!r}")
    return v


def quat_mul(a, b):
    aw, ax, ay, az = a
    bw, bx, by, bz = b
    return np.array([aw * bw - ax * bx - ay * by - az * bz, aw * bx + ax * bw + ay * bz - az * by,
                     aw * by - ax * bz + ay * bw + az * bx, aw * bz + ax * by - ay * bx + az * bw])


def quat_to_mat(q):
    w, x, y, z = q / np.linalg.norm(q)
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


def mat_to_quat(R):
    """Unit quaternion (w, x, y, z) of a proper rotation matrix."""
    t = np.trace(R)
    if t > 0:
        s = np.sqrt(t + 1.0) * 2
        q = np.array([0.25 * s, (R[2, 1] - R[1, 2]) / s, (R[0, 2] - R[2, 0]) / s, (R[1, 0] - R[0, 1]) / s])
    else:
        i = int(np.argmax(np.diag(R)))
        j, k = (i + 1) % 3, (i + 2) % 3
        s = np.sqrt(1.0 + R[i, i] - R[j, j] - R[k, k]) * 2
        q = np.zeros(4)
        q[0] = (R[k, j] - R[j, k]) / s
        q[1 + i] = 0.25 * s
        q[1 + j] = (R[j, i] + R[i, j]) / s
        q[1 + k] = (R[k, i] + R[i, k]) / s
    return q / np.linalg.norm(q)


class _Defaults:
    """The nested `<default>` classes: attributes of an element type resolved through the class chain."""

    def __init__(self, root):
        self.classes: dict[str, dict] = {}
        top = root.find("default")
        self._walk(top, "main", {}) if top is not None else self.classes.setdefault("main", {})

    def _walk(self, node, name, inherited):
        own = {k: dict(v) for k, v in inherited.items()}
        for child in node:
            if child.tag != "default":
                own.setdefault(child.tag, {}).update(child.attrib)
        self.classes[name] = own
        for child in node:
            if child.tag == "default":
                self._walk(child, child.get("class"), own)

    def resolve(self, elem, childclass):
        cls = elem.get("class") or childclass or "main"
        if cls not in self.classes:
            raise ValueError(f"unknown default class {cls!r}")
        out = dict(self.classes[cls].get(elem.tag, {}))
        out.update(elem.attrib)
        return out


def _geom_inertia(kind, size, fromto, pos, quat):
    """(mass, com, inertia tensor about the com) of a sphere or capsule geom in the body frame, density 1000."""
    if kind == "sphere":
        r = size[0]
        m = _DENSITY * 4.0 / 3.0 * np.pi * r**3
        return m, pos, np.eye(3) * (0.4 * m * r * r)
    if kind == "capsule":
        r = size[0]
        if fromto is not None:
            a, b = fromto[:3], fromto[3:]
            length, centre = np.linalg.norm(b - a), 0.5 * (a + b)
            z = (b - a) / length
        else:
            length, centre = 2 * size[1], pos
            z = quat_to_mat(quat)[:, 2]
        mc = _DENSITY * np.pi * r * r * length            # cylinder
        ms = _DENSITY * 4.0 / 3.0 * np.pi * r**3           # the two half spheres together
        h = length
        ixx = mc * (r * r / 4 + h * h / 12) + ms * (0.4 * r * r + h * h / 4 + 3.0 / 8.0 * h * r)
        izz = mc * r * r / 2 + ms * 0.4 * r * r
        x = np.cross(z, [1.0, 0, 0] if abs(z[0]) < 0.9 else [0, 1.0, 0])
        x /= np.linalg.norm(x)
        R = np.stack([x, np.cross(z, x), z], axis=1)
        return mc + ms, centre, R @ np.diag([ixx, ixx, izz]) @ R.T
    raise ValueError(f"a {kind} geom cannot give a body its inertia here (sphere and capsule only)")


class _Body:
    def __init__(self, name):
        self.name = name
        self.pos, self.quat = np.zeros(3), np.array([1.0, 0, 0, 0])
        self.joints = []                  # dicts, in the order they act
        self.parts = []                   # (mass, com, tensor about com) in this body's frame
        self.spheres = []                 # (pos, radius, geom name) in this body's frame
        self.sites = []                   # (name, pos, quat) in this body's frame
        self.children = []
        self.contact = None               # (friction, solref, solimp) of its collision geoms


def load_mjcf(path: str, **options) -> KinematicModel:
    """Reads an MJCF file into a KinematicModel.  `options` are ModelBuilder's (dt, iterations, integrator, ...): ksim sets
    them in code (ksim/task/rl.py:717-748), not in the file; an `<option timestep>` in the file is the default for dt."""
    root = ET.parse(path).getroot()
    if root.tag != "mujoco":
        raise ValueError("not an MJCF file")
    for tag in ("tendon", "equality"):
        if root.find(tag) is not None and len(root.find(tag)):
            raise ValueError(f"<{tag}> is outside the model subset")
    comp = root.find("compiler")
    degrees = comp is None or comp.get("angle", "degree") == "degree"
    defaults = _Defaults(root)
    opt = root.find("option")
    if opt is not None and "timestep" in opt.attrib:
        options.setdefault("dt", float(opt.get("timestep")))
    if opt is not None and opt.get("magnetic") is not None:
        options.setdefault("magnetic", tuple(_vec(opt.get("magnetic"), 3)))

    def angle(v):
        return np.radians(v) if degrees else v

    def geom_frame(attrib, kind):
        """A geom's frame; the orientation of a sphere, or of a capsule given by its end points, does not matter."""
        if kind == "sphere" or attrib.get("fromto") is not None:
            return _vec(attrib.get("pos"), 3, (0, 0, 0)), np.array([1.0, 0, 0, 0])
        return frame(attrib)

    def frame(attrib):
        for bad in ("euler", "axisangle", "xyaxes", "zaxis"):
            if bad in attrib:
                raise ValueError(f"orientation by {bad} is outside the model subset (use quat)")
        return _vec(attrib.get("pos"), 3, (0, 0, 0)), _vec(attrib.get("quat"), 4, (1, 0, 0, 0))

    contact_params = []
    limit_params = []
    world = root.find("worldbody")
    planes = {g.get("name") for g in world if g.tag == "geom" and defaults.resolve(g, None).get("type", "sphere") == "plane"}
    # condim of a geom-floor contact: an explicit pair's own, otherwise the larger of the two geoms' (MuJoCo's rule); every
    # contact of the model must agree, on 1 (frictionless, what examples/data/scene.mjcf uses) or 3 (friction pyramid)
    plane_condim = {g.get("name"): int(defaults.resolve(g, None).get("condim", 3)) for g in world
                    if g.tag == "geom" and defaults.resolve(g, None).get("type", "sphere") == "plane"}
    floor_condim = max(plane_condim.values()) if plane_condim else 3
    condims: list[int] = []
    pairs: dict[str, dict] = {}  # geom name -> attributes of its explicit contact pair with the floor
    con = root.find("contact")
    for pr in ([] if con is None else con):
        if pr.tag != "pair":
            continue  # <exclude> only matters between bodies, which never collide here
        at = defaults.resolve(pr, None)
        g1, g2 = at.get("geom1"), at.get("geom2")
        if (g1 in planes) == (g2 in planes):
            raise ValueError(f"contact pair {g1!r} / {g2!r}: only pairs of a robot geom with the floor plane are in the model subset")
        if int(at.get("condim", 3)) not in (1, 3):
            raise ValueError(f"contact pair {g1!r} / {g2!r}: condim {at.get('condim')} is outside the model subset (1 or 3)")
        pairs[g2 if g1 in planes else g1] = at

    def read_body(elem, childclass):
        b = _Body(elem.get("name", ""))
        b.pos, b.quat = frame(elem.attrib)
        b.quat = b.quat / np.linalg.norm(b.quat)
        childclass = elem.get("childclass", childclass)
        for j in (e for e in elem if e.tag in ("joint", "freejoint")):
            if j.tag == "freejoint":
                b.joints.append(dict(type="free", name=j.get("name", "")))
                continue
            a = defaults.resolve(j, childclass)
            jt = a.get("type", "hinge")
            if jt == "free":
                b.joints.append(dict(type="free", name=a.get("name", "")))
                continue
            if jt != "hinge":
                raise ValueError(f"joint {a.get('name')!r}: type {jt} is outside the model subset")
            if float(a.get("ref", 0.0)) != 0.0 or float(a.get("springref", 0.0)) != 0.0:
                raise ValueError(f"joint {a.get('name')!r}: ref and springref are outside the model subset")
            rng = _vec(a.get("range"), 2)
            limited = a.get("limited", "auto")
            if limited == "false" or (limited == "auto" and rng is None):
                rng = None
            elif rng is None:
                raise ValueError(f"joint {a.get('name')!r}: limited without a range")
            if rng is not None:
                sl = _vec(a.get("solimplimit"), None, (0.9, 0.95, 0.001, 0.5, 2.0))
                sl = np.concatenate([sl, np.array([0.9, 0.95, 0.001, 0.5, 2.0])[sl.size:]])
                limit_params.append((tuple(_vec(a.get("solreflimit"), 2, (0.02, 1.0))), tuple(sl)))
            b.joints.append(dict(type="hinge", name=a.get("name", ""), axis=_vec(a.get("axis"), 3, (0, 0, 1)),
                                 pos=_vec(a.get("pos"), 3, (0, 0, 0)), range=None if rng is None else tuple(angle(rng)),
                                 armature=float(a.get("armature", 0.0)), damping=float(a.get("damping", 0.0)),
                                 frictionloss=float(a.get("frictionloss", 0.0)), stiffness=float(a.get("stiffness", 0.0))))
        if len(b.joints) > 1 and any(j["type"] == "free" for j in b.joints):
            raise ValueError(f"body {b.name!r}: a free joint next to other joints is outside the model subset")
        inertial = elem.find("inertial")
        geoms = [defaults.resolve(g, childclass) for g in elem if g.tag == "geom"]
        if inertial is not None:
            if "fullinertia" in inertial.attrib:
                f = _vec(inertial.get("fullinertia"), 6)
                tensor = np.array([[f[0], f[3], f[4]], [f[3], f[1], f[5]], [f[4], f[5], f[2]]])
            else:
                R = quat_to_mat(_vec(inertial.get("quat"), 4, (1, 0, 0, 0)))
                tensor = R @ np.diag(_vec(inertial.get("diaginertia"), 3)) @ R.T
            b.parts.append((float(inertial.get("mass")), _vec(inertial.get("pos"), 3, (0, 0, 0)), tensor))
        else:
            for g in geoms:
                kind = g.get("type", "sphere")
                if kind == "mesh" or kind == "plane":
                    if kind == "mesh":
                        raise ValueError(f"body {b.name!r}: inertia from a mesh is outside the model subset (give <inertial>)")
                    continue
                gp, gq = geom_frame(g, kind)
                b.parts.append(_geom_inertia(kind, _vec(g.get("size")), _vec(g.get("fromto"), 6), gp, gq))
        for g in geoms:
            pair = pairs.get(g.get("name"))
            if pair is None and int(g.get("contype", 1)) == 0 and int(g.get("conaffinity", 1)) == 0:
                continue  # visual only
            kind = g.get("type", "sphere")
            if kind == "plane":
                continue
            cd = int(pair.get("condim", 3)) if pair is not None else max(int(g.get("condim", 3)), floor_condim)
            if cd not in (1, 3):
                raise ValueError(f"geom {g.get('name')!r}: condim {cd} is outside the model subset (1 or 3)")
            condims.append(cd)
            size, gp = _vec(g.get("size")), geom_frame(g, kind)[0]
            if kind == "sphere":
                b.spheres.append((gp, float(size[0]), g.get("name", "")))
            elif kind == "capsule":
                if g.get("fromto") is not None:
                    ft = _vec(g.get("fromto"), 6)
                    ends = (ft[:3], ft[3:])
                else:
                    z = quat_to_mat(frame(g)[1])[:, 2] * size[1]
                    ends = (gp - z, gp + z)
                b.spheres.extend((e, float(size[0]), g.get("name", "")) for e in ends)
            else:
                raise ValueError(f"body {b.name!r}: a colliding {kind} is outside the model subset (sphere and capsule only)")
            src = pair if pair is not None else g  # an explicit pair carries its own parameters (MuJoCo's defaults otherwise)
            si = _vec(src.get("solimp"), None, (0.9, 0.95, 0.001, 0.5, 2.0))
            si = np.concatenate([si, np.array([0.9, 0.95, 0.001, 0.5, 2.0])[si.size:]])
            contact_params.append((float(_vec(src.get("friction"), None, (1.0, 0.005, 0.0001))[0]),
                                   tuple(_vec(src.get("solref"), 2, (0.02, 1.0))), tuple(si)))
        for st in (e for e in elem if e.tag == "site"):
            sa = defaults.resolve(st, childclass)
            sp, sq = frame(sa)
            b.sites.append((sa.get("name", ""), sp, sq / np.linalg.norm(sq)))
        b.children = [read_body(c, childclass) for c in elem if c.tag == "body"]
        return b

    tops = [read_body(e, None) for e in world if e.tag == "body"]
    if len(tops) != 1:
        raise ValueError("exactly one robot body under <worldbody> is expected")

    def weld(b):
        """Moves every jointless child (recursively) into b's frame."""
        kept = []
        for c in b.children:
            weld(c)
            if c.joints:
                kept.append(c)
                continue
            R = quat_to_mat(c.quat)
            b.parts.extend((m, c.pos + R @ com, R @ I @ R.T) for m, com, I in c.parts)
            b.spheres.extend((c.pos + R @ p, r, n) for p, r, n in c.spheres)
            b.sites.extend((n, c.pos + R @ p, quat_mul(c.quat, q)) for n, p, q in c.sites)
            for g in c.children:  # grandchildren keep their joints; their frame is re-expressed in b
                g.pos, g.quat = c.pos + R @ g.pos, quat_mul(c.quat, g.quat)
                kept.append(g)
        b.children = kept

    top = tops[0]
    if not top.joints:
        raise ValueError("the robot's top body needs a joint (a fixed base is outside the model subset)")
    weld(top)

    def composite(parts):
        if not parts:
            raise ValueError("a moving body without mass")
        m = sum(p[0] for p in parts)
        com = sum(p[0] * p[1] for p in parts) / m
        I = np.zeros((3, 3))
        for mi, ci, Ii in parts:
            d = ci - com
            I += Ii + mi * (d @ d * np.eye(3) - np.outer(d, d))
        w, V = np.linalg.eigh(0.5 * (I + I.T))
        if np.linalg.det(V) < 0:
            V[:, 2] = -V[:, 2]
        return m, com, w, mat_to_quat(V)

    if condims:
        if len(set(condims)) != 1:
            raise ValueError("the contacts of the model must share one condim (all frictionless or all with friction)")
        options.setdefault("condim", condims[0])
    if contact_params:
        if len(set(contact_params)) != 1:
            raise ValueError("the collision geoms must share friction, solref and solimp")
        fr, sr, si = contact_params[0]
        options.setdefault("friction", fr)
        options.setdefault("solref", sr)
        options.setdefault("solimp", si)
    # the joints' limit rows: solreflimit / solimplimit, MuJoCo's defaults when absent (friction rows use the same pair here)
    if len(set(limit_params)) > 1:
        raise ValueError("the limited joints must share solreflimit and solimplimit")
    jr, ji = limit_params[0] if limit_params else ((0.02, 1.0), (0.9, 0.95, 0.001, 0.5, 2.0))
    options.setdefault("dof_solref", jr)
    options.setdefault("dof_solimp", ji)
    mb = ModelBuilder(**options)
    joint_body: dict[str, int] = {}

    def add(b, parent):
        m, com, inertia, iquat = composite(b.parts)
        idx = parent
        for k, j in enumerate(b.joints):
            last = k == len(b.joints) - 1
            pos, quat = (b.pos, b.quat) if k == 0 else (np.zeros(3), np.array([1.0, 0, 0, 0]))
            # all but the last joint move a massless body at the same place; the last one carries the body itself
            mass = dict(mass=m, ipos=com, iquat=iquat, inertia=inertia) if last else dict(mass=0.0, inertia=np.zeros(3))
            name = b.name if last else f"{b.name}#{j['name']}"
            if j["type"] == "free":
                idx = mb.add_body(idx, pos, joint="free", quat=quat, name=name, **mass)
            else:
                idx = mb.add_body(idx, pos, joint="hinge", axis=j["axis"], joint_pos=j["pos"], quat=quat, damping=j["damping"],
                                  armature=j["armature"], range=j["range"], frictionloss=j["frictionloss"],
                                  stiffness=j["stiffness"], name=name, **mass)
            joint_body[j["name"]] = idx
        for p, r, n in b.spheres:
            mb.add_contact_sphere(idx, p, r, name=n or None)
        for n, p, q in b.sites:
            mb.add_site(n, idx, p, q)
        for c in b.children:
            add(c, idx)

    add(top, 0)
    act = root.find("actuator")
    for a in ([] if act is None else act):
        if a.tag != "motor":
            raise ValueError(f"actuator <{a.tag}> is outside the model subset (motors only; ksim's PD law runs outside MuJoCo)")
        at = defaults.resolve(a, None)
        if at.get("joint") not in joint_body:
            raise ValueError(f"motor {at.get('name')!r} drives an unknown joint")
        cr = _vec(at.get("ctrlrange"), 2)
        limited = at.get("ctrllimited", "auto")
        mb.add_actuator(joint_body[at["joint"]], gear=float(_vec(at.get("gear"), None, (1.0,))[0]),
                        ctrlrange=None if (cr is None or limited == "false") else tuple(cr))
    sens = root.find("sensor")
    for se in ([] if sens is None else sens):  # sensors that refer to a site; others (joint, actuator sensors) are not read
        site = se.get("site") or (se.get("objname") if se.get("objtype") == "site" else None)
        if site in mb.sites and se.get("name"):
            mb.add_sensor(se.get("name"), se.tag, site)
    return mb.build()
