"""Seeded synthetic worlds for the five benchmark configurations.

Every configuration is one articulation template shared by all environments plus independent per-environment
state.  Templates are drawn from a fixed per-configuration seed; state uses one Philox stream per quantity
filled in environment order, so the first E environments are identical for every larger environment count.
Joint layout and sampling distributions follow the workload descriptions: C1 7-DoF chain, C2 12-joint quadruped
on a floating base, C3/C4 30-joint humanoid on a floating base (2x6 legs, 3 waist, 2x7 arms, 1 head: 36 DoF)
with 12 foot contact spheres, C5 64-link rope with one contact sphere per link.
"""
import math

import numpy as np

from .abi import (JOINT_FIXED, JOINT_FLOATING, JOINT_REVOLUTE, ROLE_LINK_BODY, ROLE_PROXY, ROLE_STATIC,
                  SHAPE_BOX, SHAPE_NONE, SHAPE_PLANE, SHAPE_SPHERE, Template)

SEED = 0xC0FFEE
X, Y, Z = (1, 0, 0), (0, 1, 0), (0, 0, 1)


def _rng(config, quantity):
    return np.random.Generator(np.random.Philox(key=SEED + 1000 * config + quantity))


class Config:
    def __init__(self, index, name, template, dt, vel_iters, env_count, sampler, nominal_q, floating, note=""):
        self.index, self.name, self.template = index, name, template
        self.note = note          # what the published table leaves open and this configuration fixes, for the bench line
        self.dt, self.vel_iters, self.env_count = dt, vel_iters, env_count
        self._sampler, self.nominal_q, self.floating = sampler, nominal_q, floating

    def state(self, env_count=None):
        """Seeded state arrays, float32, env-major: q, qdot, tau [E, nl]; base_pose [E, 7]; root_twist [E, 6]."""
        return self._sampler(self.env_count if env_count is None else env_count)


def _add_collidable_rows(t, spheres, mu):
    """Plane at row 0, one shapeless row per link, then the contact spheres as proxy collidables."""
    profile = t.add_profile(mu)
    t.add_body(ROLE_STATIC, kind=SHAPE_PLANE, contype=2, conaffinity=1, profile=profile)
    for link in range(t.link_count):
        t.add_body(ROLE_LINK_BODY, link=link, kind=SHAPE_NONE, contype=0, conaffinity=0)
    for link, offset, radius in spheres:
        t.add_body(ROLE_PROXY, link=link, kind=SHAPE_SPHERE, params=(radius, 0, 0, 0), local_pos=offset,
                   contype=1, conaffinity=2, profile=profile)
    t.max_contacts_per_env = len(spheres)


def chain7(env_count=64):
    g = _rng(1, 0)
    t = Template()
    t.add_link(JOINT_FIXED, None, mass=1.0)
    axes = [Z, Y, Z, Y, Z, Y, Z]
    prev_len = 0.0
    for i in range(7):
        mass, length = g.uniform(0.5, 2.0), g.uniform(0.1, 0.4)
        inertia = g.uniform(1e-3, 1e-2, size=3)
        t.add_link(JOINT_REVOLUTE, i, axis=axes[i], local_pos=(0, 0, prev_len), mass=mass, diag_inertia=inertia,
                   com=(0, 0, 0.5 * length))
        prev_len = length
    nl = t.link_count

    def sample(E):
        q = np.zeros((E, nl), np.float32)
        qd = np.zeros((E, nl), np.float32)
        tau = np.zeros((E, nl), np.float32)
        q[:, 1:] = _rng(1, 1).uniform(-math.pi, math.pi, size=(E, 7))
        qd[:, 1:] = _rng(1, 2).normal(0.0, 1.0, size=(E, 7))
        tau[:, 1:] = _rng(1, 3).normal(0.0, 5.0, size=(E, 7))
        base = np.tile(np.array([0, 0, 0, 1, 0, 0, 0], np.float32), (E, 1))
        return dict(q=q, qdot=qd, tau=tau, base_pose=base, root_twist=np.zeros((E, 6), np.float32))

    return Config(1, "chain7", t, 1.0 / 500.0, 0, env_count, sample, np.zeros(nl, np.float32), False)


def quadruped(env_count=4096):
    g = _rng(2, 0)
    t = Template()
    t.add_link(JOINT_FLOATING, None, mass=12.0, diag_inertia=(0.12, 0.35, 0.40))
    spheres, nominal = [], [0.0]
    for sx in (1, -1):
        for sy in (1, -1):
            hip = t.add_link(JOINT_REVOLUTE, 0, axis=X, local_pos=(0.2 * sx, 0.1 * sy, 0.0), mass=g.uniform(0.5, 1.5),
                             diag_inertia=g.uniform(1e-3, 5e-3, size=3), com=(0, 0.03 * sy, 0))
            thigh = t.add_link(JOINT_REVOLUTE, hip, axis=Y, local_pos=(0, 0.05 * sy, 0), mass=g.uniform(0.5, 1.5),
                               diag_inertia=g.uniform(2e-3, 8e-3, size=3), com=(0, 0, -0.1))
            shank = t.add_link(JOINT_REVOLUTE, thigh, axis=Y, local_pos=(0, 0, -0.2), mass=g.uniform(0.5, 1.5),
                               diag_inertia=g.uniform(1e-3, 5e-3, size=3), com=(0, 0, -0.1))
            spheres.append((shank, (0, 0, -0.2), 0.02))
            nominal += [0.0, 0.7, -1.4]
    _add_collidable_rows(t, spheres, 0.8)
    nl = t.link_count
    nominal = np.array(nominal, np.float32)

    def sample(E):
        q = (nominal[None, :] + _rng(2, 1).normal(0.0, 0.1, size=(E, nl))).astype(np.float32)
        q[:, 0] = 0.0
        tau = _rng(2, 3).normal(0.0, 10.0, size=(E, nl)).astype(np.float32)
        tau[:, 0] = 0.0
        base = np.tile(np.array([0, 0, 0, 1, 0, 0, 0], np.float32), (E, 1))
        base[:, 2] = _rng(2, 4).uniform(0.25, 0.35, size=E)
        return dict(q=q, qdot=np.zeros((E, nl), np.float32), tau=tau, base_pose=base,
                    root_twist=np.zeros((E, 6), np.float32))

    return Config(2, "quadruped", t, 1.0 / 200.0, 8, env_count, sample, nominal, True)


def humanoid(env_count=4096, index=3):
    g = _rng(3, 0)
    t = Template()

    def link(parent, axis, pos, com, scale=1.0):
        m = g.uniform(0.3, 4.0)
        return t.add_link(JOINT_REVOLUTE, parent, axis=axis, local_pos=pos, mass=m,
                          diag_inertia=m * scale * g.uniform(0.004, 0.02, size=3), com=com)

    pelvis = t.add_link(JOINT_FLOATING, None, mass=g.uniform(3.0, 4.0), diag_inertia=(0.04, 0.03, 0.05))
    nominal = [0.0]
    spheres = []
    for sy in (1, -1):
        hip_yaw = link(pelvis, Z, (0, 0.1 * sy, -0.05), (0, 0, -0.02))
        hip_roll = link(hip_yaw, X, (0, 0, -0.04), (0, 0, -0.02))
        hip_pitch = link(hip_roll, Y, (0, 0, -0.04), (0, 0, -0.2))
        knee = link(hip_pitch, Y, (0, 0, -0.4), (0, 0, -0.2))
        ankle_pitch = link(knee, Y, (0, 0, -0.4), (0, 0, -0.01))
        ankle_roll = link(ankle_pitch, X, (0, 0, -0.02), (0.03, 0, -0.03))
        nominal += [0.0, 0.0, -0.25, 0.5, -0.25, 0.0]
        for px, py in ((0.12, 0.04), (0.12, -0.04), (0.02, 0.045), (0.02, -0.045), (-0.06, 0.04), (-0.06, -0.04)):
            spheres.append((ankle_roll, (px, py, -0.05), 0.01))
    waist_yaw = link(pelvis, Z, (0, 0, 0.08), (0, 0, 0.03))
    waist_roll = link(waist_yaw, X, (0, 0, 0.05), (0, 0, 0.03))
    torso = link(waist_roll, Y, (0, 0, 0.05), (0, 0, 0.2))
    nominal += [0.0, 0.0, 0.0]
    for sy in (1, -1):
        sh_pitch = link(torso, Y, (0, 0.2 * sy, 0.35), (0, 0.02 * sy, 0))
        sh_roll = link(sh_pitch, X, (0, 0.03 * sy, 0), (0, 0, -0.03))
        sh_yaw = link(sh_roll, Z, (0, 0, -0.05), (0, 0, -0.12))
        elbow = link(sh_yaw, Y, (0, 0, -0.25), (0, 0, -0.1))
        wr_yaw = link(elbow, Z, (0, 0, -0.2), (0, 0, -0.02), 0.3)
        wr_pitch = link(wr_yaw, Y, (0, 0, -0.04), (0, 0, -0.02), 0.3)
        link(wr_pitch, X, (0, 0, -0.03), (0, 0, -0.04), 0.3)
        nominal += [0.0, 0.15 * sy, 0.0, -0.3, 0.0, 0.0, 0.0]
    link(torso, Z, (0, 0, 0.45), (0, 0, 0.08))
    nominal += [0.0]
    _add_collidable_rows(t, spheres, 1.0)
    nl = t.link_count
    nominal = np.array(nominal, np.float32)
    # pelvis height at which the nominal pose rests its sole spheres on the plane
    leg = 0.05 + 0.04 + 0.04 + 0.4 * math.cos(0.25) + 0.4 * math.cos(0.25) + 0.02 + 0.05 + 0.01
    c = 30   # C3 and C4 share one state stream

    def sample(E):
        q = (nominal[None, :] + _rng(c, 1).normal(0.0, 0.15, size=(E, nl))).astype(np.float32)
        q[:, 0] = 0.0
        qd = _rng(c, 2).normal(0.0, 0.5, size=(E, nl)).astype(np.float32)
        qd[:, 0] = 0.0
        tau = _rng(c, 3).normal(0.0, 20.0, size=(E, nl)).astype(np.float32)
        tau[:, 0] = 0.0
        base = np.zeros((E, 7), np.float32)
        base[:, 2] = leg - 0.015 + _rng(c, 4).uniform(-0.02, 0.02, size=E)
        tilt = _rng(c, 5).normal(0.0, 0.05, size=(E, 3))
        base[:, 3] = 1.0
        base[:, 4:7] = 0.5 * tilt
        base[:, 3:7] /= np.linalg.norm(base[:, 3:7], axis=1, keepdims=True)
        twist = _rng(c, 6).normal(0.0, 0.5, size=(E, 6)).astype(np.float32)
        return dict(q=q, qdot=qd, tau=tau, base_pose=base.astype(np.float32), root_twist=twist)

    return Config(index, "humanoid", t, 1.0 / 200.0, 8, env_count, sample, nominal, True)


ROPE_RADIUS, ROPE_LINK, ROPE_REST_DEPTH = 0.01, 0.05, 5.0e-4
# Sixty-four links of 50 to 200 g, each pressed on the plane by a penalty of a hundred times its own inverse
# response, give a Newton block whose condition number (about 1e9) is past what a single-precision Cholesky can
# factor from either end of the chain.  A reflected rotor inertia on every joint, the one term that adds to the whole
# diagonal of the mass matrix, brings it to about 1e5.
ROPE_ARMATURE = 0.01


def _rope_lie(draw):
    """Joint angles of a rope that lies on the plane, from one N(0, 0.3) draw per joint.

    Joints alternate pitch (y, even links) and yaw (z, odd links).  A yaw joint takes its draw as its angle.  Sixty-four
    independent pitch angles of that size would carry the rope metres above and below the plane (the height is the
    double sum of the pitch angles), where no contact problem is posed; a pitch joint therefore takes the angle that
    brings the joint two links on back to the rope's rest height plus its own draw read in millimetres, so that every
    sphere rests on the plane within a millimetre of the nominal penetration and each environment has its own lie.
    """
    E = draw.shape[0]
    q = np.zeros((E, 64))
    rot = np.tile(np.eye(3), (E, 1, 1))            # world rotation of the parent link
    origin = np.zeros((E, 3))                      # world position of the current joint, relative to the anchor
    for i in range(0, 64, 2):
        psi = draw[:, i + 1]
        a, b, c = rot[:, 2, 0], rot[:, 2, 1], rot[:, 2, 2]
        target = 1.0e-3 * draw[:, i] - origin[:, 2]
        k = (target / ROPE_LINK - np.sin(psi) * b) / (1.0 + np.cos(psi))
        theta = np.arctan2(a, c) - np.arcsin(np.clip(k / np.hypot(a, c), -1.0, 1.0))
        q[:, i], q[:, i + 1] = theta, psi
        ct, st, cp, sp = np.cos(theta), np.sin(theta), np.cos(psi), np.sin(psi)
        zero, one = np.zeros(E), np.ones(E)
        ry = np.stack([ct, zero, st, zero, one, zero, -st, zero, ct], 1).reshape(E, 3, 3)
        rz = np.stack([cp, -sp, zero, sp, cp, zero, zero, zero, one], 1).reshape(E, 3, 3)
        rot = rot @ ry
        origin = origin + ROPE_LINK * rot[:, :, 0]
        rot = rot @ rz
        origin = origin + ROPE_LINK * rot[:, :, 0]
    return q


def rope(env_count=8192):
    g = _rng(5, 0)
    t = Template()
    t.add_link(JOINT_FIXED, None, local_pos=(0, 0, ROPE_RADIUS - ROPE_REST_DEPTH), mass=1.0)
    spheres = []
    for i in range(64):
        m = g.uniform(0.05, 0.2)
        link = t.add_link(JOINT_REVOLUTE, i, axis=Y if i % 2 == 0 else Z, local_pos=(ROPE_LINK if i else 0.0, 0, 0),
                          mass=m, diag_inertia=(m * 2.5e-5, m * 2.3e-4, m * 2.3e-4), com=(0.5 * ROPE_LINK, 0, 0),
                          armature=ROPE_ARMATURE)
        spheres.append((link, (0.5 * ROPE_LINK, 0, 0), ROPE_RADIUS))
    _add_collidable_rows(t, spheres, 0.5)
    nl = t.link_count

    def sample(E):
        q = np.zeros((E, nl), np.float32)
        q[:, 1:] = _rope_lie(_rng(5, 1).normal(0.0, 0.3, size=(E, 64)))
        base = np.tile(np.array([0, 0, 0, 1, 0, 0, 0], np.float32), (E, 1))
        return dict(q=q, qdot=np.zeros((E, nl), np.float32), tau=np.zeros((E, nl), np.float32), base_pose=base,
                    root_twist=np.zeros((E, 6), np.float32))

    note = (f"joint armature {ROPE_ARMATURE} kg.m^2 on every joint; joint angles solved per environment so that the rope lies on "
            f"the plane, every sphere within 1 mm (sigma 0.3 mm) of {1e3 * ROPE_REST_DEPTH:.1f} mm penetration, yaw angles N(0, 0.3 rad); zero rates and torques")
    return Config(5, "rope64", t, 1.0 / 500.0, 16, env_count, sample, np.zeros(nl, np.float32), False, note)


def free_box(env_count=4096):
    """Not one of the published configurations: a free rigid body, a box of 0.4 x 0.3 x 0.2 m with its centre of mass off
    the middle, dropped a few millimetres onto the plane with a small tilt, push and spin (four-point manifolds)."""
    t = Template()
    t.free_body = True
    t.add_link(JOINT_FLOATING, None, mass=3.0, diag_inertia=(0.03, 0.04, 0.05), com=(0.03, 0.01, -0.02))
    profile = t.add_profile(0.6)
    t.add_body(ROLE_STATIC, kind=SHAPE_PLANE, contype=2, conaffinity=1, profile=profile)
    t.add_body(ROLE_LINK_BODY, link=0, kind=SHAPE_BOX, params=(0.2, 0.15, 0.1, 0.0), contype=1, conaffinity=2, profile=profile)
    t.max_contacts_per_env = 1

    def sample(E):
        pose = np.zeros((E, 7), np.float32)
        pose[:, :2] = _rng(6, 0).normal(0.0, 0.5, (E, 2))
        pose[:, 2] = 0.1 + _rng(6, 1).uniform(-0.004, 0.01, E)
        pose[:, 3] = 1.0
        pose[:, 4:] = 0.5 * _rng(6, 2).normal(0.0, 0.03, (E, 3))
        pose[:, 3:] /= np.linalg.norm(pose[:, 3:], axis=1, keepdims=True)
        linear, angular = np.zeros((E, 2, 3), np.float32), np.zeros((E, 2, 3), np.float32)   # per body row: the plane's, the box's
        linear[:, 1] = _rng(6, 3).normal(0.0, 0.3, (E, 3))
        angular[:, 1] = _rng(6, 4).normal(0.0, 1.0, (E, 3))
        zeros = np.zeros((E, 1), np.float32)
        return dict(q=zeros, qdot=zeros.copy(), tau=zeros.copy(), base_pose=pose, root_twist=np.zeros((E, 6), np.float32),
                    body_linear_velocity=linear, body_angular_velocity=angular)

    return Config(6, "free_box", t, 1.0 / 240.0, 8, env_count, sample, np.zeros(1, np.float32), True,
                  note="a free rigid body stepped by the rigid-body ops, outside the published configurations")


def config(index, env_count=None):
    """Benchmark configuration by number 1..5; 4 is the humanoid at a swept environment count; 6 is a free rigid box,
    outside the published table."""
    makers = {1: chain7, 2: quadruped, 3: humanoid, 4: lambda e=4096: humanoid(e, 4), 5: rope, 6: free_box}
    return makers[index]() if env_count is None else makers[index](env_count)
