"""Seeded articulation trees of a chosen number of generalized coordinates, for tests that must reach every compiled
width of the device kernels (the benchmark configurations stop at 7, 18, 36 and 64 coordinates)."""
import numpy as np

from conftest import nk

abi = nk.abi
AXES = ((1, 0, 0), (0, 1, 0), (0, 0, 1))
SPHERE_RADIUS = 0.03


class Tree:
    def __init__(self, template, floating, sphere_links):
        self.template, self.floating, self.sphere_links = template, floating, sphere_links
        self.link_count = template.link_count


def make_tree(dof, floating, branched, seed, mu=0.7, root_height=0.0, limb_joints=7, sphere_limbs=None, sphere_pairs=False):
    """A tree with `dof` coordinates: a floating or fixed root and revolute joints, laid out as one serial chain or as
    limbs of at most `limb_joints` (seven) joints fanning out of the root.  Every limb's last two links carry a contact
    sphere, or only those of the first `sphere_limbs` limbs: the later limbs then carry no shape, like the arms of a
    robot that stands on its feet.  With `sphere_pairs` the spheres of different links also collide with one another,
    so that some contact rows have the articulation on both sides."""
    g = np.random.default_rng(seed)
    t = abi.Template()
    if floating:
        t.add_link(abi.JOINT_FLOATING, None, mass=g.uniform(3.0, 6.0), diag_inertia=tuple(g.uniform(0.03, 0.08, 3)))
    else:
        t.add_link(abi.JOINT_FIXED, None, local_pos=(0, 0, root_height), mass=1.0)
    joints = dof - (6 if floating else 0)
    limb = limb_joints if branched else joints
    sphere_links, made, limbs = [], 0, 0
    while made < joints:
        count = min(limb, joints - made)
        parent = 0
        direction = g.normal(size=3)
        direction[2] = -abs(direction[2]) - 0.5          # limbs hang below the root
        direction /= np.linalg.norm(direction)
        for k in range(count):
            mass = g.uniform(0.3, 2.0)
            length = g.uniform(0.06, 0.14)
            offset = direction * (length if k else 0.08) + (0 if k else g.normal(0, 0.05, 3))
            parent = t.add_link(abi.JOINT_REVOLUTE, parent, axis=AXES[(made + k) % 3], local_pos=tuple(offset), mass=mass,
                                diag_inertia=tuple(mass * g.uniform(0.004, 0.02, 3)), com=tuple(0.5 * length * direction),
                                armature=0.02)
            if k >= count - 2 and (sphere_limbs is None or limbs < sphere_limbs):
                sphere_links.append((parent, tuple(length * direction), SPHERE_RADIUS))
        made += count
        limbs += 1
    profile = t.add_profile(mu)
    t.add_body(abi.ROLE_STATIC, kind=abi.SHAPE_PLANE, contype=2, conaffinity=1, profile=profile)
    for link in range(t.link_count):
        t.add_body(abi.ROLE_LINK_BODY, link=link, kind=abi.SHAPE_NONE, contype=0, conaffinity=0)
    for k, (link, offset, radius) in enumerate(sphere_links):
        # (a negative group never pairs within itself, shape_kind.hpp:26-33: the two spheres of one limb, which sit a
        # link apart, stay out of each other's way and only spheres of different limbs meet)
        t.add_body(abi.ROLE_PROXY, link=link, kind=abi.SHAPE_SPHERE, params=(radius, 0, 0, 0), local_pos=offset,
                   contype=1, conaffinity=3 if sphere_pairs else 2, group=(-(k // 2 + 1)) & 0xFFFFFFFF if sphere_pairs else 0,
                   profile=profile)
    t.max_contacts_per_env = 0 if sphere_pairs else len(sphere_links)   # 0: a slot for every admitted pair
    return Tree(t, floating, sphere_links)


def sphere_heights(oracle_py, tree, desc, state):
    """World height of every contact sphere's centre, per environment, by the oracle's forward kinematics."""
    w = oracle_py.OracleWorld(tree.template, desc, threads=4)
    w.set_state(state)
    w.op("fk_world_poses")
    w.op("sync_link_body_pose")
    E = desc.env_count
    z = w.download("body_pose").reshape(E, -1, 7)[:, -len(tree.sphere_links):, 2].copy()
    w.close()
    return z


def tree_case(oracle_py, dof, floating, branched, seed, E, dt=1.0 / 240.0, vel_iters=8, limb_joints=7, sphere_limbs=None, sphere_pairs=False):
    """(tree, desc, state): seeded joint angles, rates and torques; the root is placed so that each environment's
    lowest sphere presses a few millimetres into the plane (floating root), or so that half of the environments touch
    it (fixed root: the anchor height belongs to the template)."""
    g = np.random.default_rng(seed + 1000)
    tree = make_tree(dof, floating, branched, seed, limb_joints=limb_joints, sphere_limbs=sphere_limbs, sphere_pairs=sphere_pairs)
    nl = tree.link_count
    desc = abi.world_desc(E, dt, vel_iters=vel_iters, contact_margin=0.1)   # spheres a hand above the plane get speculative rows
    q = g.normal(0.0, 0.3, (E, nl)).astype(np.float32)
    qd = g.normal(0.0, 0.5, (E, nl)).astype(np.float32)
    tau = g.normal(0.0, 2.0, (E, nl)).astype(np.float32)
    q[:, 0] = qd[:, 0] = tau[:, 0] = 0.0
    base = np.zeros((E, 7), np.float32)
    tilt = g.normal(0.0, 0.1, (E, 3))
    base[:, 3] = 1.0
    base[:, 4:7] = 0.5 * tilt if floating else 0.0
    base[:, 3:7] /= np.linalg.norm(base[:, 3:7], axis=1, keepdims=True)
    twist = (g.normal(0.0, 0.3, (E, 6)) if floating else np.zeros((E, 6))).astype(np.float32)
    state = dict(q=q, qdot=qd, tau=tau, base_pose=base, root_twist=twist)
    lowest = sphere_heights(oracle_py, tree, desc, state).min(1)
    if floating:
        base[:, 2] = (SPHERE_RADIUS - lowest - g.uniform(0.0, 0.004, E)).astype(np.float32)
    else:
        tree = make_tree(dof, floating, branched, seed, root_height=float(SPHERE_RADIUS - np.median(lowest)), limb_joints=limb_joints,
                         sphere_limbs=sphere_limbs, sphere_pairs=sphere_pairs)
    return tree, desc, state
