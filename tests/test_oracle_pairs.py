"""Pins of the oracle beyond shape-against-plane contact: pairs of two moving collidables (both sides of a row on
the articulation), capsule and cylinder supports, and the excluded-pair list.  The manifolds themselves are pinned
bit-exact against the reference's own header (test_golden_vectors.py::test_every_analytic_pair); here the physics
that follows from them is checked against closed forms: momentum of a collision, the weight carried by a support."""
import numpy as np
import pytest

from conftest import nk

abi = nk.abi
ROW_WORDS = 26
CONTACT_NORMAL = 1 << 6
IDENTITY7 = np.array([0, 0, 0, 1, 0, 0, 0], np.float32)


def contact_step(oracle_py, template, desc, state, solve=True):
    w = oracle_py.OracleWorld(template, desc, threads=2)
    w.set_state(state)
    w.op("fk_world_poses")
    w.op("articulation_dynamics", 1)
    for op in ("sync_link_body_pose", "build_aabbs", "query_pairs", "narrowphase", "assemble_rows"):
        w.op(op)
    E, R = desc.env_count, w.rows_per_env
    out = dict(pairs=w.download("pair_count").copy(), count=w.download("ucontact_count").reshape(E, -1).copy(),
               candidate=w.download("candidate_pairs").reshape(E, -1, 2).copy())
    if solve:
        w.op("contact_warm_start", 0)
        w.op("block_descent_solve")
        out["qdot"] = w.download("qdot").reshape(E, -1).astype(np.float64)
        out["twist"] = w.download("link_velocity").reshape(E, template.link_count, 6)[:, 0, :].astype(np.float64)
        out["lambda"] = w.download("lambda").reshape(E, R).astype(np.float64)
        out["rows"] = w.download("urows").reshape(E, R, ROW_WORDS).copy()
        out["status"] = w.download("env_status").copy()
        out["residual"] = w.download("solver_residual").reshape(E, 4).copy()
    w.close()
    return out


def rails(m1, m2, radius, exclude=False, same_link=False):
    """A fixed base with two sliders along x, a sphere on each."""
    t = abi.Template()
    t.add_link(abi.JOINT_FIXED, None, mass=1.0)
    a = t.add_link(abi.JOINT_PRISMATIC, 0, axis=(1, 0, 0), mass=m1)
    b = t.add_link(abi.JOINT_PRISMATIC, 0, axis=(1, 0, 0), mass=m2)
    rows = []
    for link in (a, b):
        t.add_body(abi.ROLE_LINK_BODY, link=link, contype=0, conaffinity=0)
    for link in ((a, a) if same_link else (a, b)):
        rows.append(t.add_body(abi.ROLE_PROXY, link=link, kind=abi.SHAPE_SPHERE, params=(radius, 0, 0, 0), contype=1, conaffinity=1))
    if exclude:
        t.exclude(rows[1], rows[0])
    return t


def rail_state(q, qdot):
    q, qdot = np.asarray(q, np.float32), np.asarray(qdot, np.float32)
    z = np.zeros((len(q), 1), np.float32)
    return dict(q=np.concatenate([z, q], 1), qdot=np.concatenate([z, qdot], 1), tau=np.zeros((len(q), 3), np.float32),
                base_pose=np.tile(IDENTITY7, (len(q), 1)), root_twist=np.zeros((len(q), 6), np.float32))


def test_two_spheres_collide_and_keep_their_momentum(oracle_py):
    """Two sliders on one axis meet: the row keeps them from closing, so they leave with the common velocity
    (m1 v1 + m2 v2) / (m1 + m2); a pair that separates, or one that is still a gap apart, is left alone."""
    m1, m2, radius, dt = 0.8, 2.0, 0.05, 1.0 / 200.0
    touching = 2 * radius - 1e-3
    q = [[0.0, touching], [0.0, touching], [0.0, touching + 0.05]]
    qdot = [[1.0, -0.5], [-0.2, 0.3], [1.0, -0.5]]
    out = contact_step(oracle_py, rails(m1, m2, radius), abi.world_desc(3, dt, gravity=(0, 0, 0), vel_iters=50), rail_state(q, qdot))
    assert list(out["pairs"]) == [1, 1, 0] and np.all(out["status"] == 0) and np.all(out["residual"] < 2e-5)
    common = (m1 * 1.0 + m2 * -0.5) / (m1 + m2)
    assert np.abs(out["qdot"][0, 1:] - common).max() < 2e-5
    assert np.abs(out["qdot"][1, 1:] - [-0.2, 0.3]).max() < 1e-6 and np.abs(out["lambda"][1]).max() == 0
    assert np.abs(out["qdot"][2, 1:] - [1.0, -0.5]).max() < 1e-6
    # the impulse is the momentum either sphere gives up
    normal = np.nonzero(out["rows"].view(np.uint32)[0, :, 0] & CONTACT_NORMAL)[0]
    assert len(normal) == 1 and abs(out["lambda"][0, normal[0]] - m1 * (1.0 - common)) < 2e-5


def test_rows_of_one_link_and_excluded_rows_never_pair(oracle_py):
    """Overlapping spheres: a pair when nothing excludes it; none when the pair is listed (either order), and none for
    two rows of the same link."""
    state = rail_state([[0.0, 0.05]], [[0.0, 0.0]])
    desc = abi.world_desc(1, 1.0 / 200.0, gravity=(0, 0, 0))
    assert contact_step(oracle_py, rails(1, 1, 0.05), desc, state, solve=False)["pairs"][0] == 1
    assert contact_step(oracle_py, rails(1, 1, 0.05, exclude=True), desc, state, solve=False)["pairs"][0] == 0
    assert contact_step(oracle_py, rails(1, 1, 0.05, same_link=True), desc, state, solve=False)["pairs"][0] == 0


def floating(kind, params, mass, inertia, mu=0.8):
    t = abi.Template()
    t.add_link(abi.JOINT_FLOATING, None, mass=mass, diag_inertia=inertia)
    profile = t.add_profile(mu)
    t.add_body(abi.ROLE_STATIC, kind=abi.SHAPE_PLANE, contype=2, conaffinity=1, profile=profile)
    t.add_body(abi.ROLE_LINK_BODY, link=0, contype=0, conaffinity=0)
    t.add_body(abi.ROLE_PROXY, link=0, kind=kind, params=params, contype=1, conaffinity=2, profile=profile)
    return t


def floating_state(pose):
    z = np.zeros((1, 1), np.float32)
    return dict(q=z, qdot=z, tau=z, base_pose=np.asarray([pose], np.float32), root_twist=np.zeros((1, 6), np.float32))


@pytest.mark.parametrize("shape", ["capsule_lying", "capsule_standing", "cylinder_standing", "cylinder_lying"])
def test_supports_carry_the_weight(oracle_py, shape):
    """A capsule or cylinder at rest on the plane: the normal impulses add up to m g dt, it stays at rest, and a
    symmetric support shares the weight evenly."""
    mass, radius, half, dt, g = 1.3, 0.04, 0.1, 1.0 / 200.0, 9.81
    lying = [np.sqrt(0.5), 0, np.sqrt(0.5), 0]   # local z along world x
    kind = abi.SHAPE_CAPSULE if shape.startswith("capsule") else abi.SHAPE_CYLINDER
    if shape.endswith("lying"):
        pose, points = [0, 0, radius - 1e-3] + lying, 2
    else:
        height = (half + radius if kind == abi.SHAPE_CAPSULE else half) - 1e-3
        pose, points = [0, 0, height, 1, 0, 0, 0], 1 if kind == abi.SHAPE_CAPSULE else 4
    out = contact_step(oracle_py, floating(kind, (radius, half, 0, 0), mass, (0.01, 0.01, 0.01)),
                       abi.world_desc(1, dt, vel_iters=100), floating_state(pose))
    assert out["pairs"][0] == 1 and out["count"][0, 0] == points and out["status"][0] == 0
    normal = np.nonzero(out["rows"].view(np.uint32)[0, :, 0] & CONTACT_NORMAL)[0]
    assert len(normal) == points
    lam = out["lambda"][0, normal]
    assert abs(lam.sum() - mass * g * dt) < 3e-5 * mass
    assert np.abs(out["twist"][0]).max() < 3e-5
    if points == 2:
        assert np.abs(lam - lam.mean()).max() < 1e-3 * lam.mean()


def box_on_slab(mass):
    """A floating box over a static slab (a box as well) whose top face lies in the plane z = 0."""
    t = abi.Template()
    t.add_link(abi.JOINT_FLOATING, None, mass=mass, diag_inertia=(0.01, 0.012, 0.009))
    profile = t.add_profile(0.8)
    t.add_body(abi.ROLE_STATIC, kind=abi.SHAPE_BOX, params=(0.5, 0.4, 0.1, 0), local_pos=(0, 0, -0.1), contype=2, conaffinity=1, profile=profile)
    t.add_body(abi.ROLE_LINK_BODY, link=0, contype=0, conaffinity=0)
    t.add_body(abi.ROLE_PROXY, link=0, kind=abi.SHAPE_BOX, params=(0.08, 0.06, 0.05, 0), contype=1, conaffinity=2, profile=profile)
    return t


def test_box_rests_on_a_box(oracle_py):
    """Face on face: the clipped incident face gives four points that carry the weight between them; turned about
    the vertical by any angle the box still rests (the clip polygon changes, the support does not)."""
    mass, dt, g = 2.1, 1.0 / 200.0, 9.81
    for angle in (0.0, 0.3, 0.7853982):
        pose = [0.02, -0.01, 0.05 - 1e-3, np.cos(angle / 2), 0, 0, np.sin(angle / 2)]
        out = contact_step(oracle_py, box_on_slab(mass), abi.world_desc(1, dt, vel_iters=100), floating_state(pose))
        assert out["pairs"][0] == 1 and out["count"][0, 0] == 4 and out["status"][0] == 0
        normal = np.nonzero(out["rows"].view(np.uint32)[0, :, 0] & CONTACT_NORMAL)[0]
        lam = out["lambda"][0, normal]
        assert len(normal) == 4 and abs(lam.sum() - mass * g * dt) < 3e-5 * mass and lam.min() > 0.1 * lam.mean()
        assert np.abs(out["twist"][0]).max() < 3e-5


def test_readout_of_a_link_pair_is_action_and_reaction(oracle_py):
    """Two sliders pressed together by opposite forces: the contact readout gives each link the other's push - equal,
    opposite, of the size that holds the forces apart - and names both owners."""
    m1, m2, radius, dt = 0.8, 2.0, 0.05, 1.0 / 200.0
    state = rail_state([[0.0, 2 * radius - 1e-3]], [[0.0, 0.0]])
    state["tau"] = np.array([[0.0, 3.0, -3.0]], np.float32)
    w = oracle_py.OracleWorld(rails(m1, m2, radius), abi.world_desc(1, dt, gravity=(0, 0, 0), vel_iters=50, pos_iters=0xFFFFFFFF), threads=1)
    w.set_state(state)
    w.step(1)
    w.op("readout_contact_wrench")
    wrench = w.download("link_contact_wrench").reshape(3, 6)
    assert np.abs(w.download("qdot")).max() < 2e-5                                  # the pair stays put
    assert wrench[1, 0] == pytest.approx(-3.0, rel=1e-3) and wrench[2, 0] == pytest.approx(3.0, rel=1e-3)
    assert np.abs(wrench[1, :3] + wrench[2, :3]).max() < 1e-5 and np.abs(wrench[0]).max() == 0
    # equal and opposite about the world origin as well: the two forces share a line of action
    assert np.abs(wrench[1, 3:] + wrench[2, 3:]).max() < 1e-5
    assert w.download("contact_side_a_kind")[0] == 1 and w.download("contact_side_b_kind")[0] == 1     # both sides on the articulation
    assert sorted([int(w.download("contact_side_a_index")[0]), int(w.download("contact_side_b_index")[0])]) == [1, 2]
    w.close()
