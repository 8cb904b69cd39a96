"""Pins of the oracle's contact pipeline (poses -> boxes -> pairs -> manifolds -> rows -> chain Jacobians) by brute
force and by the geometry itself."""
import numpy as np
import pytest

from conftest import nk
from rigid_model import Model, rot

abi = nk.abi
ROW_WORDS = 26
ACTIVE, BLOCK_NORMAL, BLOCK_TANGENT, CONTACT_NORMAL, SPECULATIVE = 1, 1 << 2, 1 << 3, 1 << 6, 1 << 8


def contact_world(oracle_py, index, E, **kw):
    cfg = nk.synthetic.config(index, E)
    w = oracle_py.OracleWorld(cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters, **kw))
    state = cfg.state()
    w.set_state(state)
    for op in ("fk_world_poses", "sync_link_body_pose", "build_aabbs", "query_pairs", "narrowphase", "assemble_rows"):
        w.op(op)
    return cfg, w, state


@pytest.mark.parametrize("index", [2, 3, 5])
def test_body_poses_compose_link_pose_and_local(oracle_py, index):
    E = 3
    cfg, w, state = contact_world(oracle_py, index, E)
    nb = len(cfg.template.bodies)
    body = w.download("body_pose").reshape(E, nb, 7)
    model = Model(cfg.template, abi)
    for e in range(E):
        R, p = model.fk(state["q"][e], rot(state["base_pose"][e, 3:]), state["base_pose"][e, :3].astype(np.float64))
        for b, row in enumerate(cfg.template.bodies):
            local = np.asarray(row["local"], np.float64)
            if row["role"] == abi.ROLE_STATIC:
                expect_p, expect_R = local[:3], rot(local[3:])
            else:
                expect_p, expect_R = p[row["link"]] + R[row["link"]] @ local[:3], R[row["link"]] @ rot(local[3:])
            assert np.abs(body[e, b, :3] - expect_p).max() < 2e-5 * (1 + np.abs(expect_p).max())
            assert np.abs(rot(body[e, b, 3:]) - expect_R).max() < 2e-5
    w.close()


@pytest.mark.parametrize("index", [2, 3, 5])
def test_pairs_are_the_brute_force_overlaps_in_canonical_order(oracle_py, index):
    E = 8
    cfg, w, _ = contact_world(oracle_py, index, E)
    bodies = cfg.template.bodies
    nb = len(bodies)
    aabb = np.concatenate([w.download("body_aabb_lo").reshape(E, nb, 3), w.download("body_aabb_hi").reshape(E, nb, 3)], 2)
    slots = w.download("pair_count").size and w.download("candidate_pairs").size // (2 * E)
    pairs = w.download("candidate_pairs").reshape(E, slots, 2)
    count = w.download("pair_count")
    for e in range(E):
        expect = []
        for a in range(nb):
            for b in range(a + 1, nb):
                ra, rb = bodies[a], bodies[b]
                if ra["kind"] == abi.SHAPE_NONE or rb["kind"] == abi.SHAPE_NONE:
                    continue
                admits = (ra["contype"] & rb["conaffinity"]) or (rb["contype"] & ra["conaffinity"])
                ga, gb = ra["group"], rb["group"]
                if ga != 0 and gb != 0 and ((ga != gb and gb > 0) if ga > 0 else ga == gb):
                    admits = 0
                overlap = np.all(aabb[e, a, :3] <= aabb[e, b, 3:]) and np.all(aabb[e, b, :3] <= aabb[e, a, 3:])
                if admits and overlap:
                    expect.append((a, b))
        assert count[e] == min(len(expect), slots)
        assert [tuple(p) for p in pairs[e, :count[e]]] == expect[:slots]
    w.close()


def test_sphere_boxes_enclose_the_spheres(oracle_py):
    E = 4
    cfg, w, _ = contact_world(oracle_py, 3, E)
    nb = len(cfg.template.bodies)
    aabb = np.concatenate([w.download("body_aabb_lo").reshape(E, nb, 3), w.download("body_aabb_hi").reshape(E, nb, 3)], 2)
    body = w.download("body_pose").reshape(E, nb, 7)
    for b, row in enumerate(cfg.template.bodies):
        if row["kind"] == abi.SHAPE_SPHERE:
            r = row["params"][0]
            assert np.all(aabb[:, b, :3] <= body[:, b, :3] - r) and np.all(aabb[:, b, 3:] >= body[:, b, :3] + r)
            assert np.all(aabb[:, b, 3:] - aabb[:, b, :3] < 2 * r + 4e-3)   # tight up to the contact margin
        if row["kind"] == abi.SHAPE_PLANE:
            assert np.all(aabb[:, b, :2] < -1e30) and np.all(aabb[:, b, 3:5] > 1e30)
    w.close()


@pytest.mark.parametrize("index", [2, 3])
def test_sphere_plane_manifold_geometry(oracle_py, index):
    E = 16
    cfg, w, _ = contact_world(oracle_py, index, E)
    nb = len(cfg.template.bodies)
    slots = w.download("candidate_pairs").size // (2 * E)
    pairs = w.download("candidate_pairs").reshape(E, slots, 2)
    count, points = w.download("pair_count"), w.download("ucontact_count").reshape(E, slots)
    body = w.download("body_pose").reshape(E, nb, 7)
    point = w.download("ucontact_point").reshape(E, slots, 4, 3)
    normal = w.download("ucontact_normal").reshape(E, slots, 4, 3)
    depth = w.download("ucontact_depth").reshape(E, slots, 4)
    separation = 5e-4
    seen = 0
    for e in range(E):
        for s in range(count[e]):
            a, b = pairs[e, s]
            assert cfg.template.bodies[a]["kind"] == abi.SHAPE_PLANE and cfg.template.bodies[b]["kind"] == abi.SHAPE_SPHERE
            r, z = cfg.template.bodies[b]["params"][0], body[e, b, 2]
            gap = z - r                         # the plane is z = 0 with normal +z
            if points[e, s] == 0:
                assert gap >= 2 * separation - 1e-6
                continue
            seen += 1
            assert points[e, s] == 1
            # plane is side A: the normal that separates A from B points from the sphere into the plane... its sign
            # is fixed by the row convention checked below; here: magnitude, depth and the midway point.
            assert abs(abs(normal[e, s, 0, 2]) - 1) < 1e-6
            assert abs(depth[e, s, 0] - (-gap + separation)) < 2e-6
            assert np.abs(point[e, s, 0] - [body[e, b, 0], body[e, b, 1], 0.5 * gap]).max() < 2e-6
    assert seen > E
    w.close()


@pytest.mark.parametrize("index", [2, 3, 5])
def test_row_ranges_are_prefix_compacted_four_rows_per_point(oracle_py, index):
    E = 8
    cfg, w, _ = contact_world(oracle_py, index, E)
    R = w.rows_per_env
    slots = w.download("candidate_pairs").size // (2 * E)
    points = w.download("ucontact_count").reshape(E, slots)
    ranges = w.download("ucontact_row_range").reshape(E, slots, 2)
    flags = w.download("urows").view(np.uint32).reshape(E, R, ROW_WORDS)[:, :, 0]
    for e in range(E):
        carry = 0
        expect_active = np.zeros(R, bool)
        for s in range(slots):
            assert ranges[e, s, 0] == e * R + 4 * carry and ranges[e, s, 1] == points[e, s]
            P = points[e, s]
            for p in range(P):
                for k in range(3):
                    expect_active[4 * carry + k * P + p] = True
            carry += P
        assert np.array_equal((flags[e] & ACTIVE) != 0, expect_active)
        assert w.download("row_count")[e] == expect_active.sum()
    w.close()


@pytest.mark.parametrize("index", [2, 3, 5])
def test_chain_jacobian_gives_the_contact_point_velocity(oracle_py, index):
    """J qdot of every active row equals the row direction dotted with the velocity of the material point of the
    sphere's link at the contact point, from finite differences of the float64 kinematics."""
    E = 3
    cfg, w, state = contact_world(oracle_py, index, E)
    R, md = w.rows_per_env, w.download("chain_jacobian_b").size // (E * w.rows_per_env)
    rows = w.download("urows").reshape(E, R, ROW_WORDS)
    flags = rows.view(np.uint32)[:, :, 0]
    jb = w.download("chain_jacobian_b").reshape(E, R, md)
    ja = w.download("chain_jacobian").reshape(E, R, md)
    link_b = w.download("row_cj_link_b").reshape(E, R)
    point_b = w.download("row_cj_point_b").reshape(E, R, 3)
    model = Model(cfg.template, abi)
    nl = model.nl
    checked = 0
    for e in range(E):
        R0, p0 = rot(state["base_pose"][e, 3:]), state["base_pose"][e, :3].astype(np.float64)
        Rw, pw = model.fk(state["q"][e], R0, p0)
        v = np.array((list(state["root_twist"][e]) if model.floating else []) + [state["qdot"][e, l] for l in model.scalar_links])
        for r in np.nonzero(flags[e] & ACTIVE)[0][:24]:
            assert np.all(ja[e, r] == 0)                       # the plane side is static
            link = link_b[e, r] - e * nl
            assert 0 <= link < nl
            local = Rw[link].T @ (point_b[e, r].astype(np.float64) - pw[link])
            probe = Model(cfg.template, abi)
            probe.links = [dict(l, inertial=list(local) + [1, 0, 0, 0]) if i == link else l for i, l in enumerate(cfg.template.links)]
            _, velocity = probe.link_motion(state["q"][e], R0, p0, v)[link]
            direction = rows[e, r, 20:23]                      # side B linear direction
            expect = direction.astype(np.float64) @ velocity
            got = jb[e, r, :model.dof].astype(np.float64) @ v
            assert abs(got - expect) < 2e-5 * (1 + np.abs(velocity).max())
            checked += 1
    assert checked > 8
    w.close()


def test_rows_carry_the_contact_law(oracle_py):
    E = 16
    cfg, w, _ = contact_world(oracle_py, 2, E)
    R = w.rows_per_env
    rows = w.download("urows").reshape(E, R, ROW_WORDS)
    words = rows.view(np.uint32)
    depth = w.download("row_penetration").reshape(E, R)
    dt = cfg.dt
    normal = (words[:, :, 0] & CONTACT_NORMAL) != 0
    tangent = (words[:, :, 0] & BLOCK_TANGENT) != 0
    assert normal.sum() > 0 and tangent.sum() == 2 * normal.sum()
    assert np.all(words[:, :, 0][normal] == (ACTIVE | CONTACT_NORMAL | BLOCK_NORMAL | SPECULATIVE))
    # speculative law: only an open gap leaves a closing speed, depth / dt per step
    assert np.allclose(rows[:, :, 4][normal], np.minimum(depth[normal], 0) / (dt * dt), rtol=1e-6, atol=0)
    assert np.all(rows[:, :, 6][normal] == 0) and np.all(rows[:, :, 7][normal] > 3e38)
    assert np.all(rows[:, :, 8][normal] == np.float32(0.8)) and np.all(rows[:, :, 8][tangent] == np.float32(0.8))
    # directions: side A (the plane) gets +n, side B -n; tangents complete a right-handed frame with the normal
    for e, r in zip(*np.nonzero(normal)):
        P = words[e, r, 2]
        n, t1, t2 = rows[e, r, 12:15], rows[e, r + P, 12:15], rows[e, r + 2 * P, 12:15]
        assert np.array_equal(rows[e, r, 20:23], -n)
        assert np.abs(np.cross(n, t1) - t2).max() < 1e-6 and abs(np.linalg.norm(n) - 1) < 1e-6
        assert n[2] < -0.99   # from the sphere (B) towards the plane (A): pushing A along +n, B along -n separates them
    w.close()
