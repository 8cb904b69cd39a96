"""Pins of the oracle's MuJoCo contact law: merged profile terms against the reference's own merge, the reference
weights against closed forms and a dense evaluation, the compliant rows against the pinned row math and the row
geometry, and a resting body against the penetration the spring-damper reference fixes."""
import ctypes as C

import numpy as np
import pytest

from conftest import nk
from rigid_model import Model, rot

abi = nk.abi
F = C.c_float
ROW_WORDS = 26
ACTIVE, BLOCK_NORMAL, BLOCK_TANGENT, CONTACT_NORMAL, SPECULATIVE, MUJOCO, PYRAMIDAL = 1, 1 << 2, 1 << 3, 1 << 6, 1 << 8, 1 << 11, 1 << 12


def farr(values):
    return (F * len(values))(*[float(v) for v in values])


def test_profile_merge_matches_the_reference(oracle_py, ref_lib):
    """MergeContactParams (scene/contact_filter.hpp:89-137), the reference's own header beside the restatement, on
    random profiles: equal and different priorities, solmix weights down to the deferring zero, direct-form solref
    (the minimum branch), condim 1 and 3; then the known answers of tests/scene/test_filter_precedence.cpp."""
    L = oracle_py.lib()
    g = np.random.default_rng(5)
    for case in range(400):
        sides = []
        for _ in range(2):
            solref = g.uniform(0.005, 0.1, 2) if g.random() < 0.7 else -g.uniform(10.0, 500.0, 2)
            solmix = 0.0 if g.random() < 0.15 else g.uniform(0.1, 2.0)
            sides.append(np.concatenate([g.uniform(0.1, 1.5, 2), solref, g.uniform(0.5, 0.99, 2), g.uniform(1e-4, 1e-2, 1),
                                         g.uniform(0.1, 0.9, 1), g.uniform(1.0, 3.0, 1), g.uniform(0.0, 0.01, 2),
                                         [g.integers(-1, 2), solmix, g.choice([1, 3])]]).astype(np.float32))
        mine, theirs = (F * 12)(), (F * 12)()
        L.nko_merge_contact_params(farr(sides[0]), farr(sides[1]), mine)
        ref_lib.ref_merge_params(farr(sides[0]), farr(sides[1]), theirs)
        assert np.array_equal(np.array(mine[:], np.float32).view(np.uint32), np.array(theirs[:], np.float32).view(np.uint32)), case

    def merged(a, b):
        out = (F * 12)()
        L.nko_merge_contact_params(farr(a), farr(b), out)
        return np.array(out[:], np.float32)

    def side(mu=1.0, solref=(0.02, 1.0), solimp=(0.9, 0.95, 0.001, 0.5, 2.0), margin=0.0, gap=0.0, priority=0, solmix=1.0, condim=3):
        return [mu, mu, *solref, *solimp, margin, gap, priority, solmix, condim]

    # :37-74 equal priority: friction and condim by max, solref and solimp by solmix 1 : 3
    m = merged(side(0.3, (0.1, 2.0), (0,) * 5, 0.01, 0.02, 2, 1.0, 3), side(0.7, (0.2, 4.0), (1,) * 5, 0.03, 0.05, 2, 3.0, 1))
    assert m[0] == np.float32(0.7) and m[11] == 3
    # (EXPECT_FLOAT_EQ there: four units in the last place)
    assert m[2] == pytest.approx(0.175, rel=3e-7) and m[3] == np.float32(3.5) and (m[4:9] == np.float32(0.75)).all()
    # :80-113 the higher priority supplies friction and condim and, through the weight, solref and solimp
    hi = side(0.9, (0.07, 1.5), (0.1, 0.2, 0.3, 0.4, 0.5), 0.09, 0.08, 5, 1.0, 1)
    lo = side(0.2, (0.5, 9.0), (0.99,) * 5, 0.001, 0.002, 1, 1.0, 3)
    for m in (merged(hi, lo), merged(lo, hi)):
        assert m[0] == np.float32(0.9) and m[11] == 1 and m[2] == np.float32(0.07) and m[3] == np.float32(1.5)
        assert np.array_equal(m[4:9], np.float32([0.1, 0.2, 0.3, 0.4, 0.5]))
    # :119-145 a direct-form solref on either side takes the elementwise minimum
    assert tuple(merged(side(solref=(-3.0, -50.0)), side(solref=(-5.0, -10.0)))[2:4]) == (-5.0, -50.0)
    assert tuple(merged(side(solref=(0.2, 4.0)), side(solref=(-5.0, -10.0)))[2:4]) == (-5.0, -10.0)
    # :153-183 a zero solmix defers to the other side; two valid ones mix
    a, b = side(solref=(0.1, 1.0), solimp=(0.9, 0.95, 0.001, 0.5, 2.0)), side(solref=(0.3, 9.0), solimp=(0.5, 0.95, 0.001, 0.5, 2.0), solmix=0.0)
    for m in (merged(a, b), merged(b, a)):
        assert m[2] == np.float32(0.1) and m[3] == np.float32(1.0) and m[4] == np.float32(0.9)
    b[12] = 1.0
    m = merged(a, b)
    assert m[2] == np.float32(0.5 * np.float32(0.1) + 0.5 * np.float32(0.3)) and m[4] == np.float32(0.5 * np.float32(0.9) + 0.5 * np.float32(0.5))


def weights_world(oracle_py, template, q=None, base=None):
    w = oracle_py.OracleWorld(template, abi.world_desc(1, 0.005))
    if q is not None:
        w.upload("q", q)
    if base is not None:
        w.upload("base_pose", base)
    w.op("fk_world_poses")
    w.op("reference_weights")
    return w


def test_reference_weights_of_a_free_body(oracle_py):
    """A floating body answers a force at its centre of mass with 1/m and a moment with the mean inverse principal
    inertia, wherever the centre sits in the link frame and however the body is turned (articulation.cu:455-500)."""
    mass, inertia, com = 2.5, (0.02, 0.05, 0.09), (0.1, -0.2, 0.05)
    t = abi.Template()
    t.add_link(abi.JOINT_FLOATING, None, mass=mass, diag_inertia=inertia, com=com)
    t.add_body(abi.ROLE_LINK_BODY, link=0, kind=abi.SHAPE_SPHERE, params=(0.1, 0, 0, 0))
    quat = np.array([0.5, 0.5, -0.5, 0.5], np.float32)
    w = weights_world(oracle_py, t, base=np.concatenate([[0.3, 0.1, 1.0], quat]).astype(np.float32))
    body = w.download("body_invweight0")
    assert body[0] == pytest.approx(1.0 / mass, rel=2e-5)
    assert body[1] == pytest.approx(np.mean(1.0 / np.array(inertia)), rel=2e-5)
    # the base coordinates: rotation about the link origin (not the centre of mass), translation of the origin
    c = np.array(com)
    about_origin = np.diag(inertia) + mass * (c @ c * np.eye(3) - np.outer(c, c))
    spatial = np.block([[about_origin, mass * np.array([[0, -c[2], c[1]], [c[2], 0, -c[0]], [-c[1], c[0], 0]])],
                        [-mass * np.array([[0, -c[2], c[1]], [c[2], 0, -c[0]], [-c[1], c[0], 0]]), mass * np.eye(3)]])
    inverse = np.diag(np.linalg.inv(spatial))
    dof = w.download("dof_invweight0")
    assert np.allclose(dof[:3], inverse[:3].mean(), rtol=5e-5) and np.allclose(dof[3:6], inverse[3:].mean(), rtol=5e-5)
    w.close()


def test_reference_weights_of_a_pendulum(oracle_py):
    """One hinge: M = I_axis + m r^2 + armature; a unit force at the centre of mass moves it r^2 / M along the one
    direction the hinge allows, a unit moment 1 / M about the axis - each averaged over three axes."""
    mass, r, iyy, armature = 1.7, 0.35, 0.04, 0.015
    t = abi.Template()
    t.add_link(abi.JOINT_FIXED, None, mass=1.0)
    t.add_link(abi.JOINT_REVOLUTE, 0, axis=(0, 1, 0), mass=mass, diag_inertia=(0.01, iyy, 0.02), com=(r, 0, 0), armature=armature)
    t.add_body(abi.ROLE_LINK_BODY, link=0, kind=abi.SHAPE_NONE)
    t.add_body(abi.ROLE_LINK_BODY, link=1, kind=abi.SHAPE_SPHERE, params=(0.05, 0, 0, 0))
    w = weights_world(oracle_py, t, q=np.array([0.0, 0.8], np.float32))
    M = iyy + mass * r * r + armature
    body = w.download("body_invweight0").reshape(-1, 2)
    assert body[1, 0] == pytest.approx(r * r / M / 3.0, rel=2e-5)
    assert body[1, 1] == pytest.approx(1.0 / M / 3.0, rel=2e-5)
    assert tuple(body[0]) == (0.0, 0.0)   # the fixed root moves under nothing
    assert w.download("dof_invweight0")[0] == pytest.approx(1.0 / M, rel=2e-5)
    w.close()


def test_reference_weights_of_a_chain_match_a_dense_evaluation(oracle_py):
    """tr(J M^-1 J^T) / 3 per link with J from central differences of an independent float64 forward kinematics and M
    the oracle's own mass matrix (pinned elsewhere against the same model)."""
    cfg = nk.synthetic.config(1, 1)
    t = cfg.template
    for link in range(t.link_count):   # config 1 has no collidable rows; the weights are per collidable row of a link
        t.add_body(abi.ROLE_LINK_BODY, link=link, kind=abi.SHAPE_NONE)
    state = cfg.state(1)
    w = weights_world(oracle_py, t, q=state["q"])
    nl, n = t.link_count, t.dof
    M = w.download("m").reshape(n, n).astype(np.float64)
    model = Model(t, abi)
    q0 = state["q"][0].astype(np.float64)
    moving = [l for l in range(nl) if t.links[l]["joint_type"] != abi.JOINT_FIXED]

    def com_and_frames(q):
        R, p = model.fk(q, np.eye(3), np.zeros(3))
        return [p[l] + R[l] @ np.array(t.links[l]["inertial"][:3]) for l in range(nl)], R

    h = 1e-6
    J_lin, J_ang = np.zeros((nl, 3, n)), np.zeros((nl, 3, n))
    _, R0 = com_and_frames(q0)
    for d, link in enumerate(moving):
        qp, qm = q0.copy(), q0.copy()
        qp[link] += h
        qm[link] -= h
        cp, Rp = com_and_frames(qp)
        cm, Rm = com_and_frames(qm)
        for l in range(nl):
            J_lin[l, :, d] = (cp[l] - cm[l]) / (2 * h)
            spin = (Rp[l] - Rm[l]) @ R0[l].T / (2 * h)
            J_ang[l, :, d] = [spin[2, 1], spin[0, 2], spin[1, 0]]
    Minv = np.linalg.inv(M)
    body = w.download("body_invweight0").reshape(-1, 2)
    for l in range(nl):
        assert body[l, 0] == pytest.approx(np.trace(J_lin[l] @ Minv @ J_lin[l].T) / 3.0, rel=2e-3, abs=1e-7)
        assert body[l, 1] == pytest.approx(np.trace(J_ang[l] @ Minv @ J_ang[l].T) / 3.0, rel=2e-3, abs=1e-7)
    assert np.allclose(w.download("dof_invweight0")[:n], np.diag(Minv), rtol=2e-3)
    w.close()


def mujoco_config(index, E, cone, **profile):
    cfg = nk.synthetic.config(index, E)
    for p in cfg.template.profiles:
        p.update(law=abi.LAW_MUJOCO, **profile)
    cfg.template.contact_cone = cone
    return cfg


def assembled(oracle_py, cfg, E, qdot=None):
    w = oracle_py.OracleWorld(cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters))
    state = cfg.state(E)
    state["base_pose"][:, 2] -= 0.12   # feet into the ground band
    if qdot is not None:
        state["qdot"][:] = qdot
    w.set_state(state)
    for op in ("snapshot_step_velocity", "fk_world_poses"):
        w.op(op)
    w.op("articulation_dynamics", 1)
    for op in ("sync_link_body_pose", "build_aabbs", "query_pairs", "narrowphase", "assemble_rows"):
        w.op(op)
    return w, state


def test_compliant_rows_of_an_elliptic_world(oracle_py):
    """assemble_rows.cu:692-797 for a MuJoCo-sourced profile: the normal row carries the discretised spring-damper
    reference at its depth with the summed body weights, the tangent rows their compliance, both flagged for the
    elliptic cone; the reference gain times the start velocity along the row is part of the right-hand side."""
    E = 4
    L = oracle_py.lib()
    solref, solimp, margin = (0.03, 0.9), (0.85, 0.97, 0.002, 0.4, 2.5), 0.004
    cfg = mujoco_config(2, E, abi.CONE_ELLIPTIC, solref=solref, solimp=solimp, margin=(margin, 0.0))
    cfg.template.contact_impratio = 2.0
    rng = np.random.default_rng(3)
    nl = cfg.template.link_count
    w, state = assembled(oracle_py, cfg, E, qdot=rng.normal(0.0, 0.5, (E, nl)).astype(np.float32))
    R, md = w.rows_per_env, w.dof
    rows = w.download("urows").view(np.uint32).reshape(E, R, ROW_WORDS)
    rowsf = rows.view(np.float32)
    law = w.download("ucontact_law")
    assert set(law[w.download("ucontact_count") > 0]) == {0}   # compliant
    ranges = w.download("ucontact_row_range").reshape(E, -1, 2)
    counts = w.download("ucontact_count").reshape(E, -1)
    depth = w.download("ucontact_depth").reshape(E, -1, 4)
    weights = w.download("body_invweight0").reshape(E, -1, 2)
    gain = w.download("row_reference_velocity_gain").reshape(E, R)
    invweight_rows = w.download("row_invweight").reshape(E, R)
    ja = w.download("chain_jacobian").reshape(E, R, md)
    jb = w.download("chain_jacobian_b").reshape(E, R, md)
    start = w.download("step_qdot_flat").reshape(E, md)
    cj_link, cj_link_b = w.download("row_cj_link").reshape(E, R), w.download("row_cj_link_b").reshape(E, R)
    mu = cfg.template.profiles[0]["mu"][0]
    merged_margin = 2.0 * margin   # both sides carry the profile; margins add
    seen = 0
    for e in range(E):
        for s in range(ranges.shape[1]):
            if counts[e, s] == 0:
                continue
            base, P = ranges[e, s, 0] - e * R, ranges[e, s, 1]
            for p in range(min(counts[e, s], 4)):
                if not depth[e, s, p] + merged_margin > 0.0:
                    assert rows[e, base + p, 0] == 0
                    continue
                seen += 1
                n_row, t_rows = base + p, (base + P + p, base + 2 * P + p)
                assert rows[e, n_row, 0] == ACTIVE | CONTACT_NORMAL | BLOCK_NORMAL | MUJOCO
                # the plane is static (weight 0); the sphere's weight is that of its link's own collidable row, 1 + link
                link = min(cj_link[e, n_row], cj_link_b[e, n_row]) - e * nl
                invweight = weights[e, 1 + link, 0]
                assert invweight_rows[e, n_row] == np.float32(invweight)
                pos = np.float32(-depth[e, s, p]) - np.float32(merged_margin)
                terms, discrete = (F * 6)(), (F * 3)()
                L.nko_compliant_row_terms(farr(solref), farr(solimp), F(pos), F(pos), F(0.0), F(invweight), F(cfg.dt), 1, terms)
                L.nko_discretize_compliant_row(F(terms[4]), F(terms[5]), F(terms[1]), F(cfg.dt), discrete)
                velocity = np.float32(0.0)   # side A's row, then side B's (the plane's is empty)
                for side in (ja, jb):
                    for d in range(md):
                        velocity = np.float32(velocity + np.float32(side[e, n_row, d] * start[e, d]))
                assert velocity != 0.0
                assert rowsf[e, n_row, 5] == np.float32(discrete[0])
                assert gain[e, n_row] == np.float32(discrete[2])
                assert rowsf[e, n_row, 4] == np.float32(np.float32(discrete[1]) + np.float32(gain[e, n_row] * velocity))
                for k, tr in enumerate(t_rows):
                    assert rows[e, tr, 0] == ACTIVE | BLOCK_TANGENT | MUJOCO
                    tangent_weight = np.float32(np.float32(invweight) / np.float32(2.0) * np.float32(mu * mu) / np.float32(mu * mu))
                    L.nko_compliant_row_terms(farr(solref), farr(solimp), F(pos), F(0.0), F(0.0), F(tangent_weight), F(cfg.dt), 1, terms)
                    L.nko_discretize_compliant_row(F(terms[4]), F(terms[5]), F(terms[1]), F(cfg.dt), discrete)
                    assert rowsf[e, tr, 5] == np.float32(discrete[0])
                    assert invweight_rows[e, tr] == tangent_weight
    assert seen >= E
    w.close()


def test_pyramidal_rows_are_the_edges_of_the_friction_pyramid(oracle_py):
    """assemble_rows.cu:651-690: four scalar rows a point along n +- mu t; two opposite edges sum to twice the normal
    direction, their difference is 2 mu times a unit tangent orthogonal to the normal, and the two tangents are
    orthogonal.  The Jacobian rows are linear in the direction, so the same holds for them."""
    E = 4
    cfg = mujoco_config(2, E, abi.CONE_PYRAMIDAL)
    w, _ = assembled(oracle_py, cfg, E)
    R, md = w.rows_per_env, w.dof
    rows = w.download("urows").view(np.uint32).reshape(E, R, ROW_WORDS)
    rowsf = rows.view(np.float32)
    ranges = w.download("ucontact_row_range").reshape(E, -1, 2)
    counts = w.download("ucontact_count").reshape(E, -1)
    normals = w.download("ucontact_normal").reshape(E, -1, 4, 3)
    ja = w.download("chain_jacobian").reshape(E, R, md).astype(np.float64)
    mu = cfg.template.profiles[0]["mu"][0]
    seen = 0
    for e in range(E):
        for s in range(ranges.shape[1]):
            base, P = ranges[e, s, 0] - e * R, ranges[e, s, 1]
            for p in range(min(counts[e, s], 4)):
                edge_rows = [base + k * P + p for k in range(4)]
                if rows[e, edge_rows[0], 0] == 0:
                    continue
                seen += 1
                for k, r in enumerate(edge_rows):
                    assert rows[e, r, 0] == ACTIVE | MUJOCO | PYRAMIDAL | (CONTACT_NORMAL if k == 0 else 0)
                    assert rows[e, r, 2] == 1 and rowsf[e, r, 6] == 0.0 and rowsf[e, r, 5] > 0.0
                dirs = rowsf[e, edge_rows, 12:15].astype(np.float64)
                n = normals[e, s, p].astype(np.float64)
                n /= np.linalg.norm(n)
                assert np.allclose(dirs[0] + dirs[1], 2 * n, atol=1e-6) and np.allclose(dirs[2] + dirs[3], 2 * n, atol=1e-6)
                t1, t2 = (dirs[0] - dirs[1]) / (2 * mu), (dirs[2] - dirs[3]) / (2 * mu)
                assert abs(np.linalg.norm(t1) - 1) < 1e-5 and abs(np.linalg.norm(t2) - 1) < 1e-5
                assert abs(t1 @ n) < 1e-5 and abs(t2 @ n) < 1e-5 and abs(t1 @ t2) < 1e-5
                assert np.allclose(ja[e, edge_rows[0]] + ja[e, edge_rows[1]], ja[e, edge_rows[2]] + ja[e, edge_rows[3]], atol=1e-5)
    assert seen >= E
    w.close()


def resting_sphere(cone, solref, solimp):
    t = abi.Template()
    t.add_link(abi.JOINT_FLOATING, None, mass=3.0, diag_inertia=(0.02, 0.02, 0.02))
    profile = t.add_profile(0.9, law=abi.LAW_MUJOCO, solref=solref, solimp=solimp)
    t.add_body(abi.ROLE_STATIC, kind=abi.SHAPE_PLANE, profile=profile)
    t.add_body(abi.ROLE_LINK_BODY, link=0, kind=abi.SHAPE_SPHERE, params=(0.1, 0, 0, 0), profile=profile)
    t.contact_cone = cone
    return t


@pytest.mark.parametrize("free_body", [False, True])
@pytest.mark.parametrize("cone", [abi.CONE_ELLIPTIC, abi.CONE_PYRAMIDAL])
def test_a_resting_sphere_sinks_to_the_depth_of_the_spring_reference(oracle_py, cone, free_body):
    """At rest the contact force is the weight and the row equation a + R f = aref holds with a = 0: f = aref / R with
    aref = k imp depth and R = invweight (1 - imp) / imp (constraint/solref_solimp.hpp:55-86), which fixes the depth.
    A pyramid's four edges share the load and each is softer, with the edge weight of assemble_rows.cu:652.  The ball as
    a one-link articulation and as a free rigid body (the rigid-body ops, BodyReferenceWeightsKernel's inverse mass)."""
    L = oracle_py.lib()
    solref, solimp, dt, mass, g = (0.02, 1.0), (0.9, 0.95, 0.001, 0.5, 2.0), 0.002, 3.0, 9.81
    t = resting_sphere(cone, solref, solimp)
    t.free_body = free_body
    w = oracle_py.OracleWorld(t, abi.world_desc(1, dt, vel_iters=16, velocity_tolerance=1e-7))
    w.upload("base_pose", np.array([0, 0, 0.0999, 1, 0, 0, 0], np.float32))
    w.step(1500)
    assert w.download("env_status")[0] == 0
    height = w.download("base_pose")[2]
    assert abs(w.download("body_linear_velocity").reshape(2, 3)[1, 2] if free_body else w.download("link_velocity")[5]) < 1e-4
    if free_body:
        assert np.allclose(w.download("body_invweight0").reshape(2, 2)[1], [1.0 / mass, 1.0 / 0.02], rtol=1e-6)
    depth = 0.1 - height
    mu = 0.9
    invweight = 1.0 / mass
    if cone == abi.CONE_PYRAMIDAL:
        invweight = (invweight + mu * mu * invweight) * 2.0 * mu * mu
    # the normal row carries m g; a pyramid's four edges a quarter of it each, their tangent parts cancelling
    force = mass * g if cone == abi.CONE_ELLIPTIC else mass * g / 4.0
    lo, hi = 0.0, 0.01
    for _ in range(60):   # bisection on depth: aref / R rises with depth
        mid = 0.5 * (lo + hi)
        terms = (F * 6)()
        L.nko_compliant_row_terms(farr(solref), farr(solimp), F(-mid), F(-mid), F(0.0), F(invweight), F(dt), 1, terms)
        if terms[5] / terms[4] < force:
            lo = mid
        else:
            hi = mid
    assert depth == pytest.approx(0.5 * (lo + hi), rel=0.03), (depth, lo)
    w.close()


def test_frictionless_contacts_have_the_normal_row_alone(oracle_py):
    """condim 1 (assemble_rows.cu:721, 763): the normal row is a single-axis head, no tangent rows; both laws."""
    E = 2
    for law, cone in ((abi.LAW_NATIVE, abi.CONE_PYRAMIDAL), (abi.LAW_MUJOCO, abi.CONE_PYRAMIDAL), (abi.LAW_MUJOCO, abi.CONE_ELLIPTIC)):
        cfg = nk.synthetic.config(2, E)
        for p in cfg.template.profiles:
            p.update(law=law, condim=1)
        cfg.template.contact_cone = cone
        w, _ = assembled(oracle_py, cfg, E)
        R = w.rows_per_env
        flags = w.download("urows").view(np.uint32).reshape(E, R, ROW_WORDS)[:, :, 0]
        active = flags[(flags & ACTIVE) != 0]
        assert active.size >= E
        assert ((active & (BLOCK_NORMAL | BLOCK_TANGENT | PYRAMIDAL)) == 0).all() and ((active & CONTACT_NORMAL) != 0).all()
        assert (((active & MUJOCO) != 0) == (law == abi.LAW_MUJOCO)).all()
        w.step(20)   # and the solve runs on such heads
        assert (w.download("env_status") == 0).all()
        w.close()


def hinge(law, **joint):
    """A fixed base and one hinge about y carrying a point-like link: M = I_yy + m r^2 + armature."""
    t = abi.Template()
    t.add_link(abi.JOINT_FIXED, None, mass=1.0)
    t.add_link(abi.JOINT_REVOLUTE, 0, axis=(0, 1, 0), mass=1.5, diag_inertia=(0.01, 0.03, 0.02), com=(0.2, 0, 0), armature=0.01, law=law, **joint)
    return t, 0.03 + 1.5 * 0.2 * 0.2 + 0.01


def test_a_compliant_joint_limit_gives_way_as_the_spring_reference_says(oracle_py):
    """A constant torque presses a MuJoCo-sourced hinge against its upper limit (assemble_rows.cu:860-877): at rest the
    row equation a + R f = aref holds with a = 0 and f the torque, with the coordinate's reference weight 1 / M as the
    row's weight, which fixes how far the joint passes its limit.  The lower row of the same joint stays inactive."""
    L = oracle_py.lib()
    reference, torque, dt, upper = (0.03, 1.0, 0.85, 0.96, 0.002, 0.5, 2.0), 2.0, 0.002, 0.3
    t, M = hinge(abi.LAW_MUJOCO, lower=-0.4, upper=upper, damping=0.4, limit_reference=reference, limit_margin=0.0)
    w = oracle_py.OracleWorld(t, abi.world_desc(1, dt, gravity=(0, 0, 0), vel_iters=16, velocity_tolerance=1e-7))
    assert w.download("dof_invweight0")[0] == pytest.approx(1.0 / M, rel=1e-5)
    w.upload("q", np.array([0.0, 0.25], np.float32))
    tau = np.array([0.0, torque], np.float32)
    for _ in range(3000):
        w.upload("tau", tau)
        w.step()
    assert w.download("env_status")[0] == 0 and abs(w.download("qdot")[1]) < 1e-5
    R = w.rows_per_env
    flags = w.download("urows").view(np.uint32).reshape(R, ROW_WORDS)[:, 0]
    # two limit row slots a link: the hinge's are 2 and 3; its lower bound is off, its upper bound on
    assert flags[2] == (1 << 4) | MUJOCO and flags[3] == ACTIVE | (1 << 5) | MUJOCO
    assert w.download("lambda")[3] / dt == pytest.approx(torque, rel=1e-3)
    passed = w.download("q")[1] - upper
    lo, hi = 0.0, 0.05
    for _ in range(60):
        mid = 0.5 * (lo + hi)
        terms = (F * 6)()
        L.nko_compliant_row_terms(farr(reference[:2]), farr(reference[2:]), F(-mid), F(-mid), F(0.0), F(1.0 / M), F(dt), 1, terms)
        lo, hi = (mid, hi) if terms[5] / terms[4] < torque else (lo, mid)
    assert passed == pytest.approx(0.5 * (lo + hi), rel=0.03)
    w.close()


def test_mujoco_dry_friction_row_carries_its_reference(oracle_py):
    """assemble_rows.cu:921-931: the friction row of a MuJoCo-sourced joint is regularised by its own solref / solimp
    at the coordinate's reference weight; a torque below the friction loss leaves the joint at rest but for the slip the
    regularisation admits, R times the held impulse."""
    L = oracle_py.lib()
    reference, dt, loss, torque = (0.01, 1.0, 0.9, 0.95, 0.001, 0.5, 2.0), 0.002, 0.5, 0.3
    t, M = hinge(abi.LAW_MUJOCO, frictionloss=loss, friction_reference=reference)
    w = oracle_py.OracleWorld(t, abi.world_desc(1, dt, gravity=(0, 0, 0), vel_iters=16, velocity_tolerance=1e-8))
    w.upload("tau", np.array([0.0, torque], np.float32))
    w.step()
    rows = w.download("urows").view(np.uint32).reshape(-1, ROW_WORDS)
    assert rows[1, 0] == ACTIVE | (1 << 7) | MUJOCO          # one friction row slot a link: the hinge's is 1
    terms, discrete = (F * 6)(), (F * 3)()
    L.nko_compliant_row_terms(farr(reference[:2]), farr(reference[2:]), F(0.0), F(0.0), F(0.0), F(1.0 / M), F(dt), 1, terms)
    L.nko_discretize_compliant_row(F(terms[4]), F(terms[5]), F(terms[1]), F(dt), discrete)
    assert rows.view(np.float32)[1, 5] == np.float32(discrete[0]) and discrete[0] > 0.0
    # the friction holds (its impulse stays inside the bounds) and the momentum balance M v = dt torque + lambda closes;
    # what the regularisation lets through is a small slip along the torque, where the native row holds v = 0
    lam, v = float(w.download("lambda")[1]), float(w.download("qdot")[1])
    assert -loss * dt < lam < 0.0
    assert M * v == pytest.approx(dt * torque + lam, rel=1e-3, abs=1e-8)
    assert 0.0 < v < 0.2 * dt * torque / M
    w.close()
    t, _ = hinge(abi.LAW_NATIVE, frictionloss=loss)
    w = oracle_py.OracleWorld(t, abi.world_desc(1, dt, gravity=(0, 0, 0), vel_iters=16, velocity_tolerance=1e-8))
    w.upload("tau", np.array([0.0, torque], np.float32))
    w.step()
    assert abs(float(w.download("qdot")[1])) < 1e-7
    w.close()


def test_mujoco_integrator_applies_joint_damping_implicitly(oracle_py):
    """ArticulationDamping (articulation.cu:950-1000) on one hinge: v+ = v + dt (tau - b v) / (M + dt b), the implicit
    Euler step of the damping, against the explicit one of the native integrator; then on the seven-joint chain the
    step's velocity change against (M + dt D)^-1 M applied densely in float64."""
    dt, b, torque = 0.01, 3.0, 0.7
    t, M = hinge(abi.LAW_NATIVE, damping=b)
    for integrator in (abi.INTEGRATOR_NATIVE, abi.INTEGRATOR_MUJOCO_EULER):
        t.integrator = integrator
        w = oracle_py.OracleWorld(t, abi.world_desc(1, dt, gravity=(0, 0, 0)))
        v = 0.0
        for _ in range(50):
            w.upload("tau", np.array([0.0, torque], np.float32))
            w.step()
            v = v + dt * (torque - b * v) / (M + (dt * b if integrator else 0.0))
            assert w.download("qdot")[1] == pytest.approx(v, rel=2e-5)
        w.close()
    cfg = nk.synthetic.config(1, 2)
    for link in cfg.template.links[1:]:
        link["damping"] = 0.8
    cfg.template.integrator = abi.INTEGRATOR_MUJOCO_EULER
    w = oracle_py.OracleWorld(cfg.template, abi.world_desc(2, cfg.dt))
    state = cfg.state(2)
    w.set_state(state)
    w.op("snapshot_step_velocity"); w.op("fk_world_poses"); w.op("articulation_dynamics", 1)
    n = w.dof
    before, solved = state["qdot"][:, 1:].astype(np.float64), w.download("qdot").reshape(2, -1)[:, 1:].astype(np.float64)
    mass = w.download("m").reshape(2, n, n).astype(np.float64)
    w.op("articulation_damping")
    after = w.download("qdot").reshape(2, -1)[:, 1:]
    for e in range(2):
        D = cfg.dt * 0.8 * np.eye(n)
        expect = before[e] + np.linalg.solve(mass[e] + D, mass[e] @ (solved[e] - before[e]))
        assert np.allclose(after[e], expect, rtol=2e-4, atol=1e-6)
    assert np.abs(after - solved).max() > 1e-4
    w.close()
