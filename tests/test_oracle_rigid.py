"""The oracle's free rigid body against what the mechanics fix: Newton-Euler in free flight (the parabola of the centre of
mass, angular momentum and kinetic energy of a tumbling body, the precession of a symmetric top), the free-rotation
solve against the midpoint rule it states, the six row entries against the velocity of the contact point, and a box on
a plane that carries its weight and stops by Coulomb's law.  The reference's rigid-body ops restated:
articulation.cu:1019-1117, rigid_types.cuh, block_descent_rigid.cuh, block_descent_tile.cuh:541-603."""
import ctypes as C

import numpy as np
import pytest

from conftest import nk
from rigid import body_field, box_template, of_body, rotation_matrix

abi = nk.abi


def make(oracle_py, template, E, dt, gravity=(0.0, 0.0, -9.81), **kw):
    desc = abi.world_desc(E, dt, gravity=gravity, **kw)
    return oracle_py.OracleWorld(template, desc, threads=4), desc


def test_free_rotation_solve_satisfies_the_midpoint_rule(oracle_py):
    """m1 - m0 = dt (m_mid x w_mid) with m = I w in the principal frame: Euler's equations dm/dt = m x w by the implicit
    midpoint rule.  A wrong sign of one of the three products fails it, and so does a midpoint that is not the mean."""
    lib = oracle_py.lib()
    lib.nko_solve_free_rotation.restype = C.c_uint32
    g = np.random.default_rng(5)
    for case in range(50):
        inertia = g.uniform(0.01, 0.5, 3)
        w0 = g.normal(0.0, 8.0, 3)
        dt = float(g.choice([1.0 / 60.0, 1.0 / 240.0, 0.01]))
        f3 = (C.c_float * 3)
        mid, residual, iterations = f3(), C.c_float(), C.c_uint32()
        status = lib.nko_solve_free_rotation(f3(*w0.astype(np.float32)), f3(*(1.0 / inertia).astype(np.float32)), C.c_float(dt), mid,
                                             C.byref(residual), C.byref(iterations))
        assert status == 0 and residual.value <= 1e-6 and iterations.value <= 12
        w_mid = np.array(list(mid), np.float64)
        m0, m_mid = inertia * w0, inertia * w_mid
        m1 = 2.0 * m_mid - m0
        scale = np.abs(m0).max()
        assert np.abs((m1 - m0) - dt * np.cross(m_mid, w_mid)).max() <= 4e-6 * scale, case
        assert abs(np.linalg.norm(m1) - np.linalg.norm(m0)) <= 1e-5 * scale      # the rule keeps |m|
    # nothing turning: no step, status clear; a body without inertia: refused
    mid, residual, iterations = (C.c_float * 3)(), C.c_float(), C.c_uint32()
    assert lib.nko_solve_free_rotation((C.c_float * 3)(0, 0, 0), (C.c_float * 3)(1, 2, 3), C.c_float(0.01), mid, C.byref(residual), C.byref(iterations)) == 0
    assert list(mid) == [0.0, 0.0, 0.0] and iterations.value == 0
    assert lib.nko_solve_free_rotation((C.c_float * 3)(1, 0, 0), (C.c_float * 3)(1, 0, 3), C.c_float(0.01), mid, C.byref(residual), C.byref(iterations)) == 2


def test_free_flight_follows_the_parabola_and_keeps_momentum_and_energy(oracle_py):
    """No contacts: the centre of mass (not the body's origin: the inertial frame sits off it) follows the discrete
    parabola of v += g dt, x += v dt exactly up to rounding; the angular momentum R I R^T w in world axes and the
    rotational energy stay put over two thousand steps of a tumbling body."""
    E, dt, steps = 16, 1.0 / 240.0, 2000
    com = (0.05, -0.02, 0.03)
    t = box_template(half=(0.1, 0.2, 0.05), mass=2.0, diag=(0.02, 0.05, 0.035), com=com, plane=False)
    w, _ = make(oracle_py, t, E, dt)
    g = np.random.default_rng(2)
    pose = np.zeros((E, 7), np.float32)
    pose[:, :3] = g.normal(0.0, 1.0, (E, 3))
    pose[:, 3:] = g.normal(0.0, 1.0, (E, 4))
    pose[:, 3:] /= np.linalg.norm(pose[:, 3:], axis=1, keepdims=True)
    v0 = g.normal(0.0, 1.0, (E, 3)).astype(np.float32)
    w0 = g.normal(0.0, 4.0, (E, 3)).astype(np.float32)
    w.upload("base_pose", pose); w.upload("body_linear_velocity", body_field(t, v0)); w.upload("body_angular_velocity", body_field(t, w0))
    inertia = np.diag([0.02, 0.05, 0.035])

    def measures():
        p = w.download("base_pose").reshape(E, 7).astype(np.float64)
        R = np.stack([rotation_matrix(q) for q in p[:, 3:]])
        centre = p[:, :3] + np.einsum("eij,j->ei", R, np.array(com))
        omega = of_body(t, w.download("body_angular_velocity"), E).astype(np.float64)
        world_inertia = np.einsum("eij,jk,elk->eil", R, inertia, R)
        momentum = np.einsum("eij,ej->ei", world_inertia, omega)
        return centre, momentum, 0.5 * np.einsum("ei,ei->e", omega, momentum)

    c0, l0, k0 = measures()
    w.step(steps)
    c1, l1, k1 = measures()
    assert not w.download("env_status").any() and not w.download("body_gyro_status").any()
    n = steps
    expect = c0 + n * dt * v0.astype(np.float64) + np.array([0.0, 0.0, -9.81]) * dt * dt * n * (n + 1) / 2.0
    assert np.abs(c1 - expect).max() <= 2e-4 * np.abs(expect).max()
    assert np.allclose(of_body(t, w.download("body_linear_velocity"), E), v0 + np.array([0, 0, -9.81]) * dt * n, rtol=2e-5, atol=1e-4)
    # (single precision over two thousand steps: the momentum is rebuilt from the angular velocity at every step)
    assert np.abs(l1 - l0).max() <= 1e-3 * np.abs(l0).max()
    assert np.abs(k1 - k0).max() <= 2e-3 * k0.max()
    assert np.abs(l1 - l0).max() >= 0.0 and np.linalg.norm(w.download("base_pose").reshape(E, 7)[:, 3:], axis=1).max() <= 1.0 + 1e-5
    w.close()


def test_symmetric_top_precesses_at_the_closed_form_rate(oracle_py):
    """A body with two equal principal moments spinning about the third: in the body's frame the transverse angular
    velocity turns about the symmetry axis at (I3 - I1) / I1 * w3 (Euler's equations), and w3 and the transverse size
    stay constant.  The sense of the turn fixes the sign conventions of the whole update."""
    dt, steps = 1.0 / 480.0, 480
    i1, i3 = 0.04, 0.10
    t = box_template(half=(0.1, 0.1, 0.1), mass=1.0, diag=(i1, i1, i3), plane=False)
    w, _ = make(oracle_py, t, 1, dt, gravity=(0.0, 0.0, 0.0))
    w3, wt = 6.0, 1.5
    w.upload("body_angular_velocity", body_field(t, np.array([[wt, 0.0, w3]], np.float32)))
    w.step(steps)
    pose = w.download("base_pose").reshape(7).astype(np.float64)
    body = rotation_matrix(pose[3:]).T @ of_body(t, w.download("body_angular_velocity"), 1)[0].astype(np.float64)
    rate = (i3 - i1) / i1 * w3
    angle = rate * dt * steps
    # Euler: dw1/dt = -(I3 - I1)/I1 w3 w2, dw2/dt = +(I3 - I1)/I1 w3 w1: the transverse part turns by +rate about axis 3
    expect = np.array([wt * np.cos(angle), wt * np.sin(angle), w3])
    assert np.abs(body - expect).max() <= 2e-3 * w3, (body, expect)
    w.close()


def test_row_entries_times_the_coordinates_are_the_contact_point_velocity(oracle_py):
    """J [v; w] of every active row = direction . (v + w x (point - com)), the point velocity of a rigid body, with the
    centre of mass off the body's origin."""
    E, dt = 24, 1.0 / 240.0
    com = (0.03, 0.01, -0.02)
    t = box_template(half=(0.2, 0.15, 0.1), mass=3.0, diag=(0.03, 0.04, 0.05), com=com)
    w, desc = make(oracle_py, t, E, dt, vel_iters=8, contact_margin=0.05)
    g = np.random.default_rng(9)
    pose = np.zeros((E, 7), np.float32)
    pose[:, 2] = 0.1 + g.uniform(-0.004, 0.01, E)
    tilt = g.normal(0.0, 0.03, (E, 3))
    pose[:, 3] = 1.0; pose[:, 4:] = 0.5 * tilt
    pose[:, 3:] /= np.linalg.norm(pose[:, 3:], axis=1, keepdims=True)
    v = g.normal(0.0, 0.3, (E, 3)).astype(np.float32)
    om = g.normal(0.0, 1.0, (E, 3)).astype(np.float32)
    w.upload("base_pose", pose); w.upload("body_linear_velocity", body_field(t, v)); w.upload("body_angular_velocity", body_field(t, om))
    zero_gravity = w
    for name in ("body_integrate_velocity", "fk_world_poses", "sync_link_body_pose", "build_aabbs", "query_pairs", "narrowphase", "assemble_rows"):
        zero_gravity.op(name)
    R = w.rows_per_env
    rows = w.download("urows").reshape(E, R, 26)
    flags = rows.view(np.uint32)[:, :, 0]
    J = w.download("chain_jacobian").reshape(E, R, -1)[:, :, :6].astype(np.float64) + w.download("chain_jacobian_b").reshape(E, R, -1)[:, :, :6].astype(np.float64)
    points = w.download("row_cj_point").reshape(E, R, 3).astype(np.float64) + 0.0
    points_b = w.download("row_cj_point_b").reshape(E, R, 3).astype(np.float64)
    link_a = w.download("row_cj_link").reshape(E, R)
    vel = of_body(t, w.download("body_linear_velocity"), E).astype(np.float64)
    omega = of_body(t, w.download("body_angular_velocity"), E).astype(np.float64)
    p = w.download("base_pose").reshape(E, 7).astype(np.float64)
    checked = 0
    for e in range(E):
        centre = p[e, :3] + rotation_matrix(p[e, 3:]) @ np.array(com)
        for r in range(R):
            if not flags[e, r] & 1:
                continue
            on_a = link_a[e, r] != 0xFFFFFFFF
            point = points[e, r] if on_a else points_b[e, r]
            direction = rows[e, r, 12:15].astype(np.float64) if on_a else rows[e, r, 20:23].astype(np.float64)
            expect = direction @ (vel[e] + np.cross(omega[e], point - centre))
            got = J[e, r] @ np.concatenate([vel[e], omega[e]])
            assert abs(got - expect) <= 2e-6 * (1.0 + abs(expect)), (e, r, got, expect)
            checked += 1
    assert checked >= 4 * E
    w.close()


def test_a_box_at_rest_carries_its_weight_and_a_sliding_box_stops_by_coulombs_law(oracle_py):
    E, dt = 2, 1.0 / 240.0
    mu, mass = 0.5, 2.0
    t = box_template(half=(0.2, 0.2, 0.1), mass=mass, diag=(0.04, 0.04, 0.06), mu=mu)
    w, _ = make(oracle_py, t, E, dt, vel_iters=16, pos_iters=4)
    pose = np.zeros((E, 7), np.float32)
    pose[:, 2] = 0.1; pose[:, 3] = 1.0
    v = np.zeros((E, 3), np.float32)
    v[1, 0] = 1.0                                       # the second box slides along x
    w.upload("base_pose", pose); w.upload("body_linear_velocity", body_field(t, v))
    R = w.rows_per_env
    n = 30
    w.step(n)
    assert not w.download("env_status").any()
    lam = w.download("lambda").reshape(E, R)
    rows = w.download("urows").reshape(E, R, 26).view(np.uint32)
    normal = (rows[:, :, 0] & (1 << 6)) != 0
    support = np.where(normal, lam, 0.0).sum(1) / dt     # the rows' impulses over the step: a force
    assert np.allclose(support, mass * 9.81, rtol=2e-3), support
    speeds = of_body(t, w.download("body_linear_velocity"), E)
    assert np.abs(speeds[0]).max() <= 1e-4                                   # at rest stays at rest
    assert abs(speeds[1, 0] - (1.0 - mu * 9.81 * n * dt)) <= 5e-3, speeds[1]  # Coulomb: deceleration mu g
    assert abs(w.download("base_pose").reshape(E, 7)[0, 2] - 0.1) <= 1e-3
    w.step(80)                                                               # ... and comes to a stop, not back
    assert np.abs(of_body(t, w.download("body_linear_velocity"), E)[1]).max() <= 2e-3
    w.close()
