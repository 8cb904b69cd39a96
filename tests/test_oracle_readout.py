"""Pins of the oracle's contact readout (ReadoutContactWrench) against statics and momentum: a resting ball reads its
weight, a sliding ball reads Coulomb friction and its moment about the centre, and on the quadruped the link
wrenches add up to the base-frame generalized impulse J^T lambda that the solve itself applied."""
import numpy as np
import pytest

from conftest import nk
from test_oracle_solver import ball, ball_state

abi = nk.abi
G = 9.81


def stepped(oracle_py, template, desc, state, steps=1):
    w = oracle_py.OracleWorld(template, desc, threads=2)
    w.set_state(state)
    w.step(steps)
    w.op("readout_contact_wrench")
    return w


def test_resting_ball_reads_its_weight(oracle_py):
    mass, radius, dt = 0.7, 0.05, 1.0 / 200.0
    desc = abi.world_desc(1, dt, vel_iters=8, pos_iters=0xFFFFFFFF)
    w = stepped(oracle_py, ball(mass, radius), desc, ball_state([radius], [[0, 0, 0, 0, 0, 0]]))
    wrench = w.download("link_contact_wrench").reshape(1, 1, 6)[0, 0]
    assert wrench[2] == pytest.approx(mass * G, rel=2e-4)
    assert np.abs(wrench[[0, 1, 3, 4, 5]]).max() <= 1e-5 * mass * G
    force = w.download("contact_force").reshape(1, 1, 3)[0, 0]
    assert force[0] == pytest.approx(mass * G, rel=2e-4) and abs(force[1]) < 1e-4 and abs(force[2]) < 1e-4
    impulse = w.download("ucontact_impulse").reshape(1, 1, 4, 3)[0, 0]
    # side A of the pair (plane, sphere) is the plane: the normal of side A points the way the plane must move
    assert impulse[0, 2] == pytest.approx(-mass * G * dt, rel=2e-4) and not impulse[1:].any()
    assert w.download("contact_side_a_kind")[0] == 3 and w.download("contact_side_b_kind")[0] == 1
    assert w.download("contact_side_a_index")[0] == 0xFFFFFFFF and w.download("contact_side_b_index")[0] == 0
    assert w.download("contact_link")[0] == 0
    point = w.download("contact_point").reshape(1, 1, 3)[0, 0]
    assert abs(point[2]) < 1e-3 and w.download("contact_normal").reshape(1, 1, 3)[0, 0, 2] == pytest.approx(-1.0)
    w.close()


def test_sliding_ball_reads_coulomb_friction_and_its_moment(oracle_py):
    mass, radius, mu, dt = 0.7, 0.05, 0.3, 1.0 / 200.0
    desc = abi.world_desc(1, dt, vel_iters=8, pos_iters=0xFFFFFFFF)
    # fast slide along +x without spin: friction saturates at mu m g along -x, acting at the sphere's lowest point
    w = stepped(oracle_py, ball(mass, radius, mu), desc, ball_state([radius], [[0, 0, 0, 2.0, 0, 0]]))
    wrench = w.download("link_contact_wrench").reshape(6)
    assert wrench[2] == pytest.approx(mass * G, rel=2e-4)
    assert wrench[0] == pytest.approx(-mu * mass * G, rel=5e-4)
    lever = w.download("contact_point").reshape(3) - w.download("link_pose").reshape(7)[:3]
    assert np.allclose(wrench[3:], np.cross(lever, wrench[:3]), rtol=1e-4, atol=1e-7)
    # about +y: r_z f_x - r_x f_z with f = (-mu m g, 0, m g).  The readout runs at the end of the step, so the lever goes
    # from the link's pose after the integration (the ball has slid v dt further) back to the point the narrowphase found:
    # r = (-v dt, 0, -radius)
    assert wrench[4] == pytest.approx(radius * mu * mass * G + 2.0 * dt * mass * G, rel=2e-2)
    w.close()


def test_link_wrenches_add_up_to_the_generalized_impulse(oracle_py):
    E = 16
    cfg = nk.synthetic.config(2, E)
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    w = stepped(oracle_py, cfg.template, desc, cfg.state())
    R, nl = w.rows_per_env, cfg.template.link_count
    J = w.download("chain_jacobian").reshape(E, R, -1) + w.download("chain_jacobian_b").reshape(E, R, -1)
    generalized = np.einsum("eri,er->ei", J.astype(np.float64), w.download("lambda").reshape(E, R).astype(np.float64))
    wrench = w.download("link_contact_wrench").reshape(E, nl, 6).astype(np.float64)
    total_force = wrench[:, :, :3].sum(1) * cfg.dt
    # the floating base's linear coordinates are expressed in the base frame (DoFs 3..5): rotate the world sum into it.
    # The poses read here are those after the step's integration; the Jacobian was taken before it, one small rotation apart.
    assert np.abs(total_force).max() > 0.0
    base = w.download("base_pose").reshape(E, 7).astype(np.float64)
    qw, qx, qy, qz = base[:, 3], base[:, 4], base[:, 5], base[:, 6]
    rot = np.stack([np.stack([1 - 2 * (qy * qy + qz * qz), 2 * (qx * qy - qw * qz), 2 * (qx * qz + qw * qy)], -1),
                    np.stack([2 * (qx * qy + qw * qz), 1 - 2 * (qx * qx + qz * qz), 2 * (qy * qz - qw * qx)], -1),
                    np.stack([2 * (qx * qz - qw * qy), 2 * (qy * qz + qw * qx), 1 - 2 * (qx * qx + qy * qy)], -1)], 1)
    in_base = np.einsum("eji,ej->ei", rot, total_force)
    assert np.linalg.norm(in_base, axis=1) == pytest.approx(np.linalg.norm(generalized[:, 3:6], axis=1), rel=1e-4, abs=1e-7)
    assert np.abs(in_base - generalized[:, 3:6]).max() <= 2e-2 * np.abs(generalized[:, 3:6]).max()
    # every slot's force components are the sums of its rows' multipliers over dt
    S = cfg.template.max_contacts_per_env
    lam = w.download("lambda").reshape(E, R)
    ranges = w.download("ucontact_row_range").reshape(E, S, 2)
    force = w.download("contact_force").reshape(E, S, 3)
    for e in range(E):
        for s in range(S):
            first, pts = int(ranges[e, s, 0]) - e * R, int(ranges[e, s, 1])
            want = [lam[e, first + k * pts:first + (k + 1) * pts].sum() / cfg.dt for k in range(3)] if pts else [0, 0, 0]
            assert np.allclose(force[e, s], want, rtol=1e-5, atol=1e-6)
    w.close()
