"""Pins of the oracle's articulation dynamics by what the mechanics fixes: closed forms, an independent float64
model built from rotation matrices and finite differences (tests/rigid_model.py), conservation laws."""
import ctypes as C

import numpy as np
import pytest

from conftest import nk
from rigid_model import Model, rot

abi = nk.abi
F = C.c_float
IDENTITY7 = np.array([0, 0, 0, 1, 0, 0, 0], np.float32)


def small_tree(floating, seed=0, prismatic=True):
    """A branching tree with skew axes, offsets, rotated joint frames, offset centres of mass."""
    g = np.random.default_rng(seed)
    t = abi.Template()
    t.add_link(abi.JOINT_FLOATING if floating else abi.JOINT_FIXED, None, mass=2.0, diag_inertia=(0.05, 0.07, 0.04),
               com=(0.01, -0.02, 0.03))
    parents = [0, 1, 1, 0, 4, 5]
    for i, parent in enumerate(parents):
        axis = g.normal(0, 1, 3)
        q = g.normal(0, 1, 4)
        q /= np.linalg.norm(q)
        kind = abi.JOINT_PRISMATIC if (prismatic and i == 2) else abi.JOINT_REVOLUTE
        t.add_link(kind, parent, axis=tuple(axis / np.linalg.norm(axis)), local_pos=tuple(g.normal(0, 0.2, 3)),
                   local_rot=tuple(q), mass=float(g.uniform(0.3, 1.5)), diag_inertia=tuple(g.uniform(0.005, 0.03, 3)),
                   com=tuple(g.normal(0, 0.08, 3)))
    return t


def random_state(t, E, seed, floating):
    g = np.random.default_rng(seed)
    nl = t.link_count
    q = g.uniform(-1.2, 1.2, (E, nl)).astype(np.float32)
    qdot = g.normal(0, 1.0, (E, nl)).astype(np.float32)
    q[:, 0] = qdot[:, 0] = 0
    base = np.tile(IDENTITY7, (E, 1))
    twist = np.zeros((E, 6), np.float32)
    if floating:
        quat = g.normal(0, 1, (E, 4))
        base[:, 3:] = quat / np.linalg.norm(quat, axis=1, keepdims=True)
        base[:, :3] = g.normal(0, 0.5, (E, 3))
        twist = g.normal(0, 0.8, (E, 6)).astype(np.float32)
    return dict(q=q, qdot=qdot, tau=np.zeros((E, nl), np.float32), base_pose=base.astype(np.float32), root_twist=twist)


def generalized_velocity(model, state, e):
    v = [state["qdot"][e, l] for l in model.scalar_links]
    return np.array((list(state["root_twist"][e]) if model.floating else []) + v, np.float64)


def test_spatial_inertia_closed_form(oracle_py):
    L, g = oracle_py.lib(), np.random.default_rng(0)
    for _ in range(100):
        mass, diag, com = float(g.uniform(0.1, 5)), g.uniform(0.01, 0.2, 3), g.normal(0, 0.2, 3)
        q = g.normal(0, 1, 4)
        q /= np.linalg.norm(q)
        out = (F * 36)()
        L.nko_make_spatial_inertia(F(mass), (F * 3)(*diag), (F * 7)(*com, *q), out)
        got = np.array(out).reshape(6, 6)
        cx = np.array([[0, -com[2], com[1]], [com[2], 0, -com[0]], [-com[1], com[0], 0]])
        R = rot(q)
        expect = np.block([[R @ np.diag(diag) @ R.T + mass * cx @ cx.T, mass * cx], [mass * cx.T, mass * np.eye(3)]])
        assert np.abs(got - expect).max() < 2e-6 * max(1.0, np.abs(expect).max())


@pytest.mark.parametrize("index", [1, 2, 3, 5])
def test_world_poses_match_rotation_matrix_kinematics(oracle_py, index):
    E = 4
    cfg = nk.synthetic.config(index, E)
    w = oracle_py.OracleWorld(cfg.template, abi.world_desc(E, cfg.dt))
    state = cfg.state()
    w.set_state(state)
    w.op("fk_world_poses")
    pose = w.download("link_pose").reshape(E, -1, 7)
    model = Model(cfg.template, abi)
    for e in range(E):
        R, p = model.fk(state["q"][e], rot(state["base_pose"][e, 3:]), state["base_pose"][e, :3].astype(np.float64))
        for i in range(model.nl):
            assert np.abs(pose[e, i, :3] - p[i]).max() < 2e-5 * (1 + np.abs(p[i]).max())   # 64-deep chains accumulate
            assert np.abs(rot(pose[e, i, 3:]) - R[i]).max() < 2e-5
    w.close()


def test_pendulum_closed_form(oracle_py):
    t = abi.Template()
    t.add_link(abi.JOINT_FIXED, None)
    mass, l, inertia, damping, armature, stiffness, ref = 1.3, 0.4, 0.02, 0.1, 0.03, 2.0, 0.25
    t.add_link(abi.JOINT_REVOLUTE, 0, axis=(0, 1, 0), mass=mass, diag_inertia=(inertia,) * 3, com=(0, 0, -l),
               damping=damping, armature=armature, stiffness=stiffness, spring_ref=ref)
    E = 4
    w = oracle_py.OracleWorld(t, abi.world_desc(E, 0.002))
    theta = np.array([0.3, -1.0, 2.0, 0.0], np.float32)
    rate = np.array([0.5, -0.2, 1.0, 0.0], np.float32)
    tau = np.array([0.2, 0.0, -1, 3], np.float32)
    zero = np.zeros(E, np.float32)
    w.set_state(dict(q=np.stack([zero, theta], 1), qdot=np.stack([zero, rate], 1), tau=np.stack([zero, tau], 1),
                     base_pose=np.tile(IDENTITY7, (E, 1)), root_twist=np.zeros((E, 6))))
    w.op("fk_world_poses")
    w.op("articulation_dynamics", 0)
    qdd = w.download("qddot").reshape(E, 2)[:, 1]
    # a turn by theta about +y carries the centre of mass to (-l sin, 0, -l cos); gravity torque about y = -m g l sin
    expect = (tau - mass * 9.81 * l * np.sin(theta) - damping * rate - stiffness * (theta - ref)) / (inertia + mass * l * l + armature)
    assert np.abs(qdd - expect).max() < 2e-6 * np.abs(expect).max()
    # integrate_velocity = 1 advances qdot by dt * qdd (semi-implicit Euler)
    w.op("articulation_dynamics", 1)
    assert np.abs(w.download("qdot").reshape(E, 2)[:, 1] - (rate + 0.002 * expect)).max() < 1e-6
    w.close()


@pytest.mark.parametrize("floating", [False, True])
def test_mass_matrix_is_the_kinetic_energy_form(oracle_py, floating):
    t = small_tree(floating, seed=3)
    E = 3
    state = random_state(t, E, 5, floating)
    w = oracle_py.OracleWorld(t, abi.world_desc(E, 0.001))
    w.set_state(state)
    w.op("fk_world_poses")
    w.op("articulation_dynamics", 0)
    n = w.dof
    M = w.download("m").reshape(E, n, n)
    model = Model(t, abi)
    assert n == model.dof
    for e in range(E):
        expect = model.mass_matrix(state["q"][e], rot(state["base_pose"][e, 3:]), state["base_pose"][e, :3].astype(np.float64))
        assert np.abs(M[e] - expect).max() < 5e-6 * np.abs(expect).max()
    w.close()


def test_humanoid_mass_matrix_is_the_kinetic_energy_form(oracle_py):
    cfg = nk.synthetic.config(3, 1)
    state = cfg.state()
    w = oracle_py.OracleWorld(cfg.template, abi.world_desc(1, cfg.dt))
    w.set_state(state)
    w.op("fk_world_poses")
    w.op("articulation_dynamics", 0)
    M = w.download("m").reshape(36, 36)
    model = Model(cfg.template, abi)
    expect = model.mass_matrix(state["q"][0], rot(state["base_pose"][0, 3:]), state["base_pose"][0, :3].astype(np.float64))
    assert np.abs(M - expect).max() < 5e-6 * np.abs(expect).max()
    w.close()


def test_fixed_base_bias_is_the_euler_lagrange_bias(oracle_py):
    t = small_tree(False, seed=7)
    E = 3
    state = random_state(t, E, 8, False)
    w = oracle_py.OracleWorld(t, abi.world_desc(E, 0.001))
    w.set_state(state)
    w.op("fk_world_poses")
    w.op("articulation_dynamics", 0)
    n = w.dof
    bias = w.download("articulation_bias").reshape(E, n)
    qdd = w.download("articulation_qdd").reshape(E, n)
    M = w.download("m").reshape(E, n, n)
    model = Model(t, abi)
    for e in range(E):
        expect = model.lagrange_bias(state["q"][e], state["qdot"][e], (0, 0, -9.81))
        assert np.abs(bias[e] - expect).max() < 2e-5 * np.abs(expect).max()
        # and the acceleration solves M qdd = tau - bias (tau = 0, no damping here)
        assert np.abs(M[e].astype(np.float64) @ qdd[e] + expect).max() < 2e-4 * np.abs(expect).max()
    w.close()


def run_free_flight(oracle_py, t, state, dt, steps, gravity):
    w = oracle_py.OracleWorld(t, abi.world_desc(1, dt, gravity=gravity))
    w.set_state(state)
    w.op("fk_world_poses")
    for _ in range(steps):
        w.op("articulation_dynamics", 1)
        w.op("integrate_position")
        w.op("fk_world_poses")
        w.op("fk_link_velocities")
    nl = t.link_count
    out = dict(q=w.download("q").reshape(1, nl), qdot=w.download("qdot").reshape(1, nl),
               base_pose=w.download("base_pose").reshape(1, 7),
               root_twist=w.download("link_velocity").reshape(1, nl, 6)[:, 0, :])
    w.close()
    return out


def mechanics(model, state, gravity):
    R, p = rot(state["base_pose"][0, 3:]), state["base_pose"][0, :3].astype(np.float64)
    v = generalized_velocity(model, state, 0)
    energy = model.kinetic_energy(state["q"][0], R, p, v) + model.potential(state["q"][0], R, p, gravity)
    return energy, model.momentum(state["q"][0], R, p, v)


@pytest.mark.parametrize("floating", [False, True])
def test_energy_drift_is_first_order_in_dt(oracle_py, floating):
    """Free motion under gravity: semi-implicit Euler keeps the energy to O(dt); a wrong velocity-product or gravity
    term would leave a drift that does not shrink with dt."""
    t = small_tree(floating, seed=11)
    state = random_state(t, 1, 12, floating)
    model = Model(t, abi)
    gravity = (0.0, 0.0, -9.81)
    e0, _ = mechanics(model, state, gravity)
    kinetic = model.kinetic_energy(state["q"][0], rot(state["base_pose"][0, 3:]), state["base_pose"][0, :3].astype(np.float64),
                                   generalized_velocity(model, state, 0))
    horizon = 0.05
    drift = []
    for dt in (1e-3, 5e-4, 2.5e-4):
        end = run_free_flight(oracle_py, t, state, dt, int(round(horizon / dt)), gravity)
        drift.append(abs(mechanics(model, end, gravity)[0] - e0))
    assert drift[0] < 0.02 * kinetic
    assert 1.5 < drift[0] / drift[1] < 2.7 and 1.5 < drift[1] / drift[2] < 2.7


def test_free_floating_momentum(oracle_py):
    """Floating tree with internal motion: linear momentum gains m g t, and with gravity off the angular momentum
    about the origin stays put, both to O(dt)."""
    t = small_tree(True, seed=13)
    state = random_state(t, 1, 14, True)
    model = Model(t, abi)
    total_mass = sum(l["mass"] for l in t.links)
    dt, steps = 2.5e-4, 200
    for gravity in ((0.0, 0.0, -9.81), (0.0, 0.0, 0.0)):
        _, (p0, l0) = mechanics(model, state, gravity)
        _, (p1, l1) = mechanics(model, run_free_flight(oracle_py, t, state, dt, steps, gravity), gravity)
        assert np.abs(p1 - p0 - total_mass * np.asarray(gravity) * dt * steps).max() < 2e-3 * max(np.abs(p0).max(), 1.0)
        if gravity[2] == 0.0:
            assert np.abs(l1 - l0).max() < 2e-3 * max(np.abs(l0).max(), 1.0)


def test_factorisation_reconstructs_and_solves(oracle_py):
    L, g = oracle_py.lib(), np.random.default_rng(21)
    for n in (1, 7, 18, 36, 64):
        A = g.normal(0, 1, (n, n))
        M = (A @ A.T + n * np.eye(n)).astype(np.float32)
        factor = np.zeros((n, n), np.float32)
        L.nko_factor_mass(M.ctypes.data_as(C.c_void_p), factor.ctypes.data_as(C.c_void_p), n, n)
        unit_lower = np.tril(factor, -1).astype(np.float64) + np.eye(n)
        rebuilt = unit_lower @ np.diag(np.diag(factor).astype(np.float64)) @ unit_lower.T
        assert np.abs(rebuilt - M).max() < 2e-6 * np.abs(M).max()
        b = g.normal(0, 1, n).astype(np.float32)
        x = b.copy()
        L.nko_solve_mass(factor.ctypes.data_as(C.c_void_p), x.ctypes.data_as(C.c_void_p), n, n)
        assert np.abs(x - np.linalg.solve(M.astype(np.float64), b)).max() < 1e-5 * np.abs(x).max()
        # J M^-1 J^T for one row against the dense solve
        v = g.normal(0, 1, n).astype(np.float32)
        coupling = L.nko_mass_coupling(factor.ctypes.data_as(C.c_void_p), n, v.ctypes.data_as(C.c_void_p), None)
        assert abs(coupling - v @ np.linalg.solve(M.astype(np.float64), v)) < 1e-5 * coupling


def test_link_velocities_are_the_pose_rates(oracle_py):
    """Body-frame link twists against central differences of the float64 kinematics."""
    t = small_tree(True, seed=17)
    state = random_state(t, 1, 18, True)
    w = oracle_py.OracleWorld(t, abi.world_desc(1, 0.001))
    w.set_state(state)
    w.op("fk_world_poses")
    w.op("fk_link_velocities")
    twists = w.download("link_velocity").reshape(-1, 6)
    model = Model(t, abi)
    R0, p0 = rot(state["base_pose"][0, 3:]), state["base_pose"][0, :3].astype(np.float64)
    R, _ = model.fk(state["q"][0], R0, p0)
    zero_com = [dict(l, inertial=[0, 0, 0, 1, 0, 0, 0]) for l in t.links]
    origin_model = Model(t, abi)
    origin_model.links = zero_com
    for i, (omega, v) in enumerate(origin_model.link_motion(state["q"][0], R0, p0, generalized_velocity(model, state, 0))):
        assert np.abs(twists[i, :3] - R[i].T @ omega).max() < 5e-6 * (1 + np.abs(omega).max())
        assert np.abs(twists[i, 3:] - R[i].T @ v).max() < 5e-6 * (1 + np.abs(v).max())
    w.close()
