"""Pins of the oracle's drives and joint rows (ApplyDrives, the limit / friction / drive rows of AssembleRows,
ReadoutDrives) against closed forms of a one-joint pendulum without gravity, and against the direct-torque path on
a seven-joint chain.  A pendulum of inertia I about its axis makes every row a scalar equation, so each expected
value below is the textbook implicit-Euler or impulse formula, not a restatement of the code under test."""
import numpy as np
import pytest

from conftest import nk

abi = nk.abi
DT = 1.0 / 200.0
ROW_WORDS = 26
IDENTITY7 = np.array([0, 0, 0, 1, 0, 0, 0], np.float32)
MASS, LENGTH, INERTIA = 1.3, 0.4, 0.02
I_AXIS = INERTIA + MASS * LENGTH * LENGTH   # about the joint axis (parallel-axis theorem)


def pendulum(mode=abi.DRIVE_TORQUE, drive_rows=True, lower=None, upper=None, frictionloss=0.0):
    t = abi.Template()
    t.add_link(abi.JOINT_FIXED, None, mass=1.0)
    t.add_link(abi.JOINT_REVOLUTE, 0, axis=(0, 1, 0), mass=MASS, diag_inertia=(INERTIA,) * 3, com=(0, 0, -LENGTH),
               lower=lower, upper=upper, frictionloss=frictionloss)
    t.drive_mode, t.drive_rows = mode, drive_rows
    return t


def world(oracle_py, template, E, pos_iters=0xFFFFFFFF, fold=True, gravity=(0.0, 0.0, 0.0)):
    desc = abi.world_desc(E, DT, gravity=gravity, vel_iters=8, pos_iters=pos_iters, fold_drive_damping=fold)
    return oracle_py.OracleWorld(template, desc, threads=2)


def joint(values):
    """[E] values of the pendulum joint as an [E, 2] per-link array (link 0 is the fixed root)."""
    values = np.asarray(values, np.float32)
    return np.stack([np.zeros_like(values), values], 1)


def set_state(w, q, qdot, tau=None):
    E = len(q)
    z = np.zeros(E, np.float32)
    w.set_state(dict(q=joint(q), qdot=joint(qdot), tau=joint(z if tau is None else tau), base_pose=np.tile(IDENTITY7, (E, 1)),
                     root_twist=np.zeros((E, 6), np.float32)))


def test_mass_of_the_pendulum_is_its_axis_inertia(oracle_py):
    w = world(oracle_py, pendulum(drive_rows=False), 1)
    set_state(w, [0.3], [0.0])
    w.op("fk_world_poses")
    w.op("articulation_dynamics", 0)
    assert w.download("m")[0] == pytest.approx(I_AXIS, rel=1e-6)


@pytest.mark.parametrize("fold", [True, False])
def test_pd_drive_is_the_implicit_euler_step(oracle_py, fold):
    rng = np.random.default_rng(5)
    E = 16
    q, v = rng.uniform(-1, 1, E), rng.normal(0, 2, E)
    kp, kd = rng.uniform(5, 80, E), rng.uniform(0.1, 2, E)
    target, vt = rng.uniform(-1, 1, E), rng.normal(0, 1, E)
    w = world(oracle_py, pendulum(abi.DRIVE_PD_POSITION), E, fold=fold)
    set_state(w, q, v)
    for name, values in (("drive_stiffness", kp), ("drive_damping", kd), ("drive_target", target), ("velocity_target", vt)):
        w.upload(name, joint(values))
    w.step()
    got = w.download("qdot").reshape(E, 2)[:, 1]
    q32, v32 = q.astype(np.float32).astype(np.float64), v.astype(np.float32).astype(np.float64)
    if fold:   # I (v' - v)/dt = kp (target - q) + D (vt - v'), D = kd + dt kp
        D = kd + DT * kp
        want = (I_AXIS * v32 + DT * (kp * (target - q32) + D * vt)) / (I_AXIS + DT * D)
    else:      # the explicit step: the effort is evaluated at the step start
        want = v32 + DT * (kp * (target - q32) + kd * (vt - v32)) / I_AXIS
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    assert not w.download("env_status").any()
    # ReadoutDrives: the applied effort is the impulse over dt less the dissipation at the new velocity
    applied = w.download("actuator_effort").reshape(E, 2)[:, 1]
    D = (kd + DT * kp) if fold else 0.0 * kd
    command = kp * (target - q32) + (D * vt if fold else kd * (vt - v32))
    assert np.abs(applied - (command - D * got)).max() <= 1e-4 * np.abs(command).max()
    assert np.array_equal(w.download("tau").reshape(E, 2)[:, 1], applied)   # joint_f is zero


def test_force_limit_clamps_the_effort(oracle_py):
    E = 4
    q, v = np.zeros(E), np.zeros(E)
    kp, target, limit = np.full(E, 100.0), np.array([1.0, -1.0, 0.01, 0.5]), np.full(E, 3.0)
    w = world(oracle_py, pendulum(abi.DRIVE_PD_POSITION), E)
    set_state(w, q, v)
    w.upload("drive_stiffness", joint(kp)); w.upload("drive_target", joint(target)); w.upload("drive_force_limit", joint(limit))
    w.step()
    got = w.download("qdot").reshape(E, 2)[:, 1]
    effort = kp * target
    saturated = np.abs(effort) > limit
    # a saturated drive applies its clamped effort without the implicit derivative; the others step implicitly
    want = np.where(saturated, DT * np.clip(effort, -limit, limit) / I_AXIS, DT * effort / (I_AXIS + DT * DT * kp))
    assert np.allclose(got, want, rtol=2e-5)
    assert np.array_equal(w.download("actuator_saturated").reshape(E, 2)[:, 1], saturated.astype(np.float32))


def test_torque_drive_rows_match_the_direct_torque_path(oracle_py):
    cfg = nk.synthetic.config(1, 32)
    state = cfg.state()
    direct = oracle_py.OracleWorld(cfg.template, abi.world_desc(32, cfg.dt, vel_iters=8), threads=2)
    direct.set_state(state)
    direct.step()
    import copy
    t = copy.deepcopy(cfg.template)
    t.drive_rows, t.drive_mode = True, abi.DRIVE_TORQUE
    driven = oracle_py.OracleWorld(t, abi.world_desc(32, cfg.dt, vel_iters=8), threads=2)
    driven.set_state(state)
    driven.upload("drive_target", state["tau"])
    driven.step()
    assert driven.rows_per_env == t.link_count and direct.rows_per_env == 0
    a, b = driven.download("qdot"), direct.download("qdot")
    assert np.abs(a - b).max() <= 2e-5 * np.abs(b).max()
    assert np.abs(driven.download("q") - direct.download("q")).max() <= 1e-6
    # the applied effort read back is the commanded torque
    assert np.allclose(driven.download("actuator_effort"), state["tau"].reshape(-1), rtol=1e-5, atol=1e-6)


def test_joint_limit_stops_at_the_bound(oracle_py):
    # no position pass: the limit row removes the whole violation in one step, q' = bound, when the free motion
    # would cross it; a joint moving away, or far from the bound, feels nothing
    lower, upper = -0.5, 0.7
    q = np.array([-0.49, -0.45, 0.69, 0.1, -0.52], np.float64)
    v = np.array([-8.0, 3.0, 5.0, 1.0, 0.0], np.float64)
    w = world(oracle_py, pendulum(drive_rows=False, lower=lower, upper=upper), len(q))
    set_state(w, q, v)
    w.step()
    got_q = w.download("q").reshape(-1, 2)[:, 1]
    got_v = w.download("qdot").reshape(-1, 2)[:, 1]
    want_q = np.array([lower, -0.45 + 3.0 * DT, upper, 0.1 + 1.0 * DT, lower])
    assert np.allclose(got_q, want_q, atol=2e-6)
    impulse = w.download("joint_limit_impulse").reshape(-1, 2, 2)[:, 1, :]
    q32, v32 = q.astype(np.float32).astype(np.float64), v.astype(np.float32).astype(np.float64)
    want_lower = np.where(want_q == lower, I_AXIS * ((lower - q32) / DT - v32), 0.0)
    want_upper = np.where(want_q == upper, -I_AXIS * ((upper - q32) / DT - v32), 0.0)
    assert np.allclose(impulse[:, 0], want_lower, rtol=1e-4, atol=1e-7)
    assert np.allclose(impulse[:, 1], want_upper, rtol=1e-4, atol=1e-7)
    assert (impulse >= 0.0).all()
    assert np.allclose(got_v, (got_q - q32) / DT, rtol=1e-4, atol=1e-4)


def test_joint_limit_with_position_pass_splits_velocity_and_push(oracle_py):
    # with the position pass the velocity row only stops further violation; the pass pushes the joint back by
    # beta (violation - slop) through the pseudo velocity and leaves the real velocity at rest
    lower = -0.5
    q, v = np.array([-0.56]), np.array([-1.0])
    w = world(oracle_py, pendulum(drive_rows=False, lower=lower), 1, pos_iters=4)
    set_state(w, q, v)
    w.step()
    assert w.download("qdot").reshape(-1, 2)[0, 1] == pytest.approx(0.0, abs=1e-6)
    violation = lower - float(np.float32(q[0]))
    # one augmented-Lagrangian solve from a zero multiplier with the penalty at its cap rho = 100 / (J M^-1 J^T)
    # reaches rho / (M + rho) = 100/101 of the bias
    push = 0.3 * (violation - 1e-3) * 100.0 / 101.0
    assert w.download("q").reshape(-1, 2)[0, 1] == pytest.approx(float(np.float32(q[0])) + push, abs=2e-6)


def test_dry_friction_holds_then_slips(oracle_py):
    friction = 0.8
    tau = np.array([0.5, -0.79, 1.3, -2.0])
    w = world(oracle_py, pendulum(drive_rows=False, frictionloss=friction), len(tau))
    set_state(w, np.zeros(len(tau)), np.zeros(len(tau)), tau)
    w.step()
    got = w.download("qdot").reshape(-1, 2)[:, 1]
    want = np.where(np.abs(tau) <= friction, 0.0, DT * (tau - np.sign(tau) * friction) / I_AXIS)
    assert np.allclose(got, want, rtol=2e-5, atol=1e-5)   # the solve stops at a velocity residual of 1e-5


def test_row_slots_follow_the_contact_rows(oracle_py):
    t = pendulum(abi.DRIVE_TORQUE, True, lower=-1.0, frictionloss=0.1)
    w = world(oracle_py, t, 2)
    assert w.rows_per_env == 2 * 2 + 2 + 2   # limit pairs, friction and drive slots of two links, no contact slots
    set_state(w, [0.0, -0.999], [0.0, -1.0])
    w.upload("drive_target", joint([0.25, 0.0]))
    w.op("fk_world_poses"); w.op("apply_drives"); w.op("articulation_dynamics", 1); w.op("assemble_rows")
    rows = w.download("urows").reshape(2, w.rows_per_env, ROW_WORDS).view(np.uint32)
    flags = rows[:, :, 0]
    J = w.download("chain_jacobian").reshape(2, w.rows_per_env, -1)
    lower_row, friction_row, drive_row = 2, 4 + 1, 6 + 1
    assert flags[0, lower_row] == flags[1, lower_row] == (1 | 1 << 4)              # an authored bound always has its row
    assert flags[0, lower_row + 1] == 0                                             # no upper bound authored
    assert flags[0, friction_row] == flags[1, friction_row] == (1 | 1 << 7)
    assert flags[0, drive_row] == (1 | 1 << 7) and flags[1, drive_row] == 0         # a zero command emits no row
    assert J[1, lower_row, 0] == 1.0 and J[0, friction_row, 0] == 1.0 and J[0, drive_row, 0] == 1.0
    assert w.download("lambda").reshape(2, -1)[0, drive_row] == pytest.approx(0.25 * DT)
    assert list(w.download("row_count")) == [3, 2]


def test_invalid_gains_raise_the_control_status(oracle_py):
    w = world(oracle_py, pendulum(abi.DRIVE_PD_POSITION), 2)
    set_state(w, [0.0, 0.0], [0.0, 0.0])
    w.upload("drive_stiffness", joint([10.0, -1.0]))
    w.op("apply_drives")
    assert list(w.download("env_status")) == [0, 1 << 10]
