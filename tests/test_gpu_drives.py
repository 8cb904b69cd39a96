"""Parity of the HIP drives and joint rows (ApplyDrives, the limit / friction / drive rows of AssembleRows, the unit
rows of the block-descent solve, ReadoutDrives) with the CPU oracle, through the C ABI on an MI355X.  Bars as in
test_gpu_parity: integer words bit-exact, fp32 norm-wise relative error <= 1e-4."""
import copy

import numpy as np
import pytest

from conftest import nk, relative_error

pytestmark = pytest.mark.gpu
abi = nk.abi
TOL = 1e-4
ROW_WORDS = 26
DRIVE_FIELDS = ("drive_target", "drive_stiffness", "drive_damping", "drive_force_limit", "velocity_target", "joint_f")


def driven_pair(oracle_py, device, index, E, mode, limits=True, friction=0.15, fold=True, pos_iters=0, seed=3):
    """A benchmark configuration with the reference's actuation switched on: drive rows in `mode`, joint ranges
    around the nominal pose (some of the seeded joints start outside them) and dry joint friction."""
    cfg = nk.synthetic.config(index, E)
    t = copy.deepcopy(cfg.template)
    t.drive_rows, t.drive_mode = True, mode
    rng = np.random.default_rng(seed)
    for l, link in enumerate(t.links):
        if link["joint_type"] != abi.JOINT_REVOLUTE:
            continue
        if limits and l % 3 != 0:
            link["lower"], link["upper"] = float(cfg.nominal_q[l]) - 0.2, float(cfg.nominal_q[l]) + 0.25
        if friction and l % 2 == 0:
            link["frictionloss"] = friction
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters, pos_iters=pos_iters, fold_drive_damping=fold)
    oracle = oracle_py.OracleWorld(t, desc, threads=8)
    world = nk.World(device, t, desc)
    state = cfg.state()
    nl = t.link_count
    gains = dict(
        drive_target=(cfg.nominal_q[None, :] + rng.normal(0, 0.2, (E, nl))) if mode == abi.DRIVE_PD_POSITION else rng.normal(0, 8.0, (E, nl)),
        drive_stiffness=rng.uniform(20, 80, (E, nl)), drive_damping=rng.uniform(0.5, 3, (E, nl)),
        drive_force_limit=np.where(rng.uniform(size=(E, nl)) < 0.5, rng.uniform(5, 30, (E, nl)), 0.0),
        velocity_target=rng.normal(0, 0.5, (E, nl)), joint_f=rng.normal(0, 1.0, (E, nl)))
    for w in (oracle, world):
        w.set_state(state)
        for name in DRIVE_FIELDS:
            w.upload(name, gains[name].astype(np.float32))
    return cfg, t, oracle, world


def compare_fields(world, oracle, names, tol=TOL):
    for name in names:
        error = relative_error(world.download(name), oracle.download(name))
        assert error <= tol, f"{name}: relative error {error:.3e}"


@pytest.mark.parametrize("index,E,mode", [(3, 256, abi.DRIVE_PD_POSITION), (2, 256, abi.DRIVE_TORQUE), (3, 128, abi.DRIVE_VELOCITY),
                                          (2, 128, abi.DRIVE_ACTUATOR)])
def test_drive_ops_and_joint_rows_match_the_oracle(oracle_py, device, index, E, mode):
    cfg, t, oracle, world = driven_pair(oracle_py, device, index, E, mode)
    R, nl = world.rows_per_env, t.link_count
    assert R == oracle.rows_per_env == world.info.contact_slots_per_env * 16 + 4 * nl
    if mode == abi.DRIVE_ACTUATOR:
        for w in (oracle, world):
            w.upload("actuator_noload_speed", np.full((E, nl), 6.0, np.float32))
    oracle.op("fk_world_poses"); world.op("FkWorldPoses")
    oracle.op("apply_drives"); world.op("ApplyDrives")
    compare_fields(world, oracle, ("drive_command", "drive_dissipation", "drive_lower", "drive_upper", "tau"), tol=1e-6)
    oracle.op("articulation_dynamics", 1); world.op("ArticulationDynamics")
    compare_fields(world, oracle, ("m", "m_factor", "articulation_bias", "articulation_qdd", "qdot"))
    for name, oname in (("SyncLinkBodyPose", "sync_link_body_pose"), ("BuildAabbs", "build_aabbs"), ("LbvhQueryPairs", "query_pairs"),
                        ("NarrowphasePrimitives", "narrowphase"), ("AssembleRows", "assemble_rows")):
        oracle.op(oname); world.op(name)
    world.synchronize()
    first = world.info.contact_slots_per_env * 16
    grow = world.download("urows").reshape(E, R, ROW_WORDS)[:, first:]
    orow = oracle.download("urows").reshape(E, R, ROW_WORDS)[:, first:]
    gw, ow = grow.view(np.uint32), orow.view(np.uint32)
    assert np.array_equal(gw[:, :, 0], ow[:, :, 0])          # flags of every joint slot
    active = (ow[:, :, 0] & 1) != 0
    assert active.sum() > E * nl                             # limit, friction and drive rows are all present
    for word in (1, 2, 3, 10, 11):
        assert np.array_equal(gw[:, :, word][active], ow[:, :, word][active]), f"joint row word {word}"
    assert relative_error(grow[:, :, 4:8][active], orow[:, :, 4:8][active]) <= 1e-6      # rhs, compliance, bounds
    gj = world.download("chain_jacobian").reshape(E, R, -1)[:, first:]
    oj = oracle.download("chain_jacobian").reshape(E, R, -1)[:, first:]
    assert np.array_equal(gj, oj)                            # +-1 on the joint's coordinate, zeros elsewhere
    assert np.array_equal(world.download("row_count"), oracle.download("row_count"))
    compare_fields(world, oracle, ("lambda", "row_penetration"), tol=1e-6)
    oracle.op("contact_warm_start", 0); world.op("ContactWarmStart")
    oracle.op("block_descent_solve"); world.op("BlockDescentSolve")
    world.synchronize()
    assert np.array_equal(world.download("env_status"), oracle.download("env_status"))
    compare_fields(world, oracle, ("qdot", "link_velocity", "qdot_flat"))
    lam_g, lam_o = world.download("lambda").reshape(E, R), oracle.download("lambda").reshape(E, R)
    assert relative_error(lam_g[:, first:], lam_o[:, first:]) <= TOL        # every joint row acts on its own coordinate
    compare_fields(world, oracle, ("joint_limit_impulse",))
    oracle.op("contact_warm_start", 1); world.op("ContactWarmStart", 1)
    oracle.op("readout_drives"); world.op("ReadoutDrives")
    compare_fields(world, oracle, ("actuator_effort_requested", "actuator_effort", "tau"))
    assert np.array_equal(world.download("actuator_saturated"), oracle.download("actuator_saturated"))
    world.close(); oracle.close()


@pytest.mark.parametrize("index,E,mode,pos_iters,fold", [(3, 256, abi.DRIVE_PD_POSITION, 0, True), (2, 256, abi.DRIVE_PD_POSITION, 0xFFFFFFFF, False),
                                                         (1, 64, abi.DRIVE_PD_POSITION, 0, True)])
def test_driven_steps_match_the_oracle(oracle_py, device, index, E, mode, pos_iters, fold):
    """Whole steps with drives, limits and friction (the chain has no collidables: joint rows alone)."""
    cfg, t, oracle, world = driven_pair(oracle_py, device, index, E, mode, pos_iters=pos_iters, fold=fold)
    steps = 3
    world.step(steps); world.synchronize()
    oracle.step(steps)
    assert np.array_equal(world.download("env_status"), oracle.download("env_status"))
    compare_fields(world, oracle, ("q", "qdot", "link_pose", "base_pose", "actuator_effort", "joint_limit_impulse", "qdot_pseudo"),
                   tol=4e-4 if index == 3 else TOL)   # three steps of the humanoid's indeterminate foot impulses
    world.close(); oracle.close()


def test_pd_drive_closed_form_on_the_gpu(device):
    """One pendulum without gravity: the implicit drive is the implicit-Euler step, computed in float64 here."""
    dt, mass, length, inertia = 1.0 / 200.0, 1.3, 0.4, 0.02
    axis_inertia = inertia + mass * length * length
    t = abi.Template()
    t.add_link(abi.JOINT_FIXED, None, mass=1.0)
    t.add_link(abi.JOINT_REVOLUTE, 0, axis=(0, 1, 0), mass=mass, diag_inertia=(inertia,) * 3, com=(0, 0, -length))
    t.drive_mode, t.drive_rows = abi.DRIVE_PD_POSITION, True
    E = 64
    rng = np.random.default_rng(11)
    q, v = rng.uniform(-1, 1, E).astype(np.float32), rng.normal(0, 2, E).astype(np.float32)
    kp, kd = rng.uniform(5, 80, E).astype(np.float32), rng.uniform(0.1, 2, E).astype(np.float32)
    target, vt = rng.uniform(-1, 1, E).astype(np.float32), rng.normal(0, 1, E).astype(np.float32)
    world = nk.World(device, t, abi.world_desc(E, dt, gravity=(0, 0, 0), vel_iters=8, pos_iters=0xFFFFFFFF))
    pad = lambda x: np.stack([np.zeros_like(x), x], 1)
    world.set_state(dict(q=pad(q), qdot=pad(v), tau=pad(np.zeros(E, np.float32)), base_pose=np.tile(abi.IDENTITY7, (E, 1)),
                         root_twist=np.zeros((E, 6), np.float32)))
    for name, values in (("drive_stiffness", kp), ("drive_damping", kd), ("drive_target", target), ("velocity_target", vt)):
        world.upload(name, pad(values))
    world.step(); world.synchronize()
    got = world.download("qdot").reshape(E, 2)[:, 1]
    q64, v64, kp64, kd64 = (x.astype(np.float64) for x in (q, v, kp, kd))
    D = kd64 + dt * kp64
    want = (axis_inertia * v64 + dt * (kp64 * (target.astype(np.float64) - q64) + D * vt.astype(np.float64))) / (axis_inertia + dt * D)
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    assert not world.download("env_status").any()
    world.close()


def test_invalid_gains_and_modes(device):
    t = abi.Template()
    t.add_link(abi.JOINT_FIXED, None, mass=1.0)
    t.add_link(abi.JOINT_REVOLUTE, 0, axis=(0, 1, 0), mass=1.0)
    t.drive_mode, t.drive_rows = abi.DRIVE_PD_POSITION, True
    world = nk.World(device, t, abi.world_desc(2, 0.005))
    world.upload("drive_stiffness", np.array([[0, 10.0], [0, -1.0]], np.float32))
    world.step(); world.synchronize()
    assert list(world.download("env_status")) == [0, 1 << 10]      # a negative stiffness raises the control failure bit
    world.close()
    t.drive_mode = abi.DRIVE_COMPUTED_TORQUE
    with pytest.raises(nk.NukaError) as err:
        nk.World(device, t, abi.world_desc(2, 0.005))
    assert err.value.code == abi.RESULT_NOT_SUPPORTED
    t.drive_mode, t.drive_rows = abi.DRIVE_TORQUE, False
    t.links[1]["lower"], t.links[1]["upper"] = 1.0, -1.0
    with pytest.raises(nk.NukaError) as err:
        nk.World(device, t, abi.world_desc(2, 0.005))
    assert err.value.code == abi.RESULT_INVALID_ARG


READOUT_F32 = ("contact_point", "contact_normal", "contact_force", "ucontact_impulse", "link_contact_wrench")
READOUT_U32 = ("contact_side_a_kind", "contact_side_b_kind", "contact_side_a_index", "contact_side_b_index", "contact_link")


@pytest.mark.parametrize("index,E", [(2, 256), (3, 256)])
def test_contact_readout_matches_the_oracle_and_joins_the_step_on_demand(oracle_py, device, index, E):
    """ReadoutContactWrench: not part of the step until a consumer asks for one of its fields; the first request runs
    it on the current solution, and from then on every step ends with it (nk/pipeline/world.cpp:905-975)."""
    cfg = nk.synthetic.config(index, E)
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    oracle = oracle_py.OracleWorld(cfg.template, desc, threads=8)
    world = nk.World(device, cfg.template, desc)
    for w in (oracle, world):
        w.set_state(cfg.state())
    ops_before = world.info.op_count
    world.step(); world.synchronize()
    oracle.step(); oracle.op("readout_contact_wrench")
    for name in READOUT_U32:                       # the first download demands the readout
        assert np.array_equal(world.download(name), oracle.download(name)), name
    for name in READOUT_F32[:2]:
        assert relative_error(world.download(name), oracle.download(name)) <= TOL, name
    # the generalized impulse is the well-determined quantity (see test_gpu_parity): per-slot forces of the humanoid's
    # redundant foot spheres inherit the indeterminacy of the individual multipliers, the per-link wrench does not
    assert relative_error(world.download("link_contact_wrench"), oracle.download("link_contact_wrench")) <= (TOL if index == 2 else 5 * TOL)
    if index == 2:
        for name in ("contact_force", "ucontact_impulse"):
            assert relative_error(world.download(name), oracle.download(name)) <= TOL, name
    info = nk.WorldInfoC()
    nk._check(nk.lib().nuka_world_get_info(world._h, __import__("ctypes").byref(info)))
    assert info.op_count == ops_before + 1
    world.step(); world.synchronize()              # now the step itself refreshes the readout
    oracle.step(); oracle.op("readout_contact_wrench")
    assert np.array_equal(world.download("contact_link"), oracle.download("contact_link"))
    assert relative_error(world.download("link_contact_wrench"), oracle.download("link_contact_wrench")) <= 10 * TOL
    world.close(); oracle.close()
