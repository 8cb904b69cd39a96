"""The MuJoCo contact law on the device against the CPU oracle: reference weights at creation, compliant and pyramid
rows, the elliptic cone in the block descent, and whole steps; then the rest depth of the spring reference at scale.

Bars: flags, counts, ranges and status words bit-exact; fp32 fields per environment to TOL (norm-wise relative error).
The compliant rows go through powf, which the device and the host evaluate with different last-place rounding, so the
rows are held to TOL and not to the bit."""
import ctypes as C

import numpy as np
import pytest

from conftest import nk, per_env_error

pytestmark = pytest.mark.gpu
abi = nk.abi
TOL = 1e-4
ROW_WORDS = 26
F = C.c_float
CONES = {"elliptic": abi.CONE_ELLIPTIC, "pyramidal": abi.CONE_PYRAMIDAL}
ORACLE_OPS = {"SnapshotStepVelocity": ("snapshot_step_velocity",), "FkWorldPoses": ("fk_world_poses",),
              "ArticulationDynamics": ("articulation_dynamics", 1), "SyncLinkBodyPose": ("sync_link_body_pose",),
              "BuildAabbs": ("build_aabbs",), "LbvhQueryPairs": ("query_pairs",), "NarrowphasePrimitives": ("narrowphase",),
              "AssembleRows": ("assemble_rows",), "BlockDescentSolve": ("block_descent_solve",)}
UPSTREAM = ["SnapshotStepVelocity", "FkWorldPoses", "ArticulationDynamics", "SyncLinkBodyPose", "BuildAabbs", "LbvhQueryPairs",
            "NarrowphasePrimitives", "AssembleRows"]


def mujoco_pair(oracle_py, device, index, E, cone, lower=0.0, **profile):
    cfg = nk.synthetic.config(index, E)
    for p in cfg.template.profiles:
        p.update(law=abi.LAW_MUJOCO, **profile)
    cfg.template.contact_cone = cone
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    oracle = oracle_py.OracleWorld(cfg.template, desc, threads=8)
    world = nk.World(device, cfg.template, desc)
    state = cfg.state()
    state["base_pose"][:, 2] -= lower
    oracle.set_state(state)
    world.set_state(state)
    return cfg, oracle, world, state


def close(world, oracle, name, tol=TOL, floor=1e-6):
    E = world.env_count
    got, expect = world.download(name), oracle.download(name)
    errors = per_env_error(got, expect, E, floor)
    worst = float(errors.max()) if errors.size else 0.0
    assert worst <= tol, f"{name}: {int((errors > tol).sum())} of {E} environments above {tol:.1e}, worst {worst:.3e}"


@pytest.mark.parametrize("index", [2, 3])
def test_reference_weights_at_creation(oracle_py, device, index):
    """ReferenceWeights (articulation.cu:425-500), dispatched at creation at the rest pose."""
    E = 8
    cfg, oracle, world, _ = mujoco_pair(oracle_py, device, index, E, abi.CONE_ELLIPTIC)
    world.synchronize()
    for name in ("body_invweight0", "dof_invweight0"):
        assert np.abs(oracle.download(name)).max() > 0.0
        close(world, oracle, name, floor=1e-12)
    # and at another pose, dispatched again
    for side in (oracle, world):
        (side.op("fk_world_poses") if side is oracle else side.op("FkWorldPoses"))
        (side.op("reference_weights") if side is oracle else side.op("ReferenceWeights"))
    world.synchronize()
    for name in ("body_invweight0", "dof_invweight0"):
        close(world, oracle, name, floor=1e-12)
    oracle.close(); world.close()


@pytest.mark.parametrize("cone", list(CONES))
@pytest.mark.parametrize("index", [2, 3])
def test_rows_of_the_mujoco_law(oracle_py, device, index, cone):
    """Narrowphase law and depth, then AssembleRows: flags and layout to the bit, the compliant terms to TOL."""
    E = 32
    cfg, oracle, world, state = mujoco_pair(oracle_py, device, index, E, CONES[cone], lower=0.12 if index == 2 else 0.05,
                                            solref=(0.03, 0.9), solimp=(0.85, 0.97, 0.002, 0.4, 2.0), margin=(0.004, 0.001))
    rng = np.random.default_rng(11)
    qdot = rng.normal(0.0, 0.5, state["qdot"].shape).astype(np.float32)
    oracle.upload("qdot", qdot); world.upload("qdot", qdot)
    for name in UPSTREAM:
        oracle.op(*ORACLE_OPS[name])
        world.op(name)
    world.synchronize()
    R = world.rows_per_env
    assert np.array_equal(world.download("ucontact_law"), oracle.download("ucontact_law"))
    assert np.array_equal(world.download("ucontact_count"), oracle.download("ucontact_count"))
    assert (oracle.download("ucontact_law")[oracle.download("ucontact_count") > 0] == 0).all()
    assert np.array_equal(world.download("ucontact_row_range"), oracle.download("ucontact_row_range"))
    assert np.array_equal(world.download("contact_material"), oracle.download("contact_material"))
    close(world, oracle, "ucontact_depth")
    close(world, oracle, "step_qdot_flat")
    got = world.download("urows").view(np.uint32).reshape(E, R, ROW_WORDS)
    expect = oracle.download("urows").view(np.uint32).reshape(E, R, ROW_WORDS)
    integer_words = [0, 1, 2, 3, 10, 11, 18, 19]
    assert np.array_equal(got[:, :, integer_words], expect[:, :, integer_words])
    active = (expect[:, :, 0] & 1) != 0
    assert active.sum() >= E
    mujoco_rows = (expect[:, :, 0] & (1 << 11)) != 0
    assert (mujoco_rows[:, :cfg.template.max_contacts_per_env * 16] == active[:, :cfg.template.max_contacts_per_env * 16]).all()
    if cone == "pyramidal":
        assert ((expect[:, :, 0] & (1 << 12)) != 0)[active].all()
    gotf, expectf = got.view(np.float32), expect.view(np.float32)
    for word in (4, 5, 6, 8, 9, 12, 13, 14, 20, 21, 22):   # rhs, compliance, lower, mu, mu2, both directions
        a, b = np.where(active, gotf[:, :, word], 0.0), np.where(active, expectf[:, :, word], 0.0)
        errors = per_env_error(a, b, E)
        assert errors.max() <= TOL, (word, float(errors.max()))
    for name in ("row_invweight", "row_reference_velocity_gain"):
        a = np.where(active, world.download(name).reshape(E, R), 0.0)
        b = np.where(active, oracle.download(name).reshape(E, R), 0.0)
        assert per_env_error(a, b, E).max() <= TOL, name
    for name in ("chain_jacobian", "chain_jacobian_b"):
        md = world.download(name).size // (E * R)
        a = np.where(active[:, :, None], world.download(name).reshape(E, R, md), 0.0)
        b = np.where(active[:, :, None], oracle.download(name).reshape(E, R, md), 0.0)
        assert per_env_error(a, b, E).max() <= TOL, name
    oracle.close(); world.close()


@pytest.mark.parametrize("cone", list(CONES))
@pytest.mark.parametrize("index", [2, 3])
def test_solve_of_the_mujoco_law_from_the_oracles_rows(oracle_py, device, index, cone):
    """The block descent alone: the device solves the rows the oracle assembled (every input of the solve uploaded
    from the oracle), so the comparison holds the elliptic cone and the compliant scalar heads to the oracle's own
    arithmetic."""
    E = 32
    cfg, oracle, world, state = mujoco_pair(oracle_py, device, index, E, CONES[cone], lower=0.12 if index == 2 else 0.05)
    for name in UPSTREAM:
        oracle.op(*ORACLE_OPS[name])
        world.op(name)
    world.synchronize()
    for name in ("urows", "lambda", "chain_jacobian", "chain_jacobian_b", "m", "m_factor", "qdot", "link_velocity", "row_penetration",
                 "contact_row_extent", "ucontact_row_range", "ucontact_count", "ucontact_depth", "row_cj_link", "row_cj_link_b"):
        world.upload(name, oracle.download(name))
    oracle.op("block_descent_solve")
    world.op("BlockDescentSolve")
    world.synchronize()
    assert np.array_equal(world.download("env_status"), oracle.download("env_status"))
    assert (oracle.download("env_status") == 0).all()
    # the sweep counts agree except where the oracle's own last residual sits within a factor of three of the tolerance,
    # where the last bit decides whether one more sweep runs (either result meets TOL below)
    sweeps = oracle.download("vbd_velocity_sweep_count")
    residual = oracle.download("solver_residual").reshape(E, 4).max(1)
    settled = (residual < 1e-5 / 3.0) | (residual > 3e-5)
    assert np.array_equal(world.download("vbd_velocity_sweep_count")[settled], sweeps[settled])
    assert np.abs(world.download("vbd_velocity_sweep_count").astype(np.int64) - sweeps).max() <= 1
    assert np.abs(oracle.download("lambda")).max() > 0.0
    close(world, oracle, "qdot_flat")
    R = world.rows_per_env
    J = oracle.download("chain_jacobian").reshape(E, R, -1).astype(np.float64) + oracle.download("chain_jacobian_b").reshape(E, R, -1)
    impulse = lambda w: np.einsum("eri,er->ei", J, w.download("lambda").reshape(E, R).astype(np.float64))
    assert per_env_error(impulse(world), impulse(oracle), E).max() <= TOL
    oracle.close(); world.close()


@pytest.mark.parametrize("cone", list(CONES))
@pytest.mark.parametrize("index", [2, 3])
def test_steps_of_the_mujoco_law(oracle_py, device, index, cone):
    E, steps = 32, 6
    cfg, oracle, world, _ = mujoco_pair(oracle_py, device, index, E, CONES[cone], lower=0.1 if index == 2 else 0.03)
    oracle.step(steps)
    world.step(steps)
    world.synchronize()
    assert np.array_equal(world.download("env_status"), oracle.download("env_status"))
    assert (oracle.download("env_status") == 0).all()
    assert oracle.download("contact_count").sum() > 0
    for name in ("q", "qdot", "base_pose", "link_velocity"):
        close(world, oracle, name, tol=5e-4)
    oracle.close(); world.close()


@pytest.mark.parametrize("cone", list(CONES))
def test_resting_spheres_sink_to_the_depth_of_the_spring_reference(oracle_py, device, cone):
    """At rest the row equation a + R f = aref holds with a = 0 and f the weight: f = aref / R with aref = k imp depth
    and R = invweight (1 - imp) / imp, which fixes the depth (a pyramid's four edges carry a quarter each, at the edge
    weight).  4096 environments, none may differ."""
    E, dt, mass, g, mu = 4096, 0.002, 3.0, 9.81, 0.9
    solref, solimp = (0.02, 1.0), (0.9, 0.95, 0.001, 0.5, 2.0)
    t = abi.Template()
    t.add_link(abi.JOINT_FLOATING, None, mass=mass, diag_inertia=(0.02, 0.02, 0.02))
    profile = t.add_profile(mu, law=abi.LAW_MUJOCO, solref=solref, solimp=solimp)
    t.add_body(abi.ROLE_STATIC, kind=abi.SHAPE_PLANE, profile=profile)
    t.add_body(abi.ROLE_LINK_BODY, link=0, kind=abi.SHAPE_SPHERE, params=(0.1, 0, 0, 0), profile=profile)
    t.contact_cone = CONES[cone]
    world = nk.World(device, t, abi.world_desc(E, dt, vel_iters=16, velocity_tolerance=1e-7))
    base = np.tile(np.array([0, 0, 0.0999, 1, 0, 0, 0], np.float32), (E, 1))
    base[:, 2] += np.linspace(0.0, 0.002, E, dtype=np.float32)   # dropped from slightly different heights
    world.upload("base_pose", base)
    world.step(2000)
    world.synchronize()
    assert (world.download("env_status") == 0).all()
    depth = 0.1 - world.download("base_pose").reshape(E, 7)[:, 2]
    assert np.abs(world.download("link_velocity").reshape(E, 6)[:, 5]).max() < 1e-4
    invweight = 1.0 / mass
    if cone == "pyramidal":
        invweight = (invweight + mu * mu * invweight) * 2.0 * mu * mu
    force = mass * g if cone == "elliptic" else mass * g / 4.0
    L = oracle_py.lib()
    lo, hi = 0.0, 0.01
    for _ in range(60):
        mid = 0.5 * (lo + hi)
        terms = (F * 6)()
        L.nko_compliant_row_terms((F * 2)(*solref), (F * 5)(*solimp), F(-mid), F(-mid), F(0.0), F(invweight), F(dt), 1, terms)
        lo, hi = (mid, hi) if terms[5] / terms[4] < force else (lo, mid)
    assert np.abs(depth / (0.5 * (lo + hi)) - 1.0).max() < 0.03
    world.close()


@pytest.mark.parametrize("law", [abi.LAW_NATIVE, abi.LAW_MUJOCO])
def test_priority_solmix_and_frictionless_profiles(oracle_py, device, law):
    """The merge's other branches on the device: the plane and the feet carry different profiles - a higher priority on
    one side, unequal solmix on equal priority, a direct-form solref, condim 1 - and every merged outcome (material key,
    row flags and terms, the steps that follow) matches the oracle."""
    E = 16
    variants = [dict(priority=2), dict(solmix=3.0, solref=(0.05, 0.7)), dict(solref=(-400.0, -30.0)), dict(condim=1), dict(priority=1, condim=1)]
    for variant in variants:
        cfg = nk.synthetic.config(2, E)
        t = cfg.template
        feet = dict(t.profiles[0])
        feet.update(law=law, mu=(0.5, 0.5), solref=(0.03, 1.1), solimp=(0.8, 0.9, 0.002, 0.5, 2.0), margin=(0.002, 0.0))
        feet.update(variant)
        t.profiles[0].update(law=law, mu=(0.9, 0.9))
        t.profiles.append(feet)
        for body in t.bodies:
            if body["kind"] == abi.SHAPE_SPHERE:
                body["profile"] = 1
        t.contact_cone = abi.CONE_ELLIPTIC
        desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
        oracle = oracle_py.OracleWorld(t, desc, threads=8)
        world = nk.World(device, t, desc)
        state = cfg.state()
        state["base_pose"][:, 2] -= 0.12
        oracle.set_state(state); world.set_state(state)
        for name in UPSTREAM:
            oracle.op(*ORACLE_OPS[name])
            world.op(name)
        world.synchronize()
        R = world.rows_per_env
        assert np.array_equal(world.download("contact_material"), oracle.download("contact_material")), variant
        got = world.download("urows").view(np.uint32).reshape(E, R, ROW_WORDS)
        expect = oracle.download("urows").view(np.uint32).reshape(E, R, ROW_WORDS)
        assert np.array_equal(got[:, :, [0, 1, 2, 3, 10, 11, 18, 19]], expect[:, :, [0, 1, 2, 3, 10, 11, 18, 19]]), variant
        active = (expect[:, :, 0] & 1) != 0
        assert active.sum() >= E
        # condim 1 prevails only from the side of higher priority; at equal priority the larger condim does
        frictionless = variant.get("condim") == 1 and variant.get("priority", 0) > 0
        assert (((expect[:, :, 0] & ((1 << 2) | (1 << 3)))[active] == 0).all()) == frictionless
        for word in (4, 5, 8, 9):
            a = np.where(active, got.view(np.float32)[:, :, word], 0.0)
            b = np.where(active, expect.view(np.float32)[:, :, word], 0.0)
            assert per_env_error(a, b, E).max() <= TOL, (variant, word)
        oracle.step(4); world.step(4); world.synchronize()
        assert np.array_equal(world.download("env_status"), oracle.download("env_status")) and (oracle.download("env_status") == 0).all()
        for name in ("q", "qdot", "link_velocity"):
            close(world, oracle, name, tol=5e-4)
        oracle.close(); world.close()


def mujoco_joint_pair(oracle_py, device, index, E, integrator, mode=abi.DRIVE_PD_POSITION, seed=5):
    """A benchmark configuration as an imported MJCF would have it: every joint MuJoCo-sourced with ranges around the
    nominal pose (some seeded joints start beyond them), dry friction, passive damping, servos, and the MuJoCo
    integrator."""
    import copy
    cfg = nk.synthetic.config(index, E)
    t = copy.deepcopy(cfg.template)
    t.drive_rows, t.drive_mode, t.integrator = True, mode, integrator
    for p in t.profiles:
        p.update(law=abi.LAW_MUJOCO)
    t.contact_cone = abi.CONE_ELLIPTIC
    rng = np.random.default_rng(seed)
    for l, link in enumerate(t.links):
        if link["joint_type"] != abi.JOINT_REVOLUTE:
            continue
        link["law"] = abi.LAW_MUJOCO
        link["damping"] = 0.3 + 0.05 * (l % 4)
        if l % 3 != 0:
            link["lower"], link["upper"] = float(cfg.nominal_q[l]) - 0.2, float(cfg.nominal_q[l]) + 0.25
            link["limit_margin"] = 0.01 * (l % 2)
            link["limit_reference"] = (0.02 + 0.005 * (l % 3), 1.0, 0.9, 0.95, 0.001, 0.5, 2.0)
        if l % 2 == 0:
            link["frictionloss"] = 0.15
            link["friction_reference"] = (0.01, 1.0, 0.85, 0.95, 0.001, 0.5, 2.0)
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    oracle = oracle_py.OracleWorld(t, desc, threads=8)
    world = nk.World(device, t, desc)
    state = cfg.state()
    state["base_pose"][:, 2] -= 0.1 if index == 2 else 0.03
    nl = t.link_count
    gains = dict(drive_target=cfg.nominal_q[None, :] + rng.normal(0, 0.2, (E, nl)), drive_stiffness=rng.uniform(20, 80, (E, nl)),
                 drive_damping=rng.uniform(0.5, 3, (E, nl)), drive_force_limit=np.where(rng.uniform(size=(E, nl)) < 0.5, rng.uniform(5, 30, (E, nl)), 0.0),
                 velocity_target=rng.normal(0, 0.5, (E, nl)))
    for w in (oracle, world):
        w.set_state(state)
        for name, values in gains.items():
            w.upload(name, values.astype(np.float32))
    return cfg, t, oracle, world


@pytest.mark.parametrize("index,integrator", [(2, abi.INTEGRATOR_MUJOCO_EULER), (3, abi.INTEGRATOR_MUJOCO_EULER), (3, abi.INTEGRATOR_MUJOCO_IMPLICIT)])
def test_mujoco_joint_rows_and_integrator(oracle_py, device, index, integrator):
    """Compliant limit and dry-friction rows (assemble_rows.cu:860-877, 921-931) and ArticulationDamping
    (articulation.cu:950-1000), op by op and then over whole steps."""
    E = 64
    cfg, t, oracle, world = mujoco_joint_pair(oracle_py, device, index, E, integrator)
    R = world.rows_per_env
    first = world.info.contact_slots_per_env * 16
    sequence = [("SnapshotStepVelocity", ("snapshot_step_velocity",)), ("FkWorldPoses", ("fk_world_poses",)), ("ApplyDrives", ("apply_drives",)),
                ("ArticulationDynamics", ("articulation_dynamics", 1)), ("SyncLinkBodyPose", ("sync_link_body_pose",)),
                ("BuildAabbs", ("build_aabbs",)), ("LbvhQueryPairs", ("query_pairs",)), ("NarrowphasePrimitives", ("narrowphase",)),
                ("AssembleRows", ("assemble_rows",))]
    for name, call in sequence:
        oracle.op(*call)
        world.op(name)
    world.synchronize()
    got = world.download("urows").view(np.uint32).reshape(E, R, ROW_WORDS)
    expect = oracle.download("urows").view(np.uint32).reshape(E, R, ROW_WORDS)
    assert np.array_equal(got[:, first:, [0, 1, 2, 3, 10, 11]], expect[:, first:, [0, 1, 2, 3, 10, 11]])
    joint_flags = expect[:, first:, 0]
    mujoco_rows = (joint_flags & (1 << 11)) != 0
    assert ((joint_flags & 1) != 0)[mujoco_rows].sum() >= E and (mujoco_rows & ((joint_flags & 1) == 0)).sum() > 0   # live ones, and limits left off
    active = (expect[:, :, 0] & 1) != 0
    for word in (4, 5, 6, 7):   # rhs (with the start-velocity forcing), compliance, bounds
        a = np.where(active, got.view(np.float32)[:, :, word], 0.0)
        b = np.where(active, expect.view(np.float32)[:, :, word], 0.0)
        a, b = np.clip(a, -1e30, 1e30), np.clip(b, -1e30, 1e30)
        assert per_env_error(a, b, E).max() <= TOL, word
    assert np.array_equal(world.download("lambda").reshape(E, R)[:, first:] != 0, oracle.download("lambda").reshape(E, R)[:, first:] != 0)
    for name, call in (("ContactWarmStart", ("contact_warm_start", 0)), ("BlockDescentSolve", ("block_descent_solve",))):
        oracle.op(*call)
        world.op(name)
    oracle.op("contact_warm_start", 1); world.op("ContactWarmStart", 1)
    oracle.op("readout_drives"); world.op("ReadoutDrives")
    world.synchronize()
    close(world, oracle, "qdot", tol=2e-4)
    before = world.download("qdot").copy()
    oracle.op("articulation_damping"); world.op("ArticulationDamping")
    world.synchronize()
    assert np.abs(world.download("qdot") - before).max() > 1e-4          # the op did something
    for name in ("qdot", "link_velocity", "qdot_flat", "actuator_effort", "tau"):
        close(world, oracle, name, tol=2e-4)
    oracle.close(); world.close()
    cfg, t, oracle, world = mujoco_joint_pair(oracle_py, device, index, E, integrator)
    oracle.step(6); world.step(6); world.synchronize()
    assert np.array_equal(world.download("env_status"), oracle.download("env_status")) and (oracle.download("env_status") == 0).all()
    for name in ("q", "qdot", "base_pose", "link_velocity", "actuator_effort"):
        close(world, oracle, name, tol=1e-3)
    oracle.close(); world.close()


def test_mjcf_scene_runs_the_mujoco_joint_law_unless_told_otherwise(oracle_py, device):
    """An MJCF file's joints and integrator (mjcf_importer.cpp:1193, 1720): MuJoCo-sourced by default, native with the
    scene flags; either way the device follows the oracle."""
    import os
    path = os.path.join(os.path.dirname(__file__), "data", "capsule_walker.xml")
    for flags, law, integrator in ((0, abi.LAW_MUJOCO, abi.INTEGRATOR_MUJOCO_EULER),
                                   (nk.SCENE_NATIVE_JOINT_LAW | nk.SCENE_NATIVE_CONTACT_LAW, abi.LAW_NATIVE, abi.INTEGRATOR_NATIVE)):
        scene = nk.Scene(path, flags)
        arrays = scene.template_arrays()
        assert (arrays["joint_law"] == law).all() and arrays["integrator"] == integrator
        E = 16
        desc = abi.world_desc(E, scene.info.timestep, vel_iters=8)
        oracle, world = oracle_py.OracleWorld(scene, desc, threads=8), nk.World(device, scene, desc)
        state = scene.initial_state()
        for w in (oracle, world):
            for name in ("q", "drive_stiffness", "drive_damping", "drive_force_limit", "drive_joint_force_limit"):
                w.upload(name, np.tile(state[name], E))
            w.upload("base_pose", np.tile(state["base_pose"], E))
            w.upload("drive_target", np.tile(state["q"], E))
        oracle.op("fk_world_poses"); oracle.op("sync_link_body_pose"); oracle.op("reference_weights")
        world.op("FkWorldPoses"); world.op("SyncLinkBodyPose")
        if law == abi.LAW_MUJOCO:
            world.op("ReferenceWeights")
        oracle.step(20); world.step(20); world.synchronize()
        assert np.array_equal(world.download("env_status"), oracle.download("env_status"))
        for name in ("q", "qdot", "base_pose"):
            close(world, oracle, name, tol=1e-3)
        oracle.close(); world.close()
