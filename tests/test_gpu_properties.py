"""Size-independent properties of the HIP path at the published sizes, edge cases and error paths (MI355X)."""
import ctypes as C

import numpy as np
import pytest

from conftest import per_env_error, nk, relative_error

pytestmark = pytest.mark.gpu
abi = nk.abi
ROW_WORDS = 26
IDENTITY7 = np.array([0, 0, 0, 1, 0, 0, 0], np.float32)


def stepped(device, index, E, **kw):
    cfg = nk.synthetic.config(index, E)
    world = nk.World(device, cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters, **kw))
    world.set_state(cfg.state())
    return cfg, world


def test_humanoid_4096_contact_solution_properties(device):
    """The headline batch: cone, non-negative normal impulses, momentum balance M dv = J^T lambda with the GPU's own
    M and J, finite state, and environments independent of the batch they run in."""
    E = 4096
    cfg, world = stepped(device, 3, E)
    for name in ("FkWorldPoses", "ArticulationDynamics", "SyncLinkBodyPose", "BuildAabbs", "LbvhQueryPairs",
                 "NarrowphasePrimitives", "AssembleRows"):
        world.op(name)
    world.synchronize()
    n, R, nl = world.dof, world.rows_per_env, world.link_count
    free = world.download("qdot_flat").reshape(E, -1)[:, :n].astype(np.float64)
    world.op("BlockDescentSolve")
    world.synchronize()
    rows = world.download("urows").reshape(E, R, ROW_WORDS)
    words = rows.view(np.uint32)
    lam = world.download("lambda").reshape(E, R).astype(np.float64)
    assert np.all(world.download("env_status") == 0) and np.all(np.isfinite(lam))
    normal = (words[:, :, 0] & (1 << 6)) != 0
    assert normal.sum() > E
    assert np.all(lam[normal] >= 0)
    e_idx, r_idx = np.nonzero(normal)
    P = words[e_idx, r_idx, 2]
    tangent = np.hypot(lam[e_idx, r_idx + P], lam[e_idx, r_idx + 2 * P])
    mu = rows[e_idx, r_idx, 8]
    assert np.all(tangent <= mu * lam[e_idx, r_idx] * (1 + 1e-5) + 1e-7)
    assert np.all(lam[(words[:, :, 0] & 1) == 0] == 0)                         # dead rows hold no impulse
    M = world.download("m").reshape(E, n, n).astype(np.float64)
    J = (world.download("chain_jacobian").reshape(E, R, -1) + world.download("chain_jacobian_b").reshape(E, R, -1))[:, :, :n]
    scalar = [i for i, l in enumerate(cfg.template.links) if l["joint_type"] in (abi.JOINT_REVOLUTE, abi.JOINT_PRISMATIC)]
    v = np.concatenate([world.download("link_velocity").reshape(E, nl, 6)[:, 0, :], world.download("qdot").reshape(E, nl)[:, scalar]], 1)
    impulse = np.einsum("eri,er->ei", J.astype(np.float64), lam)
    balance = np.einsum("eij,ej->ei", M, v - free) - impulse
    imbalance = np.abs(np.linalg.solve(M, balance[:, :, None])[:, :, 0]).max(1)        # in velocity units
    residual = world.download("solver_residual").reshape(E, 4)
    # environments that met the tolerance inside the sweep budget hold the balance to rounding; the others stop with
    # the impulses one dual update ahead of the velocity, which solver_residual reports
    converged = world.download("vbd_velocity_sweep_count") < cfg.vel_iters
    assert converged.mean() > 0.5
    assert np.all(imbalance[converged] < 1.2e-5)                                       # the velocity tolerance is 1e-5
    assert np.all(np.isfinite(residual[:, :3])) and np.all(residual[converged].max(1) < 2e-5)
    # batch independence: the first 64 environments of the 4096 equal a 64-environment world bit for bit
    _, small = stepped(device, 3, 64)
    small.step()
    small.synchronize()
    world.reset()
    world.set_state(cfg.state())
    world.step()
    world.synchronize()
    for name, per in (("q", nl), ("qdot", nl), ("lambda", R), ("link_pose", nl * 7)):
        assert np.array_equal(world.download(name).reshape(E, per)[:64], small.download(name).reshape(64, per)), name
    small.close()
    world.close()


@pytest.mark.parametrize("index,E", [(2, 4096), (4, 1024), (4, 16384), (4, 65536)])
def test_full_size_batches_step_cleanly(device, index, E):
    """Every environment count of the humanoid sweep (and the quadruped batch) steps twice without a status bit, with
    finite state and unit quaternions; the first 64 environments of the batch equal a 64-environment world bit for
    bit, whatever the batch size and the launch order the larger batch gives them."""
    cfg, world = stepped(device, index, E)
    _, small = stepped(device, index, 64)
    world.step()
    small.step()
    world.synchronize()
    small.synchronize()
    nl, R = world.link_count, world.rows_per_env
    for name, per in (("q", nl), ("qdot", nl), ("lambda", R), ("link_pose", nl * 7), ("candidate_pairs", None)):
        big, few = world.download(name), small.download(name)
        per = per if per is not None else few.size // 64
        assert np.array_equal(big.reshape(E, per)[:64], few.reshape(64, per)), name
    small.close()
    world.step()
    world.synchronize()
    assert np.all(world.download("env_status") == 0)
    for name in ("q", "qdot", "link_pose", "lambda"):
        assert np.all(np.isfinite(world.download(name))), name
    pose = world.download("link_pose").reshape(E, -1, 7)
    assert np.abs(np.linalg.norm(pose[:, :, 3:], axis=2) - 1).max() < 1e-5      # unit quaternions
    assert np.all(world.download("pair_count") <= world.info.contact_slots_per_env)
    sweeps = world.download("vbd_velocity_sweep_count")
    assert sweeps.min() >= 1 and sweeps.max() <= cfg.vel_iters
    world.close()


def test_scene_files_at_full_batch_size(device):
    """The capsule walker (links meeting links and the floor) and the URDF walker at 4096 environments, a hundred
    steps from the authored pose with per-environment pushes: no status bit, finite state, unit quaternions, the
    identical environments 0 and 1 stay identical, and the robots end up carried by contacts rather than falling."""
    import os
    from conftest import ROOT
    E = 4096
    for path, flags in ((os.path.join(ROOT, "tests", "data", "capsule_walker.xml"), 0),
                        (os.path.join(ROOT, "tests", "data", "legged.urdf"), nk.SCENE_GROUND_PLANE | nk.SCENE_PLANE_CONTACTS_ONLY)):
        scene = nk.Scene(path, flags)
        world = nk.World(device, scene, abi.world_desc(E, 0.0 if path.endswith(".xml") else 1.0 / 240.0, vel_iters=8))
        nl = scene.link_count
        rng = np.random.default_rng(5)
        twist = np.zeros((E, nl, 6), np.float32)
        twist[2:, 0] = rng.normal(0, 0.2, (E - 2, 6))
        base = world.download("base_pose").reshape(E, 7).copy()
        base[:, 2] = 0.545 if path.endswith(".xml") else 0.488          # soles on the floor
        world.upload("base_pose", base)
        world.upload("link_velocity", twist)
        world.step(100)
        world.synchronize()
        assert not world.download("env_status").any()
        for name in ("q", "qdot", "link_pose", "lambda"):
            assert np.all(np.isfinite(world.download(name))), name
        pose = world.download("link_pose").reshape(E, nl, 7)
        assert np.abs(np.linalg.norm(pose[:, :, 3:], axis=2) - 1).max() < 1e-5
        assert np.array_equal(pose[0], pose[1])
        assert (world.download("contact_count") >= 1).mean() > 0.9 and np.median(pose[:, 0, 2]) > 0.15
        world.close()


def test_long_run_of_an_authored_robot_stays_bounded(device):
    """Ten simulated seconds of the capsule walker holding its authored pose on damped, driven joints (graph replay):
    every environment stays finite and flagged clean, velocities stay small and the robots stay carried by their
    contacts.  (The benchmark configurations are no such test: their seeded torques act on undamped joints.)"""
    import os
    from conftest import ROOT
    E, steps = 1024, 2000
    scene = nk.Scene(os.path.join(ROOT, "tests", "data", "capsule_walker.xml"))
    world = nk.World(device, scene, abi.world_desc(E, 0.0, vel_iters=8))
    nl = scene.link_count
    rng = np.random.default_rng(11)
    twist = np.zeros((E, nl, 6), np.float32)
    twist[:, 0] = rng.normal(0, 0.3, (E, 6))
    base = world.download("base_pose").reshape(E, 7).copy()
    base[:, 2] = 0.545
    world.upload("base_pose", base)
    world.upload("link_velocity", twist)
    world.set_execution_mode(True)
    peak = 0.0
    for _ in range(4):
        world.step(steps // 4); world.synchronize()
        qdot = world.download("qdot")
        assert np.all(np.isfinite(qdot)) and not world.download("env_status").any()
        peak = max(peak, float(np.abs(qdot).max()))
    assert peak < 50.0, peak
    pose = world.download("link_pose").reshape(E, nl, 7)
    assert np.all(np.isfinite(pose)) and np.abs(np.linalg.norm(pose[:, :, 3:], axis=2) - 1).max() < 1e-5
    assert (world.download("contact_count") >= 1).mean() > 0.9 and pose[:, 0, 2].min() > 0.0
    world.close()


def test_rope_full_batch_steps(device):
    """All 8192 environments of the rope for several steps: no environment may raise a status bit (a failed
    factorisation, a non-finite velocity), every link keeps its contact, and the step's own result balances momentum:
    M (v - v_free) = J^T lambda to the solve's tolerance, the size-independent check of the whole batch."""
    E = 8192
    cfg, world = stepped(device, 5, E)
    n, R = world.dof, world.rows_per_env
    for step in range(3):
        for name in ("FkWorldPoses", "ArticulationDynamics", "SyncLinkBodyPose", "BuildAabbs", "LbvhQueryPairs",
                     "NarrowphasePrimitives", "AssembleRows"):
            world.op(name)
        world.op("ContactWarmStart", 0)
        world.synchronize()
        free = world.download("qdot_flat").reshape(E, -1)[:, :n].astype(np.float64)
        world.op("BlockDescentSolve")
        world.synchronize()
        status = world.download("env_status")
        assert not status.any(), f"step {step}: {int((status != 0).sum())} of {E} environments raised a status bit"
        contacts = world.download("contact_count")
        assert contacts.mean() > 56.0 and contacts.min() >= 32        # links pushed out of the plane leave their contact
        sweeps = world.download("vbd_velocity_sweep_count")
        assert sweeps.min() >= 1 and sweeps.max() <= cfg.vel_iters
        velocity = world.download("qdot_flat").reshape(E, -1)[:, :n].astype(np.float64)
        M = world.download("m").reshape(E, n, n).astype(np.float64)
        J = (world.download("chain_jacobian").reshape(E, R, -1) + world.download("chain_jacobian_b").reshape(E, R, -1))[:, :, :n]
        impulse = np.einsum("eri,er->ei", J.astype(np.float64), world.download("lambda").reshape(E, R).astype(np.float64))
        momentum = np.einsum("eij,ej->ei", M, velocity - free)
        # the solve's own measure (MeasureTilePrimal): the velocity that the unbalanced momentum stands for
        balance = np.abs(np.linalg.solve(M, (momentum - impulse)[:, :, None])[:, :, 0]).max(1)
        converged = sweeps < cfg.vel_iters
        print(f"rope step {step}: sweeps mean {sweeps.mean():.2f}, at the cap {int((~converged).sum())}, "
              f"momentum balance worst {balance[converged].max():.2e} m/s against free velocities of {np.abs(free).max():.2e}")
        assert balance[converged].max() <= 1e-4
        world.op("ContactWarmStart", 1)
        for name in ("IntegratePosition", "FkWorldPoses", "FkLinkVelocities"):
            world.op(name)
        world.synchronize()
    pose = world.download("link_pose").reshape(E, -1, 7)
    assert np.all(np.isfinite(world.download("q"))) and np.all(np.isfinite(pose))
    assert pose[:, 1:, 2].min() > 0.005 and pose[:, 1:, 2].max() < 0.02        # the rope stays on the plane
    world.close()


def test_a_world_reports_the_width_and_the_occupancy_of_its_solve(device):
    """What the benchmark line quotes as `solver_width` and `blocks_per_cu`: the humanoid's contacts reach the root and the
    legs (18 coordinates), so its sweeps run 20 wide, eight blocks a compute unit like the quadruped's; the rope's block
    is 64 wide, keeps no contact rows and runs four a unit (one wavefront a SIMD); a world without contacts has no solve."""
    expected = {1: (7, 0), 2: (18, 8), 3: (20, 8), 5: (64, 4)}
    for index, (width, blocks) in expected.items():
        cfg = nk.synthetic.config(index, 8)
        world = nk.World(device, cfg.template, abi.world_desc(8, cfg.dt, vel_iters=cfg.vel_iters))
        assert (world.info.solver_width, world.info.solver_blocks_per_cu) == (width, blocks), f"config {index}"
        world.close()


def test_single_environment_and_contact_free_worlds(oracle_py, device):
    for index in (1, 3):
        cfg = nk.synthetic.config(index, 1)
        desc = abi.world_desc(1, cfg.dt, vel_iters=cfg.vel_iters)
        world, oracle = nk.World(device, cfg.template, desc), oracle_py.OracleWorld(cfg.template, desc)
        state = cfg.state()
        world.set_state(state)
        oracle.set_state(state)
        world.step()
        world.synchronize()
        oracle.step()
        for name in ("q", "qdot", "link_pose"):
            assert relative_error(world.download(name), oracle.download(name)) <= 1e-4
        world.close()
        oracle.close()


@pytest.mark.parametrize("index", [2, 3])
def test_a_non_finite_environment_is_flagged_and_alone(oracle_py, device, index):
    """Environments that start from a coordinate, a velocity, a base height or a torque that is not a number raise
    their own status word (as the oracle does) and change nothing in any other environment: every other environment's
    state after three steps equals, bit for bit, that of a batch without them."""
    E = 256
    cfg = nk.synthetic.config(index, E)
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    clean, dirty, oracle = nk.World(device, cfg.template, desc), nk.World(device, cfg.template, desc), oracle_py.OracleWorld(cfg.template, desc, threads=8)
    state = cfg.state()
    clean.set_state(state)
    bad = cfg.state()
    bad["q"][7, 3] = np.nan
    bad["qdot"][11, 2] = np.inf
    bad["base_pose"][13, 2] = np.nan
    bad["tau"][17, 4] = np.inf
    poisoned = [7, 11, 13, 17]
    dirty.set_state(bad)
    oracle.set_state(bad)
    for w in (clean, dirty, oracle):
        w.step(3)
    dirty.synchronize(); clean.synchronize()
    status = dirty.download("env_status")
    assert (status[poisoned] != 0).all() and np.array_equal(status[poisoned], oracle.download("env_status")[poisoned])
    others = np.setdiff1d(np.arange(E), poisoned)
    assert (status[others] == 0).all()
    for name in ("q", "qdot", "base_pose", "link_velocity", "lambda"):
        got, expect = dirty.download(name).reshape(E, -1), clean.download(name).reshape(E, -1)
        assert np.array_equal(got[others].view(np.uint32), expect[others].view(np.uint32)), name
    for w in (clean, dirty, oracle):
        w.close()


def box_template(plane_first):
    t = abi.Template()
    t.add_link(abi.JOINT_FLOATING, None, mass=1.2, diag_inertia=(0.004, 0.006, 0.005))
    t.add_link(abi.JOINT_REVOLUTE, 0, axis=(0, 1, 0), local_pos=(0.1, 0, 0.05), mass=0.3, diag_inertia=(0.001,) * 3, com=(0.05, 0, 0))
    profile = t.add_profile(0.6)
    plane = dict(kind=abi.SHAPE_PLANE, contype=2, conaffinity=1, profile=profile)
    if plane_first:
        t.add_body(abi.ROLE_STATIC, **plane)
    t.add_body(abi.ROLE_LINK_BODY, link=0, contype=0, conaffinity=0)
    t.add_body(abi.ROLE_LINK_BODY, link=1, contype=0, conaffinity=0)
    t.add_body(abi.ROLE_PROXY, link=0, kind=abi.SHAPE_BOX, params=(0.1, 0.06, 0.04, 0), contype=1, conaffinity=2, profile=profile)
    t.add_body(abi.ROLE_PROXY, link=1, kind=abi.SHAPE_SPHERE, params=(0.03, 0, 0, 0), local_pos=(0.1, 0, 0), contype=1, conaffinity=2, profile=profile)
    if not plane_first:
        t.add_body(abi.ROLE_STATIC, **plane)
    return t


@pytest.mark.parametrize("plane_first", [True, False])
def test_box_manifolds_and_either_side_order(oracle_py, device, plane_first):
    """A tilted box (up to four points per slot) plus a sphere; with the plane as the last row it is side B."""
    E = 64
    t = box_template(plane_first)
    g = np.random.default_rng(4)
    quat = np.array([1, 0, 0, 0]) + g.normal(0, 0.04, (E, 4))
    base = np.concatenate([g.normal(0, 0.2, (E, 2)), g.uniform(0.035, 0.05, (E, 1)), quat / np.linalg.norm(quat, axis=1, keepdims=True)], 1)
    zero = np.zeros((E, 1), np.float32)
    state = dict(q=np.concatenate([zero, g.uniform(-0.3, 0.6, (E, 1))], 1).astype(np.float32),
                 qdot=np.concatenate([zero, g.normal(0, 1, (E, 1))], 1).astype(np.float32), tau=np.zeros((E, 2), np.float32),
                 base_pose=base.astype(np.float32), root_twist=g.normal(0, 0.3, (E, 6)).astype(np.float32))
    desc = abi.world_desc(E, 1.0 / 200.0, vel_iters=50)
    world, oracle = nk.World(device, t, desc), oracle_py.OracleWorld(t, desc, threads=4)
    world.set_state(state)
    oracle.set_state(state)
    world.step()
    world.synchronize()
    oracle.step()
    for name in ("pair_count", "ucontact_count", "ucontact_row_range", "ucontact_id_pair", "row_count", "env_status"):
        assert np.array_equal(world.download(name), oracle.download(name)), name
    counts = oracle.download("ucontact_count")
    assert counts.max() == 4 and (counts == 1).any()
    S = world.info.contact_slots_per_env
    mask = np.arange(4)[None, None, :] < counts.reshape(E, S)[:, :, None]
    ids_g, ids_o = world.download("ucontact_id_feature").reshape(E, S, 4), oracle.download("ucontact_id_feature").reshape(E, S, 4)
    assert np.mean(ids_g[mask] == ids_o[mask]) > 0.99       # box corners carry feature ids: exact; sphere points hash a quantised position
    for name in ("qdot", "q", "link_pose", "link_velocity"):
        assert relative_error(world.download(name), oracle.download(name)) <= 1e-4, name
    world.close()
    oracle.close()


@pytest.mark.parametrize("shape", ["spheres", "boxes"])
def test_environments_on_either_side_of_the_capacity_split_match_the_oracle(oracle_py, device, shape):
    """A raft of a hundred spheres (or thirty boxes of four points each) over the plane: a tilted raft fills a few of
    its contact slots and a level one all.  The solve sends environments with few contact points to launches with
    a small LDS capacity and the others to fuller ones - two launches for the spheres, three for the boxes; either
    way an environment's result is the oracle's, which knows no such split.  Heads beyond the first sixty-four go
    through the head fields instead of lane registers."""
    E = 96
    t = abi.Template()
    t.add_link(abi.JOINT_FLOATING, None, mass=5.0, diag_inertia=(0.2, 0.2, 0.4))
    profile = t.add_profile(0.7)
    t.add_body(abi.ROLE_STATIC, kind=abi.SHAPE_PLANE, contype=2, conaffinity=1, profile=profile)
    t.add_body(abi.ROLE_LINK_BODY, link=0, contype=0, conaffinity=0)
    if shape == "spheres":
        rows, cols, pitch, kind, params, reach, bounds = 10, 10, 0.05, abi.SHAPE_SPHERE, (0.02, 0, 0, 0), 0.225, (56, 100, 100)
    else:
        rows, cols, pitch, kind, params, reach, bounds = 6, 5, 0.08, abi.SHAPE_BOX, (0.02, 0.02, 0.02, 0), 0.18, (56, 118, 120)
    for i in range(rows):
        for j in range(cols):
            t.add_body(abi.ROLE_PROXY, link=0, kind=kind, params=params, local_pos=(pitch * (i - (rows - 1) / 2), pitch * (j - (cols - 1) / 2), 0.0),
                       contype=1, conaffinity=2, profile=profile)
    g = np.random.default_rng(8)
    tilt = g.uniform(0.0, 0.12, E)
    tilt[:8] = 0.0                                               # level rafts: every shape touches
    tilt[8:32] = np.linspace(0.001, 0.03, 24)                    # nearly level ones: most do
    height = 0.02 * np.cos(tilt) + reach * np.sin(tilt) - 0.001
    base = np.stack([g.normal(0, 0.1, E), g.normal(0, 0.1, E), height, np.cos(tilt / 2), np.sin(tilt / 2), 0 * tilt, 0 * tilt], 1)
    state = dict(q=np.zeros((E, 1), np.float32), qdot=np.zeros((E, 1), np.float32), tau=np.zeros((E, 1), np.float32),
                 base_pose=base.astype(np.float32), root_twist=(g.normal(0, 0.2, (E, 6)) * [1, 1, 1, 1, 1, 0.2]).astype(np.float32))
    desc = abi.world_desc(E, 1.0 / 200.0, vel_iters=8)
    world, oracle = nk.World(device, t, desc), oracle_py.OracleWorld(t, desc, threads=8)
    assert world.info.contact_slots_per_env == rows * cols
    world.set_state(state)
    oracle.set_state(state)
    world.step(2); world.synchronize()
    oracle.step(2)
    counts = oracle.download("contact_count")
    small, middle, full = bounds
    assert (counts <= small).any() and ((counts > small) & (counts <= middle)).any() and counts.max() == full, np.sort(counts)
    for name in ("contact_count", "ucontact_count", "row_count", "env_status"):
        assert np.array_equal(world.download(name), oracle.download(name)), name
    assert not world.download("env_status").any()
    # an environment whose residual sits at the tolerance may stop a sweep earlier or later under other rounding
    assert np.mean(world.download("vbd_velocity_sweep_count") != oracle.download("vbd_velocity_sweep_count")) <= 0.05
    for name in ("qdot", "link_velocity", "base_pose"):
        error = per_env_error(world.download(name), oracle.download(name), E)
        assert error.max() <= 2e-4, (name, float(error.max()), int(counts[error.argmax()]))       # two steps
    # shapes in a row share a load in no unique way: the multipliers are compared through what they add up to
    oracle.op("readout_contact_wrench")
    error = per_env_error(world.download("link_contact_wrench"), oracle.download("link_contact_wrench"), E)
    assert np.abs(oracle.download("link_contact_wrench")).max() > 10.0 and error.max() <= 1e-3, float(error.max())
    world.close()
    oracle.close()


def test_error_paths(device):
    lib = nk.lib()
    cfg = nk.synthetic.config(2, 8)
    world = nk.World(device, cfg.template, abi.world_desc(8, cfg.dt))
    fid, view = world._field("q")
    nbytes = view.element_count * 4
    buf = (C.c_char * (nbytes + 8))()
    assert lib.nuka_world_download_field(world._h, fid, buf, nbytes + 4, 0) == 1          # past the end: refused, not clamped
    assert lib.nuka_world_upload_field(world._h, fid, buf, 8, nbytes - 4) == 1
    assert lib.nuka_world_download_field(world._h, fid, buf, 8, nbytes - 8) == 0
    assert lib.nuka_world_download_field(world._h, 10_000, buf, 4, 0) == 7
    assert lib.nuka_world_dispatch_op(world._h, 60_000, 0) == 1
    assert lib.nuka_world_set_velocity_iterations(world._h, 0) == 1
    assert lib.nuka_world_set_execution_mode(world._h, 5) == 1
    world.close()
    # templates outside the path are refused at creation
    for kinds in ((abi.SHAPE_CYLINDER, abi.SHAPE_CYLINDER), (abi.SHAPE_CAPSULE, abi.SHAPE_BOX), (abi.SHAPE_CYLINDER, abi.SHAPE_CAPSULE), (4, abi.SHAPE_PLANE)):
        t = abi.Template()   # an admitted pair without an analytic manifold, or a shape kind outside the path
        t.add_link(abi.JOINT_FLOATING, None)
        t.add_link(abi.JOINT_REVOLUTE, 0)
        t.add_body(abi.ROLE_LINK_BODY, link=0, kind=kinds[0], params=(0.1, 0.2, 0.1, 0))
        t.add_body(abi.ROLE_STATIC if kinds[1] == abi.SHAPE_PLANE else abi.ROLE_LINK_BODY, link=1, kind=kinds[1], params=(0.1, 0.2, 0.1, 0))
        with pytest.raises(nk.NukaError) as info:
            nk.World(device, t, abi.world_desc(4, 0.005))
        assert info.value.code == 7
    t.exclude(0, 1)          # the same pair, excluded: nothing left to refuse
    t.bodies[0]["kind"] = abi.SHAPE_BOX
    nk.World(device, t, abi.world_desc(4, 0.005)).close()
    t = abi.Template()
    t.add_link(abi.JOINT_FIXED, None)
    t.add_link(abi.JOINT_REVOLUTE, 5)
    with pytest.raises(nk.NukaError) as info:
        nk.World(device, t, abi.world_desc(4, 0.005))
    assert info.value.code == 1
    with pytest.raises(nk.NukaError):
        nk.World(device, nk.synthetic.config(1, 1).template, abi.world_desc(0, 0.005))


def table(handle, count):
    """The function-pointer table a seam handle starts with."""
    iface = C.cast(handle, C.POINTER(C.c_void_p))[0]
    return C.cast(iface, C.POINTER(C.c_void_p * count))[0]


def test_backend_seam_walk_through_the_tables(device):
    """Drives the PHI-shaped seam the way a foreign host would: only through the tables of include/nuka_phi.h."""
    lib = nk.lib()
    lib.nuka_hip_register_backend_entry.restype = C.c_void_p
    entry = lib.nuka_hip_register_backend_entry()
    e = table(entry, 4)
    name = C.CFUNCTYPE(C.c_char_p, C.c_void_p)(e[0])(entry)
    assert b"hip" in name.lower()
    assert C.CFUNCTYPE(C.c_size_t, C.c_void_p)(e[1])(entry) >= 1
    dev = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_size_t)(e[2])(entry, 0)
    d = table(dev, 6)
    supports = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_uint16)(d[5])
    names = [lib.nuka_hip_op_name(i).decode() for i in range(lib.nuka_hip_op_count())]
    for wanted in ("FkWorldPoses", "ArticulationDynamics", "AssembleRows", "BlockDescentSolve", "IntegratePosition"):
        assert supports(dev, names.index(wanted)) == 1
    assert supports(dev, 60_000) == 0
    free_b, total_b = C.c_size_t(), C.c_size_t()
    C.CFUNCTYPE(None, C.c_void_p, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t))(d[1])(dev, C.byref(free_b), C.byref(total_b))
    assert total_b.value > 200 * 2**30 and free_b.value <= total_b.value       # 288 GB of HBM3E
    # buffer type -> buffer -> upload / download round trip, and out-of-range transfers refused
    btype = C.CFUNCTYPE(C.c_void_p, C.c_void_p)(d[3])(dev)
    bt = table(btype, 4)
    assert C.CFUNCTYPE(C.c_int, C.c_void_p)(bt[3])(btype) == 0
    status = C.c_uint8(9)
    buf = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_size_t, C.POINTER(C.c_uint8))(bt[1])(btype, 4096, C.byref(status))
    assert buf and status.value == 0
    b = table(buf, 6)
    src = np.arange(1024, dtype=np.uint32)
    dst = np.zeros_like(src)
    upload = C.CFUNCTYPE(C.c_uint8, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t)(b[2])
    download = C.CFUNCTYPE(C.c_uint8, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t)(b[3])
    assert upload(buf, src.ctypes.data, 0, 4096) == 0 and download(buf, dst.ctypes.data, 0, 4096) == 0
    assert np.array_equal(src, dst)
    assert upload(buf, src.ctypes.data, 8, 4096) != 0
    C.CFUNCTYPE(None, C.c_void_p)(b[0])(buf)
    # the backend a device handle owns answers through its own table
    lib.nuka_device_backend.restype = C.c_void_p
    backend = lib.nuka_device_backend(device._h)
    k = table(backend, 15)
    assert b"hip" in C.CFUNCTYPE(C.c_char_p, C.c_void_p)(k[0])(backend).lower()


@pytest.mark.parametrize("index,E", [(2, 4096), (3, 4096)])
def test_published_batch_sizes_match_the_oracle_directly(oracle_py, device, index, E):
    """The whole published batch, not a sample: one step of all 4096 environments against the oracle (the oracle takes
    a fraction of a second for this on a few threads)."""
    cfg = nk.synthetic.config(index, E)
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    world, oracle = nk.World(device, cfg.template, desc), oracle_py.OracleWorld(cfg.template, desc, threads=16)
    state = cfg.state()
    world.set_state(state)
    oracle.set_state(state)
    world.step()
    world.synchronize()
    oracle.step()
    for name in ("pair_count", "ucontact_count", "ucontact_row_range", "row_count", "env_status", "contact_cache_pair",
                 "contact_cache_age", "contact_warm_start_counts"):
        assert np.array_equal(world.download(name), oracle.download(name)), name
    from test_gpu_parity import bar, one_ulp_sensitivity
    sens = one_ulp_sensitivity(oracle_py, cfg.template, desc, state, threads=16)
    for name in ("articulation_qdd", "link_pose", "body_pose", "q", "qdot", "link_velocity"):
        errors = per_env_error(world.download(name), oracle.download(name), E)
        tol = bar(sens, "velocity") if name in ("qdot", "link_velocity") else 1e-4
        print(f"{cfg.name} {E} envs {name}: worst environment {errors.max():.2e}, {int((errors > 1e-4).sum())} above 1e-4 (bar {tol:.1e})")
        assert errors.max() <= tol, f"{name}: {errors.max():.2e}"
    world.close()
    oracle.close()


def test_reset_envs_restores_the_selected_environments_only(device):
    """nuka_world_reset_envs: the chosen environments return to the state the world was created with and lose their
    contact and solver history; the others are untouched; duplicates are ignored and a bad id changes nothing."""
    E = 64
    cfg = nk.synthetic.config(2, E)
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    world = nk.World(device, cfg.template, desc)
    created = {n: world.download(n) for n in ("q", "qdot", "base_pose", "link_pose", "lambda")}
    state = cfg.state()
    world.set_state(state)
    world.step(3)
    world.synchronize()
    before = {n: world.download(n) for n in ("q", "qdot", "base_pose", "link_pose", "lambda", "contact_cache_pair", "contact_row_extent")}
    assert nk.lib().nuka_world_reset_envs(world._h, np.array([2, 99], np.uint32).ctypes.data, 2) == 1
    assert all(np.array_equal(world.download(n), v) for n, v in before.items())
    assert nk.lib().nuka_world_reset_envs(world._h, None, 0) == 0
    chosen = [3, 17, 3, 40]
    world.reset_envs(chosen)
    picked = np.zeros(E, bool)
    picked[chosen] = True
    for n in ("q", "qdot", "base_pose", "link_pose", "lambda"):
        now, was, new = (a.reshape(E, -1) for a in (world.download(n), before[n], created[n]))
        assert np.array_equal(now[~picked], was[~picked]) and np.array_equal(now[picked], new[picked]), n
    assert np.all(world.download("contact_cache_pair").reshape(E, -1)[picked] == 0)
    assert np.all(world.download("contact_row_extent").reshape(E, 2)[picked] == 0)
    assert np.array_equal(world.download("contact_cache_pair").reshape(E, -1)[~picked], before["contact_cache_pair"].reshape(E, -1)[~picked])
    # a reset environment, given its seeded state again, steps exactly as it did in a fresh world
    fresh = nk.World(device, cfg.template, desc)
    fresh.set_state(state)
    fresh.step()
    fresh.synchronize()
    for name, key in (("q", "q"), ("qdot", "qdot"), ("tau", "tau"), ("base_pose", "base_pose")):
        current = world.download(name).reshape(E, -1)
        current[picked] = np.asarray(state[key], np.float32).reshape(E, -1)[picked]
        world.upload(name, current)
    twist = world.download("link_velocity").reshape(E, -1, 6)
    twist[picked, 0, :] = state["root_twist"][picked]
    world.upload("link_velocity", twist)
    world.step()
    world.synchronize()
    for n in ("q", "qdot", "lambda", "link_pose"):
        assert np.array_equal(world.download(n).reshape(E, -1)[picked], fresh.download(n).reshape(E, -1)[picked]), n
    fresh.close()
    world.close()


@pytest.mark.parametrize("index,E", [(3, 512), (1, 64), (5, 64)])
def test_a_plan_steps_bit_for_bit_like_the_ops_one_by_one(device, index, E):
    """A plan may run neighbouring ops as one launch (the four after the solve); whatever it merges, the state after
    any number of steps must be the state the ops leave when each is dispatched by itself."""
    cfg = nk.synthetic.config(index, E)
    hashes = []
    fields = {}
    for graph in (False, True):
        world = nk.World(device, cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters))
        world.set_state(cfg.state())
        world.set_execution_mode(graph)
        world.step(5)
        world.synchronize()
        hashes.append(world.state_hash())
        fields[graph] = {name: world.download(name).copy() for name in ("q", "qdot", "base_pose", "link_pose", "link_velocity", "body_pose")}
        world.close()
    for name in fields[False]:
        assert np.array_equal(fields[False][name].view(np.uint32), fields[True][name].view(np.uint32)), name
    assert hashes[0] == hashes[1]


@pytest.mark.parametrize("case", ["substeps", "mujoco_integrator"])
def test_a_plan_merges_ops_inside_substeps_and_ahead_of_the_damping_pass(device, case):
    """The same identity where the ops a plan merges stand elsewhere in the list: inside an interval that repeats
    (two substeps, each closed by AccumulateStep), and with ArticulationDamping between the solve and the ops after it
    (the MuJoCo integrator on MuJoCo-sourced joints with servos)."""
    import copy
    E = 128
    cfg = nk.synthetic.config(3, E)
    t = copy.deepcopy(cfg.template)
    gains = {}
    if case == "mujoco_integrator":
        t.drive_rows, t.drive_mode, t.integrator = True, abi.DRIVE_PD_POSITION, abi.INTEGRATOR_MUJOCO_EULER
        for l, link in enumerate(t.links):
            if link["joint_type"] == abi.JOINT_REVOLUTE:
                link["law"] = abi.LAW_MUJOCO
                link["damping"] = 0.3
                link["lower"], link["upper"] = float(cfg.nominal_q[l]) - 0.4, float(cfg.nominal_q[l]) + 0.4
        rng = np.random.default_rng(3)
        nl = t.link_count
        gains = dict(drive_target=np.tile(cfg.nominal_q, (E, 1)), drive_stiffness=rng.uniform(20, 80, (E, nl)), drive_damping=rng.uniform(0.5, 3, (E, nl)))
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters, substeps=2 if case == "substeps" else 0)
    fields, hashes = {}, []
    for graph in (False, True):
        world = nk.World(device, t, desc)
        world.set_state(cfg.state())
        for name, values in gains.items():
            world.upload(name, values.astype(np.float32))
        world.set_execution_mode(graph)
        world.step(4)
        world.synchronize()
        assert not world.download("env_status").any()
        hashes.append(world.state_hash())
        fields[graph] = {name: world.download(name).copy() for name in ("q", "qdot", "base_pose", "link_pose", "link_velocity", "body_pose", "lambda")}
        world.close()
    for name in fields[False]:
        assert np.array_equal(fields[False][name].view(np.uint32), fields[True][name].view(np.uint32)), name
    assert hashes[0] == hashes[1]
