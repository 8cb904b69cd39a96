"""A free rigid body on the device against the oracle: the reference's rigid-body ops (BodyIntegrateVelocityKernel, the
six by six block of the tile, BodyIntegratePositionKernel with the free-rotation solve; articulation.cu:1019-1117,
block_descent_rigid.cuh, block_descent_tile.cuh:541-603) behind the same C ABI as the articulated worlds."""
import numpy as np
import pytest

from conftest import nk
from rigid import body_field, box_template, of_body
from test_gpu_parity import TOL, per_env_error

abi = nk.abi
pytestmark = pytest.mark.gpu


def seeded_boxes(E, seed, height=0.1, spread=0.01, tilt=0.03, speed=0.3, spin=1.0):
    g = np.random.default_rng(seed)
    pose = np.zeros((E, 7), np.float32)
    pose[:, :2] = g.normal(0.0, 0.5, (E, 2))
    pose[:, 2] = height + g.uniform(-0.004, spread, E)
    pose[:, 3] = 1.0
    pose[:, 4:] = 0.5 * g.normal(0.0, tilt, (E, 3))
    pose[:, 3:] /= np.linalg.norm(pose[:, 3:], axis=1, keepdims=True)
    return pose, g.normal(0.0, speed, (E, 3)).astype(np.float32), g.normal(0.0, spin, (E, 3)).astype(np.float32)


def pair(oracle_py, device, template, E, dt=1.0 / 240.0, **kw):
    desc = abi.world_desc(E, dt, **kw)
    return nk.World(device, template, desc), oracle_py.OracleWorld(template, desc, threads=8)


def put(world, oracle, template, pose, v, w):
    for side in (world, oracle):
        side.upload("base_pose", pose)
        side.upload("body_linear_velocity", body_field(template, v))
        side.upload("body_angular_velocity", body_field(template, w))


def close_env(world, oracle, name, E, tol=TOL):
    errors = per_env_error(world.download(name), oracle.download(name), E)
    assert errors.max() <= tol, f"{name}: worst environment {errors.max():.2e}"
    return float(errors.max())


def test_free_flight_matches_the_oracle_over_many_steps(oracle_py, device):
    """No contact rows: velocity update, free-rotation solve and pose update alone, two hundred steps of tumbling boxes
    with the centre of mass off the body's origin."""
    E = 256
    t = box_template(half=(0.1, 0.2, 0.05), mass=2.0, diag=(0.02, 0.05, 0.035), com=(0.05, -0.02, 0.03), plane=False)
    world, oracle = pair(oracle_py, device, t, E)
    pose, v, w = seeded_boxes(E, 3, height=1.0, tilt=0.5, spin=4.0)
    put(world, oracle, t, pose, v, w)
    for steps in (1, 199):
        world.step(steps); world.synchronize()
        oracle.step(steps)
        for name in ("base_pose", "body_linear_velocity", "body_angular_velocity", "body_pose"):
            close_env(world, oracle, name, E, tol=TOL if steps == 1 else 5 * TOL)
    assert np.array_equal(world.download("body_gyro_status"), oracle.download("body_gyro_status"))
    iterations = oracle.download("body_gyro_iterations")
    assert iterations.max() >= 1 and np.array_equal(world.download("body_gyro_iterations"), iterations)   # the Newton steps of the free-rotation solve
    assert not world.download("env_status").any()
    world.close(); oracle.close()


@pytest.mark.parametrize("mode", ["eager", "graph"])
def test_box_on_a_plane_matches_the_oracle_op_by_op_and_over_steps(oracle_py, device, mode):
    """Boxes dropped onto, resting on and sliding over the plane (four-point manifolds, the general narrowphase): every
    op of one step against the oracle - the staged block, the rows and their six entries, the solve - then thirty steps."""
    E = 128
    t = box_template(half=(0.2, 0.15, 0.1), mass=3.0, diag=(0.03, 0.04, 0.05), com=(0.03, 0.01, -0.02), mu=0.6)
    world, oracle = pair(oracle_py, device, t, E, vel_iters=8, pos_iters=4, contact_margin=0.02)
    pose, v, w = seeded_boxes(E, 11)
    put(world, oracle, t, pose, v, w)
    R = world.rows_per_env
    if mode == "eager":
        ops = [("IntegrateVelocity", "body_integrate_velocity"), ("FkWorldPoses", "fk_world_poses"), ("SyncLinkBodyPose", "sync_link_body_pose"),
               ("BuildAabbs", "build_aabbs"), ("LbvhQueryPairs", "query_pairs"), ("NarrowphasePrimitives", "narrowphase"),
               ("AssembleRows", "assemble_rows")]
        for device_op, oracle_op in ops:
            world.op(device_op); oracle.op(oracle_op)
        world.synchronize()
        for name in ("m", "body_world_inv_inertia", "body_linear_velocity", "body_angular_velocity", "qdot_flat", "body_pose", "body_aabb_lo",
                     "body_aabb_hi"):
            close_env(world, oracle, name, E)
        factor_w, factor_o = world.download("m_factor").reshape(E, -1), oracle.download("m_factor").reshape(E, -1)
        md = int(round(np.sqrt(factor_w.shape[1])))
        lower = np.tril(np.ones((md, md), bool)).reshape(-1)
        assert per_env_error(factor_w[:, lower], factor_o[:, lower], E).max() <= TOL
        for name in ("pair_count", "ucontact_count", "row_count", "contact_count", "row_cj_link", "row_cj_link_b"):
            assert np.array_equal(world.download(name), oracle.download(name)), name
        assert (oracle.download("contact_count") >= 3).mean() >= 0.5, "most boxes must touch with a whole face"
        active = (oracle.download("urows").reshape(E, R, 26).view(np.uint32)[:, :, 0] & 1) != 0
        for name in ("chain_jacobian", "chain_jacobian_b"):
            g, o = world.download(name).reshape(E, R, -1), oracle.download(name).reshape(E, R, -1)
            scale = np.abs(o).max() + 1e-30
            assert np.abs(np.where(active[..., None], g - o, 0.0)).max() <= TOL * scale, name
        world.op("ContactWarmStart"); oracle.op("contact_warm_start", 0)
        world.op("BlockDescentSolve"); oracle.op("block_descent_solve")
        world.synchronize()
        assert np.array_equal(world.download("env_status"), oracle.download("env_status"))
        got, expect = world.download("qdot_flat").reshape(E, -1)[:, :6], oracle.download("qdot_flat").reshape(E, -1)[:, :6]
        speed = np.maximum(np.abs(expect).max(1), 0.05)
        assert (np.abs(got - expect).max(1) / speed).max() <= 2e-4, (np.abs(got - expect).max(1) / speed).max()
        lam_g, lam_o = world.download("lambda").reshape(E, R), oracle.download("lambda").reshape(E, R)
        assert np.abs(lam_g - lam_o).max() <= 2e-4 * np.abs(lam_o).max()
        world.close(); oracle.close()
        return
    world.set_execution_mode(True)
    for steps in (1, 29):
        world.step(steps); world.synchronize()
        oracle.step(steps)
        assert np.array_equal(world.download("env_status"), oracle.download("env_status"))
        tol = TOL if steps == 1 else 10 * TOL
        close_env(world, oracle, "base_pose", E, tol=tol)
        close_env(world, oracle, "body_pose", E, tol=tol)
        got, expect = of_body(t, world.download("body_linear_velocity"), E), of_body(t, oracle.download("body_linear_velocity"), E)
        assert np.abs(got - expect).max() <= 20 * tol * max(1.0, np.abs(expect).max())
    # the boxes have settled on the plane: they carry their weight
    lam = world.download("lambda").reshape(E, R)
    normal = (world.download("urows").reshape(E, R, 26).view(np.uint32)[:, :, 0] & (1 << 6)) != 0
    support = np.where(normal, lam, 0.0).sum(1) * 240.0
    resting = np.abs(of_body(t, world.download("body_linear_velocity"), E)).max(1) < 0.02
    assert resting.mean() >= 0.5 and np.allclose(support[resting], 3.0 * 9.81, rtol=0.05)
    world.close(); oracle.close()


def test_a_free_body_refuses_what_it_does_not_build(device):
    t = box_template()
    t.add_link(abi.JOINT_REVOLUTE, 0)
    with pytest.raises(Exception):
        nk.World(device, t, abi.world_desc(4, 1.0 / 240.0))


def shaped_template(kind, params, mu=0.6):
    t = abi.Template()
    t.free_body = True
    t.add_link(abi.JOINT_FLOATING, None, mass=1.5, diag_inertia=(0.012, 0.015, 0.02), com=(0.01, 0.0, 0.005))
    profile = t.add_profile(mu)
    t.add_body(abi.ROLE_STATIC, kind=abi.SHAPE_PLANE, contype=2, conaffinity=1, profile=profile)
    t.add_body(abi.ROLE_LINK_BODY, link=0, kind=kind, params=params, contype=1, conaffinity=2, profile=profile)
    t.max_contacts_per_env = 1
    return t


@pytest.mark.parametrize("kind,params,height", [(abi.SHAPE_SPHERE, (0.1, 0, 0, 0), 0.1), (abi.SHAPE_CAPSULE, (0.06, 0.1, 0, 0), 0.06),
                                                (abi.SHAPE_CYLINDER, (0.08, 0.1, 0, 0), 0.08)])
def test_other_shapes_of_a_free_body_follow_the_oracle(oracle_py, device, kind, params, height):
    """A ball, a lying capsule and a lying cylinder (the single-point pairs take the merged collision kernel, the others
    the general one): forty steps of rolling and sliding on the plane, in graph mode."""
    E = 96
    t = shaped_template(kind, params)
    world, oracle = pair(oracle_py, device, t, E, vel_iters=8, pos_iters=4, contact_margin=0.02)
    pose, v, w = seeded_boxes(E, 5 + kind, height=height, spread=0.02, tilt=0.0, speed=0.5, spin=2.0)
    if kind != abi.SHAPE_SPHERE:   # lying on its side: the axis along x
        pose[:, 3:] = np.array([np.sqrt(0.5), 0.0, np.sqrt(0.5), 0.0], np.float32)
    put(world, oracle, t, pose, v, w)
    world.set_execution_mode(True)
    for steps in (1, 39):
        world.step(steps); world.synchronize()
        oracle.step(steps)
        assert np.array_equal(world.download("env_status"), oracle.download("env_status"))
        assert np.array_equal(world.download("contact_count"), oracle.download("contact_count"))
        tol = TOL if steps == 1 else 20 * TOL
        close_env(world, oracle, "base_pose", E, tol=tol)
        got, expect = of_body(t, world.download("body_angular_velocity"), E), of_body(t, oracle.download("body_angular_velocity"), E)
        assert np.abs(got - expect).max() <= 20 * tol * max(1.0, np.abs(expect).max())
    assert (oracle.download("contact_count") > 0).mean() >= 0.5
    world.close(); oracle.close()


def test_checkpoint_reset_and_large_batches_of_free_bodies(oracle_py, device):
    """The body's state is part of a checkpoint and of a reset; a batch of 8192 boxes (the solve's kernels for three waves
    a SIMD) gives in every copy the bits a batch of 64 gives."""
    E, copies = 64, 128
    t = box_template(half=(0.2, 0.15, 0.1), mass=3.0, diag=(0.03, 0.04, 0.05), mu=0.6)
    desc = abi.world_desc(E, 1.0 / 240.0, vel_iters=8, pos_iters=4, contact_margin=0.02)
    small = nk.World(device, t, desc)
    pose, v, w = seeded_boxes(E, 21)
    small.upload("base_pose", pose); small.upload("body_linear_velocity", body_field(t, v)); small.upload("body_angular_velocity", body_field(t, w))
    start = small.checkpoint()
    small.step(5); small.synchronize()
    after = {name: small.download(name) for name in ("base_pose", "body_linear_velocity", "body_angular_velocity", "lambda")}
    small.restore(start)
    assert np.array_equal(of_body(t, small.download("body_linear_velocity"), E), v) and np.array_equal(small.download("base_pose").reshape(E, 7), pose)
    small.step(5); small.synchronize()
    for name, value in after.items():
        assert np.array_equal(small.download(name), value), name
    big = nk.World(device, t, abi.world_desc(E * copies, 1.0 / 240.0, vel_iters=8, pos_iters=4, contact_margin=0.02))
    assert big.info.solver_blocks_per_cu > 8
    big.upload("base_pose", np.tile(pose, (copies, 1)))
    big.upload("body_linear_velocity", np.tile(body_field(t, v), (copies, 1, 1)))
    big.upload("body_angular_velocity", np.tile(body_field(t, w), (copies, 1, 1)))
    big.step(5); big.synchronize()
    for name, value in after.items():
        batch = big.download(name).reshape(copies, -1)
        assert np.array_equal(np.broadcast_to(value.reshape(1, -1), batch.shape), batch), name
    # a masked reset returns the chosen environments' bodies to the state of creation and leaves the others alone
    before = {name: small.download(name).reshape(E, -1) for name in ("base_pose", "body_linear_velocity", "body_angular_velocity")}
    chosen = np.array([3, 17, 40], np.uint32)
    small.reset_envs(chosen); small.synchronize()
    others = np.setdiff1d(np.arange(E), chosen)
    for name, value in before.items():
        now = small.download(name).reshape(E, -1)
        assert np.array_equal(now[others], value[others]), name
        expect = np.array([0, 0, 0, 1, 0, 0, 0], np.float32) if name == "base_pose" else 0.0
        assert np.array_equal(now[chosen], np.broadcast_to(expect, now[chosen].shape)), name
    small.reset(); small.synchronize()
    assert not small.download("body_linear_velocity").any() and not small.download("body_angular_velocity").any()
    small.close(); big.close()


def test_the_box_is_as_close_to_the_double_precision_answer_as_the_oracle(oracle_py, device):
    """One step of boxes meeting the plane on the device, in the single-precision oracle and in the oracle built in double:
    the device's velocities and poses lie within 1e-4 of the double-precision answer, or no further from it than twice
    the single-precision oracle does (median, 95th percentile and largest over the batch)."""
    E = 256
    t = box_template(half=(0.2, 0.15, 0.1), mass=3.0, diag=(0.03, 0.04, 0.05), com=(0.03, 0.01, -0.02), mu=0.6)
    desc = abi.world_desc(E, 1.0 / 240.0, vel_iters=8, pos_iters=4, contact_margin=0.02)
    world, single, double = nk.World(device, t, desc), oracle_py.OracleWorld(t, desc, threads=8), oracle_py.OracleWorld(t, desc, threads=8, double=True)
    pose, v, w = seeded_boxes(E, 31)
    put(world, single, t, pose, v, w)
    double.upload("base_pose", pose); double.upload("body_linear_velocity", body_field(t, v)); double.upload("body_angular_velocity", body_field(t, w))
    world.step(); world.synchronize(); single.step(); double.step()
    assert (single.download("contact_count") > 0).mean() >= 0.5

    def coordinates(side):
        return np.concatenate([of_body(t, side.download("body_linear_velocity"), E), of_body(t, side.download("body_angular_velocity"), E)], axis=1).astype(np.float64)

    exact = coordinates(double)
    scale = np.maximum(np.abs(exact).max(1), 0.05)
    for name, field in (("velocity", coordinates), ("pose", lambda side: side.download("base_pose").reshape(E, 7).astype(np.float64))):
        reference = field(double)
        size = scale if name == "velocity" else np.maximum(np.abs(reference).max(1), 1e-3)
        dev = np.abs(field(world) - reference).max(1) / size
        ora = np.abs(field(single) - reference).max(1) / size
        for what, measure in (("median", np.median), ("95th percentile", lambda x: np.percentile(x, 95)), ("largest", np.max)):
            d, o = float(measure(dev)), float(measure(ora))
            assert d <= max(TOL, 2.0 * o), f"{name} {what}: device {d:.2e} from the double-precision answer, oracle {o:.2e}"
        print(f"{name}: device {dev.max():.1e} (median {np.median(dev):.1e}), oracle {ora.max():.1e} (median {np.median(ora):.1e})")
    world.close(); single.close(); double.close()


@pytest.mark.parametrize("flags,cone", [("native", None), ("mujoco", "pyramidal"), ("mujoco", "elliptic")])
def test_a_scene_files_lone_free_body_is_a_free_rigid_body(oracle_py, device, flags, cone, tmp_path):
    """A body on a free joint that no joint hangs a child on is no articulation in the reference
    (articulation_cooker.cpp:148-151): the scene's template says free_body, and the world steps it with the rigid-body
    ops as the oracle does on the same template - under the native laws and under the file's own MuJoCo contact law
    (compliant rows weighted by BodyReferenceWeightsKernel's inverse mass; both cones)."""
    import os
    from conftest import ROOT
    path = os.path.join(ROOT, "tests", "data", "free_box.xml")
    if cone == "elliptic":
        text = open(path).read().replace('<option timestep="0.004"', '<option cone="elliptic" timestep="0.004"')
        path = str(tmp_path / "free_box_elliptic.xml")
        open(path, "w").write(text)
    scene = nk.Scene(path, nk.SCENE_NATIVE_CONTACT_LAW | nk.SCENE_NATIVE_JOINT_LAW if flags == "native" else 0)
    tdesc = scene.to_c()[0]
    assert tdesc.free_body == 1 and tdesc.link_count == 1 and tdesc.drive_rows == 0 and tdesc.integrator == 0
    assert (scene.template_arrays()["profile_law"] == (0 if flags == "native" else 1)).all()
    E = 64
    desc = abi.world_desc(E, scene.info.timestep, gravity=tuple(scene.info.gravity), vel_iters=8, pos_iters=4)
    world, oracle = nk.World(device, scene, desc), oracle_py.OracleWorld(scene, desc, threads=8)
    oracle.upload("base_pose", world.download("base_pose"))          # the pose the file authors, in every environment
    nb = tdesc.body_count
    own = int(np.argmax(np.ctypeslib.as_array(tdesc.body_role, shape=(nb,)) == abi.ROLE_LINK_BODY))
    if flags == "mujoco":
        weights = world.download("body_invweight0").reshape(E, nb, 2)
        assert np.allclose(weights[:, own], [1.0 / 2.5, (1 / 0.03 + 1 / 0.045 + 1 / 0.05) / 3.0], rtol=1e-6) and not np.delete(weights, own, axis=1).any()
        assert np.array_equal(weights, oracle.download("body_invweight0").reshape(E, nb, 2))
    g = np.random.default_rng(4)
    spin, push = np.zeros((E, nb, 3), np.float32), np.zeros((E, nb, 3), np.float32)
    spin[:, own] = g.normal(0.0, 0.5, (E, 3))
    push[:, own] = g.normal(0.0, 0.3, (E, 3))
    for side in (world, oracle):
        side.upload("body_angular_velocity", spin)
        side.upload("body_linear_velocity", push)
    world.set_execution_mode(True)
    for steps in (1, 59):
        world.step(steps); world.synchronize()
        oracle.step(steps)
        assert np.array_equal(world.download("env_status"), oracle.download("env_status")) and not oracle.download("env_status").any()
        assert np.array_equal(world.download("contact_count"), oracle.download("contact_count"))
        close_env(world, oracle, "base_pose", E, tol=TOL if steps == 1 else 20 * TOL)
    assert (oracle.download("contact_count") >= 3).mean() >= 0.8     # the crates lie on the floor
    world.close(); oracle.close()
