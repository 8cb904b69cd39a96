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
