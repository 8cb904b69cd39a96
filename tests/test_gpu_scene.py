"""A world created from an MJCF scene file steps on the GPU as the oracle does on the same loaded template, starts
from the state the file authors and returns to it on reset."""
import os

import numpy as np
import pytest

from conftest import ROOT, nk, relative_error

pytestmark = pytest.mark.gpu
abi = nk.abi
TOL = 1e-4
BIPED = os.path.join(ROOT, "tests", "data", "biped.xml")


def test_scene_world_matches_the_oracle_and_resets_to_the_authored_state(oracle_py, device):
    E = 128
    scene = nk.Scene(BIPED, nk.SCENE_PLANE_CONTACTS_ONLY)
    desc = abi.world_desc(E, 0.0, gravity=(0.0, 0.0, 0.0), vel_iters=8)          # time step and gravity come from the file
    world = nk.World(device, scene, desc)
    state = scene.initial_state()
    assert np.allclose(world.download("base_pose").reshape(E, 7), state["base_pose"])
    assert np.array_equal(world.download("drive_stiffness").reshape(E, -1)[5], state["drive_stiffness"])
    assert np.array_equal(world.download("drive_target").reshape(E, -1)[7], state["q"])
    # per-environment variety: each environment is pushed differently and aims at a different pose
    rng = np.random.default_rng(17)
    nl = scene.link_count
    target = (rng.normal(0, 0.15, (E, nl)) * (state["drive_stiffness"] > 0)).astype(np.float32)
    twist = rng.normal(0, 0.3, (E, nl, 6)).astype(np.float32)
    twist[:, 1:] = 0.0
    oracle = oracle_py.OracleWorld(scene, abi.world_desc(E, scene.info.timestep, gravity=tuple(scene.info.gravity), vel_iters=8), threads=8)
    for name in ("q", "drive_stiffness", "drive_damping", "drive_force_limit", "drive_joint_force_limit"):
        oracle.upload(name, np.tile(state["q" if name == "q" else name], E))
    oracle.upload("base_pose", np.tile(state["base_pose"], E))
    for w in (oracle, world):
        w.upload("drive_target", target)
        w.upload("link_velocity", twist)
    steps = 20
    world.step(steps); world.synchronize()
    oracle.step(steps)
    assert np.array_equal(world.download("env_status"), oracle.download("env_status")) and not world.download("env_status").any()
    assert np.array_equal(world.download("contact_count"), oracle.download("contact_count"))
    assert world.download("contact_count").max() >= 2
    for name in ("q", "qdot", "base_pose", "link_pose", "actuator_effort"):
        error = relative_error(world.download(name), oracle.download(name))
        assert error <= 5 * TOL, f"{name}: {error:.2e}"        # twenty steps of accumulated rounding
    world.reset(); world.synchronize()
    assert np.allclose(world.download("base_pose").reshape(E, 7), state["base_pose"])
    assert not world.download("q").any() and not world.download("qdot").any()
    assert np.array_equal(world.download("drive_stiffness").reshape(E, -1)[3], state["drive_stiffness"])
    world.close(); oracle.close()


WALKER = os.path.join(ROOT, "tests", "data", "capsule_walker.xml")


def test_capsule_walker_matches_the_oracle(oracle_py, device):
    """A robot file whose links collide with capsules, a cylinder and spheres, with each other and with the floor:
    loaded without the plane-contacts-only relaxation, stepped on the device and by the oracle from the same pushes."""
    E, steps = 128, 12
    scene = nk.Scene(WALKER)
    assert scene.info.dropped_geom_count == 0
    desc = abi.world_desc(E, scene.info.timestep, gravity=tuple(scene.info.gravity), vel_iters=8)
    world, oracle = nk.World(device, scene, desc), oracle_py.OracleWorld(scene, desc, threads=8)
    state = scene.initial_state()
    rng = np.random.default_rng(23)
    nl = scene.link_count
    joint = {name: scene.joint_names.index(name) for name in ("l_hip_x", "r_hip_x", "l_hip_y", "r_hip_y")}
    # the legs swing towards each other, one a little forward and one a little back, so that the thighs meet at an angle
    q, qdot = np.tile(state["q"], (E, 1)), np.zeros((E, nl), np.float32)
    cross, push = rng.uniform(0.05, 0.2, E), rng.uniform(0.0, 2.5, E)
    q[:, joint["l_hip_x"]], q[:, joint["r_hip_x"]] = -cross, cross
    q[:, joint["l_hip_y"]], q[:, joint["r_hip_y"]] = 0.12 + rng.normal(0, 0.02, E), -0.12 + rng.normal(0, 0.02, E)
    qdot[:, joint["l_hip_x"]], qdot[:, joint["r_hip_x"]] = -push, push
    base = np.tile(state["base_pose"], (E, 1))
    base[:, 2] -= rng.uniform(0.03, 0.045, E)                  # the soles at the floor
    for name in ("drive_stiffness", "drive_damping", "drive_force_limit", "drive_joint_force_limit"):
        oracle.upload(name, np.tile(state[name], E))
    for w in (oracle, world):
        w.upload("q", q); w.upload("qdot", qdot); w.upload("drive_target", q); w.upload("base_pose", base)
    world.step(steps); world.synchronize()
    oracle.step(steps)
    assert np.array_equal(world.download("env_status"), oracle.download("env_status")) and not world.download("env_status").any()
    S = world.info.contact_slots_per_env
    count = oracle.download("ucontact_count").reshape(E, S)
    plane_row = 0
    side_a = oracle.download("ucontact_a").reshape(E, S, 4)[:, :, 0]
    link_pairs = (count > 0) & (side_a != plane_row)
    assert link_pairs.any(1).sum() >= E // 4 and ((count > 0) & (side_a == plane_row)).any(1).sum() >= E // 4   # links meet links, soles the floor
    # closest points of two capsules jump where the axes are parallel (legs side by side): environments whose manifolds
    # differ by more than rounding are set aside, the rest has to meet the tolerance
    point_g, point_o = world.download("ucontact_point").reshape(E, S, 4, 3), oracle.download("ucontact_point").reshape(E, S, 4, 3)
    live = np.arange(4)[None, None, :] < count[:, :, None]
    same = ~((np.abs(point_g - point_o).max(3) > 1e-3) & live).any((1, 2))
    same &= (world.download("ucontact_count").reshape(E, S) == count).all(1)
    assert same.mean() >= 0.85, same.mean()
    for name in ("q", "qdot", "base_pose", "link_pose", "actuator_effort"):
        error = relative_error(world.download(name).reshape(E, -1)[same], oracle.download(name).reshape(E, -1)[same])
        assert error <= 5 * TOL, f"{name}: {error:.2e}"        # a dozen steps of accumulated rounding
    # the readout of link against link contacts: asked for, it runs on the current solution
    oracle.op("readout_contact_wrench")
    wrench_g, wrench_o = world.download("link_contact_wrench").reshape(E, nl, 6)[same], oracle.download("link_contact_wrench").reshape(E, nl, 6)[same]
    assert np.abs(wrench_o).max() > 1.0 and relative_error(wrench_g, wrench_o) <= 10 * TOL
    for name in ("contact_side_a_kind", "contact_side_b_kind", "contact_side_a_index", "contact_side_b_index"):
        assert np.array_equal(world.download(name).reshape(E, S)[same], oracle.download(name).reshape(E, S)[same]), name
    world.close(); oracle.close()


LEGGED = os.path.join(ROOT, "tests", "data", "legged.urdf")


def test_urdf_world_matches_the_oracle(oracle_py, device):
    """A URDF walker on the added ground plane: box trunk, cylinder thighs, capsule shins, sphere feet, torque motors
    bounded by the joints' efforts, knee limits and friction.  Environments start at different heights and tilts and
    with different motor commands; the device and the oracle step the same loaded template."""
    E, steps = 96, 16
    with pytest.raises(nk.NukaError) as err:      # cylinder thighs could meet capsule shins and the box trunk: no analytic manifold
        nk.World(device, nk.Scene(LEGGED, nk.SCENE_GROUND_PLANE), abi.world_desc(2, 1.0 / 240.0))
    assert err.value.code == abi.RESULT_NOT_SUPPORTED
    scene = nk.Scene(LEGGED, nk.SCENE_GROUND_PLANE | nk.SCENE_PLANE_CONTACTS_ONLY)     # the links meet the ground, not each other
    assert scene.info.dropped_geom_count == 0
    desc = abi.world_desc(E, 1.0 / 240.0, vel_iters=8)
    world, oracle = nk.World(device, scene, desc), oracle_py.OracleWorld(scene, desc, threads=8)
    state = scene.initial_state()
    rng = np.random.default_rng(31)
    nl = scene.link_count
    tilt = np.array([1, 0, 0, 0]) + rng.normal(0, 0.03, (E, 4))
    base = np.concatenate([rng.normal(0, 0.1, (E, 2)), rng.uniform(0.46, 0.5, (E, 1)), tilt / np.linalg.norm(tilt, axis=1, keepdims=True)], 1).astype(np.float32)
    q = rng.normal(0, 0.15, (E, nl)).astype(np.float32) * (state["drive_force_limit"] >= 0)
    command = (rng.normal(0, 20.0, (E, nl)) * (state["drive_force_limit"] > 0)).astype(np.float32)     # beyond the 30 N m effort now and then
    for name in ("drive_force_limit", "drive_joint_force_limit"):
        oracle.upload(name, np.tile(state[name], E))
    for w in (oracle, world):
        w.upload("q", q); w.upload("base_pose", base); w.upload("drive_target", command)
    assert np.array_equal(world.download("drive_force_limit").reshape(E, nl)[7], state["drive_force_limit"])
    world.step(steps); world.synchronize()
    oracle.step(steps)
    assert np.array_equal(world.download("env_status"), oracle.download("env_status")) and not world.download("env_status").any()
    assert np.array_equal(world.download("contact_count"), oracle.download("contact_count")) and world.download("contact_count").max() >= 2
    assert np.abs(oracle.download("actuator_effort")).max() <= 30.0 + 1e-3 and (oracle.download("actuator_saturated") != 0).any()
    for name in ("q", "qdot", "base_pose", "link_pose", "actuator_effort", "joint_limit_impulse"):
        error = relative_error(world.download(name), oracle.download(name))
        assert error <= 5 * TOL, f"{name}: {error:.2e}"
    world.close(); oracle.close()


def test_scene_with_unsupported_collision_geometry_is_refused(device, tmp_path):
    path = tmp_path / "ellipsoid.xml"
    path.write_text('<mujoco><worldbody><geom type="plane" size="1 1 1"/><body pos="0 0 1"><freejoint/>'
                    '<inertial pos="0 0 0" mass="1" diaginertia="0.01 0.01 0.01"/><geom type="ellipsoid" size="0.05 0.2 0.1"/></body></worldbody></mujoco>')
    strict = nk.Scene(str(path))
    with pytest.raises(nk.NukaError) as err:
        nk.World(device, strict, abi.world_desc(4, 0.005))
    assert err.value.code == abi.RESULT_NOT_SUPPORTED
    relaxed = nk.Scene(str(path), nk.SCENE_PLANE_CONTACTS_ONLY)
    assert relaxed.info.dropped_geom_count == 1
    world = nk.World(device, relaxed, abi.world_desc(4, 0.005))
    world.step(2); world.synchronize()
    assert not world.download("env_status").any()
    world.close()
