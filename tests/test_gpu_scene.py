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
        # the knee limits' multipliers move by 6.7e-4 in the oracle itself when its inputs move by one unit in the last
        # place (measured on this scenario); they are held to four times that, everything else to 5 TOL
        bound = 4 * 6.7e-4 if name == "joint_limit_impulse" else 5 * TOL
        assert error <= bound, f"{name}: {error:.2e}"
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


def test_reference_entry_point_reads_the_scene_file_named_by_the_descriptor(device, tmp_path):
    """nuka_world_create_from_scene(device, desc, out) with the reference's descriptor layout: the file is read by its
    extension, the world steps exactly as one made from the loaded scene handle with the same options, and the public
    field ids give views with the reference's element strides over the same bytes."""
    import ctypes as C
    E = 64
    ref_desc = abi.SceneWorldDescC()
    ref_desc.scene_path = WALKER.encode()
    ref_desc.env_count, ref_desc.fixed_dt, ref_desc.solver_vel_iters = E, 0.004, 8
    ref_desc.control_mode = abi.DRIVE_PD_POSITION
    world = nk.World(device, None, ref_desc)
    scene = nk.Scene(WALKER, 0)
    twin = nk.World(device, scene, abi.world_desc(E, 0.004, gravity=(0.0, 0.0, -9.81), vel_iters=8))
    rng = np.random.default_rng(3)
    target = rng.normal(0, 0.2, (E, scene.link_count)).astype(np.float32)
    for w in (world, twin):
        w.upload("drive_target", target)
        w.step(5)
        w.synchronize()
    for name in ("q", "qdot", "link_pose", "base_pose", "lambda", "env_status", "contact_count"):
        assert np.array_equal(world.download(name), twin.download(name)), name
    nl = scene.link_count
    for public, (fid, name, stride) in abi.PUBLIC_FIELDS.items():
        view, raw = world.public_view(public)
        assert view.element_stride_bytes == stride, public
        inner = world.download(name)
        assert view.element_count * stride == inner.nbytes and np.array_equal(raw, inner.view(np.uint8)), public
    view, _ = world.public_view("ARTICULATION_LINK_POSE")
    assert view.element_count == E * nl and view.dtype == 0
    view, _ = world.public_view("ENV_STATUS")
    assert view.element_count == E and view.dtype == 1
    # a public id this library does not serve, and the write path through a public id
    out = abi.BufferViewC()
    assert nk.lib().nuka_world_get_buffer_view(world._h, 4, C.byref(out)) == abi.RESULT_NOT_SUPPORTED      # OBSERVATIONS
    q = np.full(E * nl, 0.25, np.float32)
    assert nk.lib().nuka_world_upload_field(world._h, abi.PUBLIC_FIELDS["JOINT_POSITION"][0], q.ctypes.data, q.nbytes, 0) == 0
    assert np.array_equal(world.download("q"), q)
    world.close()
    twin.close()
    # the descriptor's own error contract (src/c_abi/world.cpp:493-527, 60-82)
    handle = C.c_void_p()
    lib = nk.lib()

    def create(**changes):
        d = abi.SceneWorldDescC()
        d.scene_path, d.env_count, d.fixed_dt = WALKER.encode(), 4, 0.004
        for k, v in changes.items():
            setattr(d, k, v)
        code = lib.nuka_world_create_from_scene(device._h, C.byref(d), C.byref(handle))
        if code == 0:
            lib.nuka_world_destroy(handle)
        return code

    assert create() == 0
    assert create(fixed_dt=0.0) == abi.RESULT_INVALID_ARG and create(env_count=0) == abi.RESULT_INVALID_ARG
    assert create(determinism=2) == abi.RESULT_INVALID_ARG and create(control_mode=6) == abi.RESULT_INVALID_ARG
    assert create(scene_path=None) == abi.RESULT_INVALID_ARG
    assert create(control_mode=4) == abi.RESULT_NOT_SUPPORTED and create(instance_count=2) == abi.RESULT_NOT_SUPPORTED
    assert create(contact_family=1) == abi.RESULT_NOT_SUPPORTED and create(terrain_step_height=0.1) == abi.RESULT_NOT_SUPPORTED
    assert create(scene_path=b"/no/such/file.xml") == 4                                     # NUKA_RESULT_FILE_NOT_FOUND
    assert create(scene_path=b"/tmp/robot.usda") == abi.RESULT_NOT_SUPPORTED and create(scene_path=b"/tmp/robot.nks") == abi.RESULT_NOT_SUPPORTED
    broken = tmp_path / "broken.xml"
    broken.write_text("<mujoco><worldbody><body>")
    assert create(scene_path=str(broken).encode()) == 5                                      # NUKA_RESULT_PARSE_ERROR
    assert lib.nuka_world_create_from_scene(None, C.byref(abi.SceneWorldDescC(WALKER.encode(), 4, 0.004)), C.byref(handle)) == abi.RESULT_NULL_HANDLE
