"""What a caller binds to before it steps a world: version and runtime records, the world's stream and an event on it,
solver options, joint names, the kinematic tree, link bindings and the collision shapes with their poses
(nuka.h:34-40, 292-299, 478-494, 1222-1301).  Names and tree against the scene file itself (ElementTree), poses against
the world's own body pose field, error codes as src/c_abi/world.cpp:1170-1413 returns them."""
import ctypes as C
import os
import xml.etree.ElementTree as ET

import numpy as np
import pytest

from conftest import ROOT, nk

pytestmark = pytest.mark.gpu
abi = nk.abi
BIPED = os.path.join(ROOT, "tests", "data", "biped.xml")
WALKER = os.path.join(ROOT, "tests", "data", "capsule_walker.xml")
INVALID_ARG, NULL_HANDLE, NOT_SUPPORTED = 1, 2, 7
UINT32_MAX = 0xFFFFFFFF


def test_version_and_runtime_records():
    assert nk.version() == (0, 1, 0)                       # src/c_abi/error.cpp:69-72
    info = nk.runtime_info()
    assert info.struct_size == C.sizeof(nk.RuntimeInfoC) and info.schema_version == 1
    assert info.cuda_runtime_version > 0 and info.cuda_driver_version > 0
    unset = nk.RuntimeInfoC()                              # the caller has to say which record it holds
    assert nk.lib().nuka_get_runtime_info(C.byref(unset)) == INVALID_ARG
    assert nk.lib().nuka_get_runtime_info(None) == INVALID_ARG


def test_an_event_on_the_worlds_stream_follows_the_submitted_steps(device):
    hip = C.CDLL("libamdhip64.so")
    E = 256
    cfg = nk.synthetic.config(3, E)
    world = nk.World(device, cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters))
    world.set_state(cfg.state())
    assert world.stream() is not None and world.stream() != 0
    event = C.c_void_p()
    assert hip.hipEventCreate(C.byref(event)) == 0
    world.step(5)
    world.record_event(event.value)
    assert hip.hipEventSynchronize(event) == 0             # returns once the five steps are done
    q = world.download("q")
    world.synchronize()
    assert np.array_equal(q, world.download("q"))         # nothing was still in flight when the event completed
    assert hip.hipEventQuery(event) == 0
    assert nk.lib().nuka_world_record_event(world._h, None) == INVALID_ARG
    assert nk.lib().nuka_world_record_event(None, event) == NULL_HANDLE
    assert nk.lib().nuka_world_get_stream(world._h, None) == INVALID_ARG
    assert hip.hipEventDestroy(event) == 0
    world.close()


def test_solver_options_report_the_files_cone_and_integrator(device, tmp_path):
    scene = nk.Scene(BIPED, nk.SCENE_PLANE_CONTACTS_ONLY)
    world = nk.World(device, scene, abi.world_desc(4, 0.0, gravity=(0.0, 0.0, 0.0), vel_iters=4))
    options = world.solver_options()
    root = ET.parse(BIPED).getroot().find("option")
    cone = (root.get("cone") if root is not None else None) or "pyramidal"
    assert options.cone == {"pyramidal": 0, "elliptic": 1}[cone]
    assert options.impratio == pytest.approx(float((root.get("impratio") if root is not None else None) or 1.0))
    assert options.refsafe == 1
    assert options.integrator in (0, 3)
    world.close(); scene.close()
    # the synthetic humanoid: the native law, an Euler step
    cfg = nk.synthetic.config(3, 2)
    plain = nk.World(device, cfg.template, abi.world_desc(2, cfg.dt, vel_iters=2))
    assert plain.solver_options().integrator == 0
    assert nk.lib().nuka_world_get_solver_options(plain._h, None) == INVALID_ARG
    plain.close()


def file_tree(path):
    """(body name, parent body name or None, joint names) of every body under <worldbody>, in document order."""
    out = []

    def walk(element, parent):
        for body in element.findall("body"):
            joints = [j.get("name") for j in body if j.tag in ("joint", "freejoint")]
            out.append((body.get("name"), parent, joints))
            walk(body, body.get("name"))
    walk(ET.parse(path).getroot().find("worldbody"), None)
    return out


def test_names_tree_and_bindings_of_a_scene_world(device):
    E = 3
    scene = nk.Scene(BIPED, nk.SCENE_PLANE_CONTACTS_ONLY)
    world = nk.World(device, scene, abi.world_desc(E, 0.0, gravity=(0.0, 0.0, 0.0), vel_iters=4))
    nl = world.link_count
    names = [world.dof_name(l) for l in range(nl)]
    # every joint of the file names exactly one link; a body with two hinges is two links, the first of them massless
    authored = [j for _, _, joints in file_tree(BIPED) for j in joints]
    assert sorted(n for n in names if n in authored) == sorted(authored)
    assert names[0] in ("root", "torso")                                # the free joint's child is the root link
    # the same names in every environment's copy of the links, and through the scene handle
    for env in range(E):
        assert [world.dof_name(env * nl + l) for l in range(nl)] == names
    assert [scene.joint_names[l] or scene.link_names[l] for l in range(nl)] == names
    # the tree: a root, then links whose parents come before them; a joint's axis is a unit vector
    root = world.kinematic_link(0)
    assert root.parent_index == UINT32_MAX and root.joint_type == nk.KINEMATIC_ROOT
    assert list(root.local_pose) == [0.0, 0.0, 0.0, 1.0, 0.0, 0.0, 0.0]
    for l in range(1, nl):
        link = world.kinematic_link(l)
        assert link.parent_index < l and link.articulation_index == 0
        assert link.joint_type in (nk.KINEMATIC_FIXED, nk.KINEMATIC_REVOLUTE, nk.KINEMATIC_PRISMATIC)
        assert abs(np.linalg.norm(np.array(link.local_pose[3:])) - 1.0) < 1e-5
        if link.joint_type != nk.KINEMATIC_FIXED:
            assert abs(np.linalg.norm(np.array(link.axis)) - 1.0) < 1e-5
    # the shin hangs off the thigh's last hinge
    knee = names.index("l_knee")
    parent_name = names[world.kinematic_link(knee).parent_index]
    assert parent_name in ("l_hip_x", "l_hip_y")
    # bindings: the root floats; every link's own collidable row, where it has one, points back at the link
    first = world.link_binding(0)
    assert first.is_root == 1 and first.is_floating == 1
    template = scene.template_arrays()
    for l in range(nl):
        binding = world.link_binding(l)
        assert binding.articulation_index == 0 and binding.is_root == (1 if l == 0 else 0)
        if binding.body_index != UINT32_MAX:
            assert template["body_role"][binding.body_index] == 1 and template["body_link"][binding.body_index] == l
    # error behaviour
    L = nk.lib()
    length = C.c_size_t(99)
    assert L.nuka_world_get_dof_name(world._h, E * nl, None, 0, C.byref(length)) == INVALID_ARG and length.value == 0
    small = C.create_string_buffer(2)
    assert L.nuka_world_get_dof_name(world._h, knee, small, 2, C.byref(length)) == INVALID_ARG and length.value == len("l_knee")
    assert L.nuka_world_get_dof_name(None, 0, None, 0, None) == NULL_HANDLE
    assert L.nuka_world_get_kinematic_link(world._h, nl, C.byref(nk.KinematicLinkC())) == INVALID_ARG
    assert L.nuka_world_get_kinematic_link(world._h, 0, None) == INVALID_ARG
    assert L.nuka_world_get_link_binding(world._h, nl, C.byref(nk.LinkBindingC())) == INVALID_ARG
    world.close(); scene.close()
    # a world cooked from arrays has no names to give
    cfg = nk.synthetic.config(2, 2)
    plain = nk.World(device, cfg.template, abi.world_desc(2, cfg.dt, vel_iters=2))
    assert L.nuka_world_get_dof_name(plain._h, 0, None, 0, C.byref(length)) == NOT_SUPPORTED
    assert plain.kinematic_link(1).parent_index == 0
    plain.close()


def test_the_kinematic_records_rebuild_the_worlds_link_poses(device):
    """Forward kinematics from nuka_world_get_kinematic_link alone (local poses, axes, the live coordinates) lands on
    the link poses the device computed: the records are the tree the device steps."""
    from scipy.spatial.transform import Rotation
    E = 2
    scene = nk.Scene(WALKER, 0)
    world = nk.World(device, scene, abi.world_desc(E, 0.0, gravity=(0.0, 0.0, 0.0), vel_iters=4))
    nl = world.link_count
    rng = np.random.default_rng(5)
    q = rng.normal(0.0, 0.3, (E, nl)).astype(np.float32)
    q[:, 0] = 0.0
    world.upload("q", q)
    world.forward_kinematics()
    world.synchronize()
    poses = world.download("link_pose").reshape(E, nl, 7)
    base = world.download("base_pose").reshape(E, 7)

    def rotation(wxyz):
        return Rotation.from_quat([wxyz[1], wxyz[2], wxyz[3], wxyz[0]])
    for env in range(E):
        position = {0: base[env, :3].astype(np.float64)}
        turn = {0: rotation(base[env, 3:])}
        for l in range(1, nl):
            link = world.kinematic_link(l)
            local_p, local_r = np.array(link.local_pose[:3], np.float64), rotation(link.local_pose[3:])
            axis = np.array(link.axis, np.float64)
            joint_p, joint_r = np.zeros(3), Rotation.identity()
            if link.joint_type == nk.KINEMATIC_REVOLUTE:
                joint_r = Rotation.from_rotvec(axis * float(q[env, l]))
            elif link.joint_type == nk.KINEMATIC_PRISMATIC:
                joint_p = axis * float(q[env, l])
            parent = link.parent_index
            position[l] = position[parent] + turn[parent].apply(local_p + local_r.apply(joint_p))
            turn[l] = turn[parent] * local_r * joint_r
            assert np.abs(position[l] - poses[env, l, :3]).max() < 2e-5, (env, l)
            device_turn = rotation(poses[env, l, 3:])
            assert (turn[l].inv() * device_turn).magnitude() < 2e-5, (env, l)
    world.close(); scene.close()


FREE_BOX = os.path.join(ROOT, "tests", "data", "free_box.xml")


@pytest.mark.parametrize("path", [WALKER, FREE_BOX], ids=["walker", "free_box"])
def test_colliders_carry_the_shape_table_and_the_live_poses(device, path):
    E = 4
    scene = nk.Scene(path, 0)
    world = nk.World(device, scene, abi.world_desc(E, 0.0, gravity=(0.0, 0.0, 0.0), vel_iters=4))
    world.step(3)
    world.synchronize()
    template = scene.template_arrays()
    nb = world.info.bodies_per_env
    body_pose = world.download("body_pose").reshape(E, nb, 7)
    for env in (0, E - 1):
        colliders = world.colliders(env)
        assert len(colliders) == nb
        for row, collider in enumerate(colliders):
            assert collider.kind == template["shape_kind"][row]
            assert np.array_equal(np.array(collider.params, np.float32), template["shape_params"].reshape(nb, 4)[row])
            assert collider.is_static == (1 if template["body_role"][row] == 0 else 0)
            # the step left the body poses in line with the link poses: the record's pose is the row's
            assert np.abs(np.array(collider.pose) - body_pose[env, row]).max() < 2e-6, (env, row)
    assert any(c.is_static for c in world.colliders(0)) and not all(c.is_static for c in world.colliders(0))
    L = nk.lib()
    count = C.c_uint32()
    records = (nk.ColliderC * nb)()
    assert L.nuka_world_get_colliders(world._h, 0, None, 0, C.byref(count)) == 0 and count.value == nb
    assert L.nuka_world_get_colliders(world._h, 0, records, nb - 1, C.byref(count)) == INVALID_ARG
    assert L.nuka_world_get_colliders(world._h, E, records, nb, C.byref(count)) == INVALID_ARG
    assert L.nuka_world_get_colliders(world._h, 0, records, nb, None) == INVALID_ARG
    assert L.nuka_world_get_colliders(None, 0, records, nb, C.byref(count)) == NULL_HANDLE
    world.close(); scene.close()


def test_resource_records_add_up_to_the_arena(device):
    """nuka_device_get_resource_info, nuka_world_get_resource_info and the field list (nuka.h:343-371): the fields tile
    the world's one arena without overlap, their sums are the three totals, and the counts are the world's."""
    gpu = device.resource_info()
    assert gpu.total_bytes >= 200 << 30 and 0 < gpu.free_bytes <= gpu.total_bytes      # an MI355X: 288 GB of HBM
    assert gpu.compute_units == 256 and gpu.threads_per_unit >= 1024
    E = 64
    cfg = nk.synthetic.config(3, E)
    before = device.resource_info().free_bytes
    world = nk.World(device, cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters))
    info = world.resource_info()
    assert (info.env_count, info.rows_per_env, info.dofs_per_articulation, info.bodies_per_env, info.particles_per_env) == \
           (E, world.rows_per_env, world.dof, world.info.bodies_per_env, 0)
    assert info.contacts_per_env == world.info.contact_slots_per_env
    fields = world.resource_fields()
    assert len(fields) == nk.lib().nuka_world_resource_field_count(world._h) > 100
    names = [f.name.decode() for f in fields]
    assert len(set(names)) == len(names)
    for expected in ("q", "qdot", "link_pose", "m", "m_factor", "lambda", "urows", "chain_jacobian", "parent_link", "link_inertia"):
        assert expected in names, expected
    # the model's tables come first, then the data; placed ranges do not overlap
    owners = [f.owner for f in fields]
    assert owners == sorted(owners) and set(owners) == {0, 1}
    placed = sorted((f.offset, f.offset + f.bytes) for f in fields if f.bytes)
    assert all(a_end <= b_start for (_, a_end), (b_start, _) in zip(placed, placed[1:]))
    pad = lambda n: (n + 255) & ~255
    assert sum(pad(f.bytes) for f in fields if f.owner == 0) == info.model_bytes
    assert sum(pad(f.bytes) for f in fields if f.owner == 1 and f.arena == 0) == info.persistent_bytes
    assert sum(pad(f.bytes) for f in fields if f.owner == 1 and f.arena == 1) == info.scratch_bytes
    by_name = {f.name.decode(): f for f in fields}
    assert by_name["q"].bytes == E * world.link_count * 4 and by_name["q"].arena == 0      # state a checkpoint keeps
    assert by_name["urows"].arena == 1                                                      # rebuilt every step
    # the arena and its reset copy came out of the device's free memory
    taken = before - device.resource_info().free_bytes
    total = info.model_bytes + info.persistent_bytes + info.scratch_bytes
    assert taken >= total
    L = nk.lib()
    assert L.nuka_world_get_resource_info(world._h, None) == INVALID_ARG
    assert L.nuka_world_get_resource_info(None, C.byref(nk.WorldResourceInfoC())) == NULL_HANDLE
    assert L.nuka_world_resource_field_count(None) == 0
    assert L.nuka_device_get_resource_info(None, C.byref(nk.DeviceResourceInfoC())) == NULL_HANDLE
    world.close()


def test_an_execution_window_times_the_steps_inside_it(device):
    """nuka_world_begin_execution_window / nuka_world_end_execution_window (src/c_abi/world.cpp:961-990): device time
    and graph replays between the two calls, and the make-up of the captured graph."""
    E = 1024
    cfg = nk.synthetic.config(3, E)
    world = nk.World(device, cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters))
    world.set_state(cfg.state())
    world.set_execution_mode(True)
    world.step(3); world.synchronize()                     # the graph is captured
    empty = world.end_execution_window(world.begin_execution_window())
    assert empty.graph_replays == 0 and 0.0 <= empty.gpu_ms < 1.0
    import time
    started = time.perf_counter()
    window = world.begin_execution_window()
    world.step(10)
    inside = world.end_execution_window(window)
    wall_ms = (time.perf_counter() - started) * 1e3
    assert inside.graph_replays == 10
    assert inside.nodes >= 8 and inside.kernels >= 8       # a step is a graph of about a dozen kernels
    assert 10 * 0.2 < inside.gpu_ms < 10 * 20.0            # ten humanoid steps: milliseconds, not microseconds or seconds
    assert inside.gpu_ms <= wall_ms                        # the host waited for the window's end
    eager = nk.World(device, cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters))
    window = eager.begin_execution_window()
    eager.step(2)
    plain = eager.end_execution_window(window)
    assert plain.graph_replays == 0 and plain.nodes == 0 and plain.gpu_ms > 0.0
    L = nk.lib()
    other = world.begin_execution_window()
    assert L.nuka_world_end_execution_window(eager._h, other, C.byref(nk.ExecutionWindowC())) == INVALID_ARG   # another world's window
    world.end_execution_window(other)
    assert L.nuka_world_begin_execution_window(world._h, None) == INVALID_ARG
    assert L.nuka_world_end_execution_window(world._h, None, C.byref(nk.ExecutionWindowC())) == INVALID_ARG
    world.close(); eager.close()
