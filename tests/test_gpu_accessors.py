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


def test_colliders_carry_the_shape_table_and_the_live_poses(device):
    E = 4
    scene = nk.Scene(WALKER, 0)
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
