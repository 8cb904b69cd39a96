"""The MJCF template loader (host code, no GPU): the expectations the reference's own importer tests assert on its
fixtures (tests/golden/mjcf), and MuJoCo's kinematic conventions checked independently on a small biped - body
frames composed straight from the XML with ElementTree, hinges turning about their anchors - against the oracle's
forward kinematics run on the loaded template."""
import os
import xml.etree.ElementTree as ET

import numpy as np
import pytest

from conftest import ROOT, nk

abi = nk.abi
GOLDEN = os.path.join(ROOT, "tests", "golden", "mjcf")
BIPED = os.path.join(ROOT, "tests", "data", "biped.xml")


def quat_mul(a, b):
    return np.array([a[0] * b[0] - a[1] * b[1] - a[2] * b[2] - a[3] * b[3], a[0] * b[1] + a[1] * b[0] + a[2] * b[3] - a[3] * b[2],
                     a[0] * b[2] - a[1] * b[3] + a[2] * b[0] + a[3] * b[1], a[0] * b[3] + a[1] * b[2] - a[2] * b[1] + a[3] * b[0]])


def rotate(q, v):
    u = np.asarray(q[1:], float)
    t = 2.0 * np.cross(u, v)
    return np.asarray(v, float) + q[0] * t + np.cross(u, t)


def test_minimal_arm_bodies_joint_and_shapes():      # test_mjcf_importer.cpp:8-57
    s = nk.Scene(os.path.join(GOLDEN, "minimal_arm.xml"))
    a = s.template_arrays()
    assert s.link_names == ["base", "link1"] and s.joint_names == ["", "joint0"]
    assert list(a["joint_type"]) == [abi.JOINT_FIXED, abi.JOINT_REVOLUTE]       # a jointless root body is static
    assert list(a["link_mass"]) == [1.0, 0.5]
    assert list(a["shape_kind"]) == [abi.SHAPE_BOX, abi.SHAPE_CAPSULE]
    assert np.allclose(a["link_local_pose"].reshape(2, 7)[1], [0, 0, 0.5, 1, 0, 0, 0])
    assert np.allclose(a["link_inertial_frame"].reshape(2, 7)[1, :3], [0, 0, 0.25])
    assert np.allclose(a["shape_params"].reshape(2, 4)[1, :2], [0.05, 0.25])     # capsule radius, half height from fromto


def test_joint_dynamics_respect_defaults_and_overrides():      # test_mjcf_importer.cpp:59-77
    s = nk.Scene(os.path.join(GOLDEN, "mjcf_joint_dynamics.xml"))
    a = s.template_arrays()
    expected = np.array([[0.3, 0.01, 0.075], [10.0, 0.2, 0.4], [100.0, 1.0, 1.0], [0.0, 0.0, 0.0], [4.0, 0.2, 0.4]], np.float32)
    assert s.joint_names[1:] == ["root_defaults", "class_defaults", "explicit_values", "explicit_zero", "partial_override"]
    got = np.stack([a["joint_damping"], a["joint_armature"], a["joint_frictionloss"]], 1)[1:]
    assert np.array_equal(got, expected)


def test_geometry_defaults_and_fromto_preserve_endpoints():      # test_mjcf_importer.cpp:106-131
    s = nk.Scene(os.path.join(GOLDEN, "mjcf_geom_frames.xml"))
    a = s.template_arrays()
    assert list(a["joint_type"]) == [abi.JOINT_FLOATING]
    local, params = a["body_local"].reshape(-1, 7), a["shape_params"].reshape(-1, 4)
    ends = lambda row, z: local[row, :3] + rotate(local[row, 3:], [0, 0, z])
    assert params[0, 0] == np.float32(0.01) and params[0, 1] == pytest.approx(0.2)
    assert np.allclose(ends(0, -params[0, 1]), [-0.2, 0, 0.1], atol=1e-7) and np.allclose(ends(0, params[0, 1]), [0.2, 0, 0.1], atol=1e-7)
    assert params[1, 0] == np.float32(0.02) and params[1, 1] == np.float32(0.15)
    assert np.allclose(ends(1, 0.15), [0.15, 0.3, 0.0], atol=1e-7)            # euler="0 90 0" in degrees
    assert params[2, 0] == np.float32(0.03) and params[2, 1] == pytest.approx(0.25)
    assert np.allclose(ends(2, -0.25), [0, 0, 0], atol=1e-7) and np.allclose(ends(2, 0.25), [0, 0.3, 0.4], atol=1e-7)


def test_inertial_sources():      # test_mjcf_mass_pipeline.cpp:27-60
    s = nk.Scene(os.path.join(GOLDEN, "mjcf_inertial_sources.xml"))
    a = s.template_arrays()
    assert s.link_names == ["empty_wrapper", "explicit_inertial", "geom_only"]
    mass, inertia = a["link_mass"], a["link_diag_inertia"].reshape(3, 3)
    assert mass[0] == 0.0 and not inertia[0].any()
    assert mass[1] == 2.5 and np.array_equal(inertia[1], np.array([0.1, 0.2, 0.3], np.float32))
    assert mass[2] == pytest.approx(24.0, abs=1e-5)
    box = 24.0 / 3.0 * np.array([0.2 ** 2 + 0.3 ** 2, 0.1 ** 2 + 0.3 ** 2, 0.1 ** 2 + 0.2 ** 2])
    frame = a["link_inertial_frame"].reshape(3, 7)[2]
    # the principal moments come back in the order the diagonalisation leaves them, with the rotation that undoes it
    R = np.stack([rotate(frame[3:], e) for e in np.eye(3)], 1)
    assert np.allclose(R @ np.diag(inertia[2]) @ R.T, np.diag(box), atol=1e-5)


def test_rotated_slider_types_axes_and_motors():
    s = nk.Scene(os.path.join(GOLDEN, "rotated_slider.xml"))
    a = s.template_arrays()
    assert s.link_names == ["base", "arm", "slider"] and s.joint_names == ["", "hinge", "slide"]
    assert list(a["joint_type"]) == [abi.JOINT_FIXED, abi.JOINT_REVOLUTE, abi.JOINT_PRISMATIC]
    assert np.allclose(a["link_local_pose"].reshape(3, 7)[2], [0.3, 0, 0, 0.70710678, 0, 0, 0.70710678])
    assert s.info.actuator_count == 2 and s.info.drive_mode == abi.DRIVE_TORQUE
    assert list(s.initial_state()["drive_force_limit"]) == [0.0, 100.0, 100.0]
    assert s.info.timestep == np.float32(0.0001) and list(s.info.gravity) == [0.0, 0.0, 0.0]
    assert not (a["shape_contype"].any() or a["shape_conaffinity"].any()) or s.info.body_count == 3   # geoms with contype 0 carry no collidable rows


# ---- the biped: MuJoCo's conventions, checked independently ----------------------------------------------------
def xml_body_frames(path):
    """World frames of every <body> at q = 0, composed from pos / quat as MuJoCo does (mj_kinematics)."""
    root = ET.parse(path).getroot()
    frames = {}

    def walk(element, position, rotation):
        for body in element.findall("body"):
            p = np.array([float(x) for x in body.get("pos", "0 0 0").split()])
            q = np.array([float(x) for x in body.get("quat", "1 0 0 0").split()])
            q = q / np.linalg.norm(q)
            world_p, world_q = position + rotate(rotation, p), quat_mul(rotation, q)
            frames[body.get("name")] = (world_p, world_q, body)
            walk(body, world_p, world_q)

    walk(root.find("worldbody"), np.zeros(3), np.array([1.0, 0, 0, 0]))
    return frames


def oracle_fk(oracle_py, scene, q=None):
    state = scene.initial_state()
    w = oracle_py.OracleWorld(scene, abi.world_desc(1, 0.005), threads=1)
    w.upload("q", state["q"] if q is None else q)
    w.upload("base_pose", state["base_pose"])
    w.op("fk_world_poses")
    pose = w.download("link_pose").reshape(-1, 7)
    w.close()
    return pose


def test_biped_link_frames_sit_on_the_joint_anchors(oracle_py):
    scene = nk.Scene(BIPED)
    frames = xml_body_frames(BIPED)
    pose = oracle_fk(oracle_py, scene)
    for l, name in enumerate(scene.link_names):
        body_name = name.split("/")[0]
        world_p, world_q, body = frames[body_name]
        joints = body.findall("joint")
        if "/" in name:                       # the massless link of a body's earlier joint sits on that joint's anchor
            anchor = next(j for j in joints if j.get("name") == name.split("/")[1]).get("pos")
        else:                                 # the body's own link sits on its last hinge's anchor
            anchor = joints[-1].get("pos", "0 0 0") if joints else "0 0 0"
        anchor = np.array([float(x) for x in anchor.split()])
        assert np.allclose(pose[l, :3], world_p + rotate(world_q, anchor), atol=2e-6), name
        assert np.allclose(np.abs(pose[l, 3:] @ world_q), 1.0, atol=1e-6), name


def test_biped_hinges_turn_about_their_anchors(oracle_py):
    scene = nk.Scene(BIPED)
    frames = xml_body_frames(BIPED)
    rest = oracle_fk(oracle_py, scene)
    knee = scene.joint_names.index("l_knee")
    foot = scene.link_names.index("l_foot")
    angle = 0.7
    q = np.zeros(scene.link_count, np.float32)
    q[knee] = angle
    turned = oracle_fk(oracle_py, scene, q)
    shin_p, shin_q, shin = frames["l_shin"]
    anchor = shin_p + rotate(shin_q, [0.01, 0, 0.01])
    axis = rotate(shin_q, [0, 1, 0])
    rot = np.concatenate([[np.cos(angle / 2)], np.sin(angle / 2) * axis])
    for link in (knee, foot):                 # every point of the shin and the foot swings about the knee's anchor line
        assert np.allclose(turned[link, :3], anchor + rotate(rot, rest[link, :3] - anchor), atol=2e-6)
    assert np.allclose(turned[: knee], rest[: knee], atol=1e-7)      # nothing above the knee moves


def test_biped_masses_limits_profiles_and_drives():
    scene = nk.Scene(BIPED)
    a, state = scene.template_arrays(), scene.initial_state()
    assert a["link_mass"].sum() == pytest.approx(6 + 2 * (1.5 + 0.3 + 800 * 8 * 0.02 * 0.02 * 0.11), rel=1e-6)
    assert scene.info.floating_root == 1 and scene.info.actuator_count == 6 and scene.info.drive_mode == abi.DRIVE_PD_POSITION
    names = scene.joint_names
    knee, hip_x = names.index("l_knee"), names.index("r_hip_x")
    assert (a["joint_limit_lower"][knee], a["joint_limit_upper"][knee], a["joint_limit_flags"][knee]) == (0.0, np.float32(2.2), 3)
    assert (a["joint_limit_lower"][hip_x], a["joint_limit_upper"][hip_x]) == (np.float32(-0.5), np.float32(0.5))
    assert a["joint_damping"][knee] == np.float32(0.6) and a["joint_frictionloss"][knee] == np.float32(0.05) and a["joint_armature"][knee] == np.float32(0.02)
    assert a["joint_stiffness"][knee] == 1.5 and a["joint_spring_reference"][knee] == np.float32(0.3)
    assert state["drive_stiffness"][knee] == 80.0 and state["drive_damping"][knee] == 3.0
    assert state["drive_force_limit"][knee] == 25.0 and state["drive_force_limit"][names.index("r_knee")] == 90.0 and state["drive_force_limit"][hip_x] == 40.0
    assert np.allclose(state["base_pose"], [0, 0, 0.62, 0.9987503, 0, 0.0499792, 0], atol=1e-6)
    # collidable rows: the floor, one body row a link (its first colliding geom, if any), further geoms as extra rows
    assert list(a["body_role"]) == [0, 1, 1, 1, 1, 1, 2, 1, 1, 1, 1, 2]
    assert list(a["shape_kind"][[0, 1, 5, 6]]) == [abi.SHAPE_PLANE, abi.SHAPE_BOX, abi.SHAPE_SPHERE, abi.SHAPE_SPHERE]
    assert list(a["profile_mu"]) == [np.float32(0.9)] * 2 + [np.float32(0.6)] * 2 and list(a["shape_profile"][[5, 6]]) == [0, 1]
    # a full inertia tensor is diagonalised: R diag(principal) R^T gives the authored tensor back
    thigh = scene.link_names.index("l_thigh")
    frame, principal = a["link_inertial_frame"].reshape(-1, 7)[thigh], a["link_diag_inertia"].reshape(-1, 3)[thigh]
    R = np.stack([rotate(frame[3:], e) for e in np.eye(3)], 1)
    assert np.allclose(R @ np.diag(principal) @ R.T, [[0.012, 0.0005, 0], [0.0005, 0.011, 0.0003], [0, 0.0003, 0.002]], atol=1e-8)
    assert np.allclose(frame[:3], [0, 0, -0.12 + 0.01], atol=1e-7)       # the centre of mass moves with the link frame onto the last anchor


def test_biped_stands_on_its_feet_in_the_oracle(oracle_py):
    scene = nk.Scene(BIPED, nk.SCENE_PLANE_CONTACTS_ONLY)
    state = scene.initial_state()
    w = oracle_py.OracleWorld(scene, abi.world_desc(2, 0.005, vel_iters=8), threads=2)
    for name, values in (("q", state["q"]), ("drive_target", state["q"]), ("drive_stiffness", state["drive_stiffness"]),
                         ("drive_damping", state["drive_damping"]), ("drive_force_limit", state["drive_force_limit"])):
        w.upload(name, np.tile(values, 2))
    w.upload("base_pose", np.tile(state["base_pose"], 2))
    w.step(100)
    assert not w.download("env_status").any()
    base = w.download("base_pose").reshape(2, 7)
    assert 0.45 < base[0, 2] < 0.65                       # it settled onto its feet and the servos hold it up
    assert np.array_equal(base[0], base[1])               # identical environments stay identical
    assert w.download("contact_count")[0] >= 2
    w.close()


WALKER = os.path.join(ROOT, "tests", "data", "capsule_walker.xml")


def test_capsule_walker_links_meet_each_other_but_not_their_parents(oracle_py, tmp_path):
    """Capsule, cylinder and sphere geoms become collidable rows; a body never pairs with its parent body (through the
    massless links of a two-joint hip too), nor with a body welded to it, nor with one an <exclude> names - the
    reference's cook-time policy (src/scene/cooker.cpp:470-538), which is MuJoCo's."""
    scene = nk.Scene(WALKER)
    a = scene.template_arrays()
    owner = [scene.link_names[l] if l < scene.link_count else "world" for l in a["body_link"]]
    kinds = {(owner[r], int(k)) for r, k in enumerate(a["shape_kind"]) if k != abi.INVALID}
    assert kinds == {("world", abi.SHAPE_PLANE), ("torso", abi.SHAPE_CAPSULE), ("torso", abi.SHAPE_CYLINDER), ("l_thigh", abi.SHAPE_CAPSULE),
                     ("l_shin", abi.SHAPE_CAPSULE), ("l_foot", abi.SHAPE_SPHERE), ("r_thigh", abi.SHAPE_CAPSULE), ("r_shin", abi.SHAPE_CAPSULE),
                     ("r_foot", abi.SHAPE_SPHERE)}
    trunk = a["shape_params"].reshape(-1, 4)[owner.index("torso")]
    assert np.allclose(trunk[:2], [0.07, 0.12])                                     # radius, half length of the fromto segment
    excluded = {frozenset((owner[p[0]], owner[p[1]])) for p in a["excluded_pairs"].reshape(-1, 2)}
    assert excluded == {frozenset(p) for p in (("torso", "l_thigh"), ("torso", "r_thigh"), ("l_thigh", "l_shin"), ("r_thigh", "r_shin"),
                                               ("l_shin", "l_foot"), ("r_shin", "r_foot"), ("l_thigh", "l_foot"), ("r_thigh", "r_foot"),
                                               ("torso", "l_shin"), ("torso", "r_shin"))}
    # it stands on its soles; crossing the legs makes the thighs meet each other (capsule against capsule)
    state = scene.initial_state()
    w = oracle_py.OracleWorld(scene, abi.world_desc(2, scene.info.timestep, vel_iters=8), threads=2)
    for name in ("q", "drive_stiffness", "drive_damping", "drive_force_limit", "drive_joint_force_limit"):
        w.upload(name, np.tile(state[name], 2))
    w.upload("base_pose", np.tile(state["base_pose"], 2))
    w.upload("drive_target", np.tile(state["q"], 2))
    w.step(80)
    assert not w.download("env_status").any() and w.download("contact_count")[0] == 2
    assert 0.5 < w.download("base_pose").reshape(2, 7)[0, 2] < 0.6
    q = w.download("q").reshape(2, -1).copy()
    q[1, scene.joint_names.index("l_hip_x")], q[1, scene.joint_names.index("r_hip_x")] = -0.35, 0.35
    w.upload("q", q)
    w.step(1)
    a_rows, b_rows = w.download("ucontact_a").reshape(2, -1, 4)[:, :, 0], w.download("ucontact_b").reshape(2, -1, 4)[:, :, 0]
    live = w.download("ucontact_count").reshape(2, -1) > 0
    met = {frozenset((owner[x], owner[y])) for x, y in zip(a_rows[1][live[1]], b_rows[1][live[1]])}
    assert frozenset(("l_thigh", "r_thigh")) in met or frozenset(("l_shin", "r_shin")) in met
    assert all("world" in pair for pair in ({frozenset((owner[x], owner[y])) for x, y in zip(a_rows[0][live[0]], b_rows[0][live[0]])}))
    w.close()


def test_inertia_and_friction_fixture_of_the_reference():
    """tests/data/inertia_friction.xml with the expectations of tests/import/test_inertia_friction.cpp: a full inertia
    tensor comes back from its principal moments and axes, the centre of mass is kept, frictionloss / damping /
    armature inherit from the class and an element's own attribute wins."""
    scene = nk.Scene(os.path.join(GOLDEN, "inertia_friction.xml"))
    a = scene.template_arrays()
    link1, link2 = scene.link_names.index("link1"), scene.link_names.index("link2")
    frame, principal = a["link_inertial_frame"].reshape(-1, 7)[link1], a["link_diag_inertia"].reshape(-1, 3)[link1]
    R = np.stack([rotate(frame[3:], e) for e in np.eye(3)], 1)
    full = R @ np.diag(principal) @ R.T
    assert np.allclose(full, [[2, 0.5, 0.3], [0.5, 3, 0.2], [0.3, 0.2, 4]], atol=1e-4)
    assert np.abs(R - np.eye(3)).max() > 1e-3 and abs(frame[2] - 0.1) < 1e-6            # rotated principal axes, the authored z of the centre
    assert a["link_mass"][link1] == 1.5
    assert np.isclose(a["joint_frictionloss"][link1], 0.075) and np.isclose(a["joint_damping"][link1], 0.3) and np.isclose(a["joint_armature"][link1], 0.01)
    assert np.isclose(a["joint_frictionloss"][link2], 0.02) and np.isclose(a["joint_damping"][link2], 0.3)
    kinds = [int(k) for k in a["shape_kind"] if k != abi.INVALID]
    assert kinds == [abi.SHAPE_BOX, abi.SHAPE_CAPSULE, abi.SHAPE_CAPSULE]
    assert np.allclose(a["shape_params"].reshape(-1, 4)[1, :2], [0.02, 0.05])


def test_contact_filtering_fixture_of_the_reference():
    """tests/data/contact_filtering.xml with the expectations of tests/import/test_mjcf_contact_filtering.cpp that bear
    on pairing: explicit and class-inherited contype / conaffinity / group, the geom that collides with nothing, the
    friction kept from a geom's first coefficient, the body pair excluded and the unknown body name skipped.  Its two
    jointless bodies both sit under <worldbody>: they hang off one static world link."""
    scene = nk.Scene(os.path.join(GOLDEN, "contact_filtering.xml"))
    assert scene.link_names == ["world", "b1", "b2"]
    a = scene.template_arrays()
    assert list(a["joint_type"]) == [abi.JOINT_FIXED] * 3 and list(a["parent_link"]) == [abi.INVALID, 0, 0]
    owner = [scene.link_names[l] for l in a["body_link"]]
    rows = [(owner[r], int(a["shape_kind"][r]), int(a["shape_contype"][r]), int(a["shape_conaffinity"][r]), int(a["shape_group"][r]))
            for r in range(len(owner)) if a["shape_kind"][r] != abi.INVALID]
    assert rows == [("b1", abi.SHAPE_BOX, 2, 4, 3),         # g_explicit
                    ("b1", abi.SHAPE_SPHERE, 1, 1, 0),      # g_default; g_visual (contype 0, conaffinity 0) has no row
                    ("b2", abi.SHAPE_BOX, 8, 1, 0),         # g_class inherits contype 8
                    ("b2", abi.SHAPE_BOX, 10, 1, 0)]        # g_class_override: its own contype wins
    explicit = [r for r in range(len(owner)) if a["shape_kind"][r] != abi.INVALID][0]
    assert a["profile_mu"].reshape(-1, 2)[a["shape_profile"][explicit]][0] == np.float32(0.7)
    # every geom is MuJoCo-sourced (mjcf_importer.cpp:790) and carries its solref, solimp, margin and gap; a class's
    # solref reaches the geoms of the class, and an unauthored geom has the defaults
    law, solref = a["profile_law"], a["profile_solref"].reshape(-1, 2)
    solimp, margin = a["profile_solimp"].reshape(-1, 5), a["profile_margin"].reshape(-1, 2)
    assert (law == abi.LAW_MUJOCO).all()
    p_explicit, p_default, p_class = (a["shape_profile"][explicit + k] for k in range(3))
    assert np.array_equal(solref[p_explicit], np.float32([0.01, 0.8])) and np.array_equal(solimp[p_explicit], np.float32([0.8, 0.9, 0.002, 0.4, 3]))
    assert np.array_equal(margin[p_explicit], np.float32([0.01, 0.005]))
    assert np.array_equal(solref[p_default], np.float32([0.02, 1.0])) and np.array_equal(solimp[p_default], np.float32([0.9, 0.95, 0.001, 0.5, 2]))
    assert np.array_equal(margin[p_default], np.float32([0, 0])) and a["profile_mu"].reshape(-1, 2)[p_default][0] == 1.0
    assert np.array_equal(solref[p_class], np.float32([0.005, 0.5])) and a["shape_profile"][explicit + 3] == p_class
    assert a["contact_cone"] == abi.CONE_PYRAMIDAL and a["contact_impratio"] == 1.0
    assert (a["profile_priority"][p_explicit], a["profile_solmix"][p_explicit], a["profile_condim"][p_explicit]) == (5, np.float32(0.5), 1)
    assert (a["profile_priority"][p_default], a["profile_solmix"][p_default], a["profile_condim"][p_default]) == (0, 1.0, 3)
    # with the native law kept, only an authored friction makes a profile
    native = nk.Scene(os.path.join(GOLDEN, "contact_filtering.xml"), nk.SCENE_NATIVE_CONTACT_LAW).template_arrays()
    assert native["shape_profile"][explicit + 1] == abi.INVALID and (native["profile_law"] == abi.LAW_NATIVE).all()
    excluded = {frozenset((owner[p[0]], owner[p[1]])) for p in a["excluded_pairs"].reshape(-1, 2)}
    assert excluded == {frozenset(("b1", "b2"))}


def test_errors(tmp_path):
    with pytest.raises(nk.NukaError) as err:
        nk.Scene(str(tmp_path / "nonexistent.xml"))
    assert err.value.code == abi.RESULT_INVALID_ARG and "failed to load" in str(err.value)
    cases = {
        "ball": '<mujoco><worldbody><body><joint type="ball"/><inertial mass="1" pos="0 0 0" diaginertia="1 1 1"/></body></worldbody></mujoco>',
        "two": '<mujoco><worldbody><body name="a"><freejoint/></body><body name="b"><freejoint/></body></worldbody></mujoco>',
        "xml": '<mujoco><worldbody><body></worldbody></mujoco>',
        "root": '<robot/>',
    }
    # contact dimensions other than 1 and 3, and negative margins or gaps, are refused as the reference's cook refuses
    # them (scene/cook/cook_to_model.cpp:188-196, nk/model/model.cpp:66), not read as something else
    geom = '<mujoco><worldbody><body><freejoint/><geom type="sphere" size="0.1" %s/></body></worldbody></mujoco>'
    for condim in (0, 2, 4, 6):
        cases[f"condim{condim}"] = geom % f'condim="{condim}"'
    cases["margin"] = geom % 'margin="-0.01"'
    cases["gap"] = geom % 'gap="-0.01"'
    expected = {"margin": "margin and gap", "gap": "margin and gap", **{f"condim{c}": f"condim {c}" for c in (0, 2, 4, 6)}}
    for name, text in cases.items():
        path = tmp_path / f"{name}.xml"
        path.write_text(text)
        with pytest.raises(nk.NukaError) as err:
            nk.Scene(str(path))
        assert err.value.code == abi.RESULT_INVALID_ARG, name
        assert expected.get(name, "") in str(err.value), (name, str(err.value))
    for attributes in ('condim="1"', 'condim="3"', 'margin="0.01" gap="0.002"'):
        path = tmp_path / "accepted.xml"
        path.write_text(geom % attributes)
        assert nk.Scene(str(path)).link_count == 1


def test_joint_law_attributes_and_integrator(tmp_path):
    """mjcf_importer.cpp:334-338, 1193-1213, 1720-1728: every joint is MuJoCo-sourced with its limit margin and the solref /
    solimp of its limit and friction rows (class defaults, then the joint's own; a partial list keeps the rest), the
    scene runs MuJoCo's integrator (Euler unless <option> names implicit or implicitfast; RK4 is refused), and the
    native flag turns both off.  A URDF is native throughout."""
    text = """<mujoco><option integrator="{integrator}"/>
      <default><default class="soft"><joint solreflimit="0.05 0.8" solimplimit="0.8" margin="0.02" solreffriction="0.03"/></default></default>
      <worldbody><body name="a"><inertial mass="1" pos="0 0 0" diaginertia="1 1 1"/>
        <joint name="j0" type="hinge" axis="0 1 0" range="-1 1" class="soft" solimplimit="0.7 0.9"/>
        <body name="b" pos="0 0 1"><inertial mass="1" pos="0 0 0" diaginertia="1 1 1"/>
          <joint name="j1" type="hinge" axis="0 1 0" solimpfriction="0.6 0.7 0.003" frictionloss="0.1"/></body></body></worldbody></mujoco>"""
    default = [0.02, 1.0, 0.9, 0.95, 0.001, 0.5, 2.0]
    for integrator, expect in (("Euler", abi.INTEGRATOR_MUJOCO_EULER), ("implicitfast", abi.INTEGRATOR_MUJOCO_IMPLICIT), ("implicit", abi.INTEGRATOR_MUJOCO_IMPLICIT)):
        path = tmp_path / f"{integrator}.xml"
        path.write_text(text.format(integrator=integrator))
        a = nk.Scene(str(path)).template_arrays()
        assert a["integrator"] == expect and (a["joint_law"] == abi.LAW_MUJOCO).all()
        limit, friction = a["joint_limit_reference"].reshape(-1, 7), a["joint_friction_reference"].reshape(-1, 7)
        j0, j1 = 1, 2                                              # link 0 is the world
        assert np.allclose(limit[j0], [0.05, 0.8, 0.7, 0.9, 0.001, 0.5, 2.0]) and np.isclose(a["joint_limit_margin"][j0], 0.02)
        assert np.allclose(friction[j0], [0.03, 1.0, 0.9, 0.95, 0.001, 0.5, 2.0])
        assert np.allclose(limit[j1], default) and a["joint_limit_margin"][j1] == 0.0
        assert np.allclose(friction[j1], [0.02, 1.0, 0.6, 0.7, 0.003, 0.5, 2.0])
    native = nk.Scene(str(tmp_path / "Euler.xml"), nk.SCENE_NATIVE_JOINT_LAW).template_arrays()
    assert native["integrator"] == abi.INTEGRATOR_NATIVE and (native["joint_law"] == abi.LAW_NATIVE).all()
    plain = tmp_path / "plain.xml"
    plain.write_text(text.replace('<option integrator="{integrator}"/>', ""))
    assert nk.Scene(str(plain)).template_arrays()["integrator"] == abi.INTEGRATOR_MUJOCO_EULER
    rk4 = tmp_path / "rk4.xml"
    rk4.write_text(text.format(integrator="RK4"))
    with pytest.raises(nk.NukaError) as err:
        nk.Scene(str(rk4))
    assert err.value.code == abi.RESULT_INVALID_ARG and "RK4" in str(err.value)   # the scene loader's code for every refusal
    urdf = nk.Scene(os.path.join(ROOT, "tests", "golden", "urdf", "minimal_arm.urdf")).template_arrays()
    assert urdf["integrator"] == abi.INTEGRATOR_NATIVE and (urdf["joint_law"] == abi.LAW_NATIVE).all() and urdf["profile_law"].size == 0 or (urdf["profile_law"] == abi.LAW_NATIVE).all()
