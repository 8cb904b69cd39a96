"""The URDF template loader (host code; runs on the CPU).  Checked against the reference's own importer fixture with
the expectations of its test (tests/import/test_urdf_importer.cpp), and, on a legged file, against the format's
conventions computed independently here (roll-pitch-yaw origins, principal inertia of a full tensor) and against
what the loaded template does in the oracle."""
import os

import numpy as np
import pytest

from conftest import ROOT, nk

abi = nk.abi
ARM = os.path.join(ROOT, "tests", "golden", "urdf", "minimal_arm.urdf")
LEGGED = os.path.join(ROOT, "tests", "data", "legged.urdf")


def rpy_matrix(roll, pitch, yaw):
    cr, sr, cp, sp, cy, sy = np.cos(roll), np.sin(roll), np.cos(pitch), np.sin(pitch), np.cos(yaw), np.sin(yaw)
    rx = np.array([[1, 0, 0], [0, cr, -sr], [0, sr, cr]])
    ry = np.array([[cp, 0, sp], [0, 1, 0], [-sp, 0, cp]])
    rz = np.array([[cy, -sy, 0], [sy, cy, 0], [0, 0, 1]])
    return rz @ ry @ rx


def quat_matrix(q):
    w, x, y, z = q
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


def test_minimal_arm_fixture_of_the_reference():
    """test_urdf_importer.cpp: two bodies named base and link1, masses 1 and 0.5, one revolute joint0 about z with
    limits -3.14 .. 3.14, one box collision shape on the base; the cooked limit flags are 3 and the base inertia 0.1."""
    scene = nk.Scene(ARM, nk.SCENE_FIXED_BASE)
    assert scene.link_names == ["base", "link1"] and scene.joint_names[1] == "joint0"
    a = scene.template_arrays()
    assert list(a["link_mass"]) == [1.0, 0.5]
    assert list(a["joint_type"]) == [abi.JOINT_FIXED, abi.JOINT_REVOLUTE] and list(a["parent_link"]) == [abi.INVALID, 0]
    assert list(a["joint_axis"].reshape(2, 3)[1]) == [0.0, 0.0, 1.0]
    assert a["joint_limit_lower"][1] == np.float32(-3.14) and a["joint_limit_upper"][1] == np.float32(3.14) and a["joint_limit_flags"][1] == 3
    assert np.allclose(a["link_local_pose"].reshape(2, 7)[1], [0, 0, 0.5, 1, 0, 0, 0])
    assert np.allclose(a["link_inertial_frame"].reshape(2, 7)[1, :3], [0, 0, 0.25])
    assert np.allclose(a["link_diag_inertia"].reshape(2, 3)[0], 0.1) and np.allclose(sorted(a["link_diag_inertia"].reshape(2, 3)[1]), [0.01, 0.05, 0.05])
    shapes = [(int(k), list(p[:3])) for k, p in zip(a["shape_kind"], a["shape_params"].reshape(-1, 4)) if k != abi.INVALID]
    assert len(shapes) == 1 and shapes[0][0] == abi.SHAPE_BOX and np.allclose(shapes[0][1], [0.1, 0.1, 0.1])     # half of size 0.2
    floating = nk.Scene(ARM)
    assert floating.info.floating_root == 1 and floating.template_arrays()["joint_type"][0] == abi.JOINT_FLOATING


def test_default_axis_missing_file_and_rejections(tmp_path):
    """The axis defaults to x (test_urdf_importer.cpp DefaultAxisAndProductionRoundtrip); a missing file, a second root,
    a mimic joint, a planar joint and a lower limit above the upper one are errors."""
    text = open(ARM).read()
    path = tmp_path / "axis.urdf"
    path.write_text(text.replace('<axis xyz="0 0 1"/>', "<!-- no authored axis -->"))
    assert list(nk.Scene(str(path)).template_arrays()["joint_axis"].reshape(2, 3)[1]) == [1.0, 0.0, 0.0]
    with pytest.raises(nk.NukaError) as err:
        nk.Scene(str(tmp_path / "nonexistent.urdf"))
    assert err.value.code == abi.RESULT_INVALID_ARG
    for name, old, new in (("root", "</robot>", '<link name="stray"/></robot>'), ("mimic", "<axis", '<mimic joint="joint0"/><axis'),
                           ("planar", 'type="revolute"', 'type="planar"'), ("limits", 'lower="-3.14"', 'lower="4"'),
                           ("parent", '<parent link="base"/>', '<parent link="nowhere"/>')):
        bad = tmp_path / f"{name}.urdf"
        bad.write_text(text.replace(old, new))
        with pytest.raises(nk.NukaError):
            nk.Scene(str(bad))


def test_legged_file_follows_the_format(oracle_py):
    scene = nk.Scene(LEGGED)
    assert scene.link_names == ["trunk", "l_thigh", "r_thigh", "l_shin", "r_shin", "l_foot", "r_foot"]      # parents before children
    a = scene.template_arrays()
    index = {n: i for i, n in enumerate(scene.link_names)}
    assert [int(a["parent_link"][index[n]]) for n in ("l_thigh", "l_shin", "l_foot")] == [0, index["l_thigh"], index["l_shin"]]
    assert list(a["joint_type"]) == [abi.JOINT_FLOATING, 0, 0, 0, 0, abi.JOINT_FIXED, abi.JOINT_FIXED]
    pose = a["link_local_pose"].reshape(-1, 7)
    assert np.allclose(pose[index["l_thigh"], :3], [0, 0.08, -0.05])
    assert np.allclose(quat_matrix(pose[index["l_thigh"], 3:]), rpy_matrix(0.1, 0, 0), atol=1e-6)
    assert np.allclose(a["joint_axis"].reshape(-1, 3)[index["l_shin"]], [0, 1, 0])                     # normalised
    flags, lower, upper = a["joint_limit_flags"], a["joint_limit_lower"], a["joint_limit_upper"]
    assert flags[index["l_thigh"]] == 0 and flags[index["l_shin"]] == 3                                  # a continuous joint has no range
    assert lower[index["r_shin"]] == np.float32(-0.1) and upper[index["r_shin"]] == np.float32(2.0)
    assert a["joint_damping"][index["l_thigh"]] == np.float32(0.2) and a["joint_frictionloss"][index["l_shin"]] == np.float32(0.05)
    state = scene.initial_state()
    assert scene.info.actuator_count == 2 and scene.info.drive_mode == abi.DRIVE_TORQUE
    assert state["drive_force_limit"][index["l_shin"]] == 30.0 and state["drive_force_limit"][index["l_thigh"]] == 0.0
    # the trunk's tensor: principal moments about rotated axes reproduce the authored matrix
    frame, principal = a["link_inertial_frame"].reshape(-1, 7)[0], a["link_diag_inertia"].reshape(-1, 3)[0]
    R = quat_matrix(frame[3:])
    assert np.allclose(R @ np.diag(principal) @ R.T, [[0.05, 0.004, 0], [0.004, 0.07, 0.002], [0, 0.002, 0.04]], atol=1e-7)
    assert np.allclose(frame[:3], [0.01, 0, 0.02])
    # shapes: half sizes, half lengths, their own origins
    owner = [scene.link_names[l] for l in a["body_link"]]
    shapes = {(owner[r], int(a["shape_kind"][r])): (a["shape_params"].reshape(-1, 4)[r], a["body_local"].reshape(-1, 7)[r])
              for r in range(len(owner)) if a["shape_kind"][r] != abi.INVALID}
    assert set(shapes) == {("trunk", abi.SHAPE_BOX), ("l_thigh", abi.SHAPE_CYLINDER), ("r_thigh", abi.SHAPE_CYLINDER), ("l_shin", abi.SHAPE_CAPSULE),
                           ("r_shin", abi.SHAPE_CAPSULE), ("l_foot", abi.SHAPE_SPHERE), ("r_foot", abi.SHAPE_SPHERE)}
    assert np.allclose(shapes[("trunk", abi.SHAPE_BOX)][0][:3], [0.15, 0.1, 0.05])
    assert np.allclose(shapes[("l_thigh", abi.SHAPE_CYLINDER)][0][:2], [0.03, 0.08]) and np.allclose(shapes[("l_thigh", abi.SHAPE_CYLINDER)][1][:3], [0, 0, -0.1])
    assert np.allclose(shapes[("r_shin", abi.SHAPE_CAPSULE)][0][:2], [0.025, 0.08])
    # exclusions: parent and child, the foot welded to the shin (and so the thigh above), and the pair the file names
    excluded = {frozenset((owner[p[0]], owner[p[1]])) for p in a["excluded_pairs"].reshape(-1, 2)}
    assert excluded == {frozenset(p) for p in (("trunk", "l_thigh"), ("trunk", "r_thigh"), ("l_thigh", "l_shin"), ("r_thigh", "r_shin"),
                                               ("l_shin", "l_foot"), ("r_shin", "r_foot"), ("l_thigh", "l_foot"), ("r_thigh", "r_foot"),
                                               ("l_shin", "r_shin"))}
    # the oracle's forward kinematics on the loaded template puts the left foot where the origins chain to
    t = abi.world_desc(1, 1.0 / 240.0)
    w = oracle_py.OracleWorld(scene, t, threads=1)
    q = np.zeros(scene.link_count, np.float32)
    q[index["l_thigh"]], q[index["l_shin"]] = 0.4, 0.7
    w.upload("q", q)
    w.upload("base_pose", np.array([0.1, -0.2, 0.6, 1, 0, 0, 0], np.float32))
    w.op("fk_world_poses")
    foot = w.download("link_pose").reshape(-1, 7)[index["l_foot"], :3]
    rot_y = lambda angle: rpy_matrix(0, angle, 0)
    hip = rpy_matrix(0.1, 0, 0) @ rot_y(0.4)
    expect = np.array([0.1, -0.2, 0.6]) + np.array([0, 0.08, -0.05]) + hip @ (np.array([0, 0, -0.2]) + rot_y(0.7) @ np.array([0, 0, -0.2]))
    assert np.allclose(foot, expect, atol=1e-6)
    w.close()


def test_legged_file_stands_in_the_oracle(oracle_py):
    """A URDF describes the robot only; with the ground-plane flag it has something to stand on.  Set down on its feet
    it stays up: the knees rest on their lower limits, the feet (spheres welded to the shins) carry the weight."""
    assert all(k != abi.SHAPE_PLANE for k in nk.Scene(LEGGED).template_arrays()["shape_kind"])
    scene = nk.Scene(LEGGED, nk.SCENE_GROUND_PLANE)
    a = scene.template_arrays()
    assert a["shape_kind"][0] == abi.SHAPE_PLANE and a["body_role"][0] == abi.ROLE_STATIC
    w = oracle_py.OracleWorld(scene, abi.world_desc(1, 1.0 / 240.0, vel_iters=8), threads=1)
    height = 0.05 + 0.4 + 0.035            # hip below the trunk origin, two leg segments, the foot's radius
    w.upload("base_pose", np.array([0, 0, height + 0.002, 1, 0, 0, 0], np.float32))
    w.step(60)
    assert not w.download("env_status").any() and w.download("contact_count")[0] >= 2
    base = w.download("base_pose")
    assert abs(base[2] - height) < 0.02 and abs(base[3]) > 0.99          # still up, still upright a quarter of a second later
    w.close()
