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


def test_scene_with_unsupported_collision_geometry_is_refused(device, tmp_path):
    path = tmp_path / "capsule.xml"
    path.write_text('<mujoco><worldbody><geom type="plane" size="1 1 1"/><body pos="0 0 1"><freejoint/>'
                    '<geom type="capsule" size="0.05 0.2"/></body></worldbody></mujoco>')
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
