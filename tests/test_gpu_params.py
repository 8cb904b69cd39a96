"""The tunable parameters of a world (nuka_world_set_param and its shorthands), the pose refresh without a step, the
state hash and checkpoint equality, through the C ABI on an MI355X.

A parameter written into a live world has to act exactly as the same value cooked into the template: the device world
gets its values through nuka_world_set_param, the oracle world is created from a template (and a world description)
that holds them from the start.  fp32 fields to norm-wise relative error 1e-4 a step, as in test_gpu_parity."""
import copy
import ctypes as C

import numpy as np
import pytest

from conftest import nk, relative_error

pytestmark = pytest.mark.gpu
abi = nk.abi
TOL = 1e-4
DRIVE_FIELDS = ("drive_target", "drive_stiffness", "drive_damping", "drive_force_limit")


def driven_template(cfg):
    t = copy.deepcopy(cfg.template)
    t.drive_rows, t.drive_mode = True, abi.DRIVE_PD_POSITION
    for l, link in enumerate(t.links):
        if link["joint_type"] == abi.JOINT_REVOLUTE and l % 2 == 0:
            link["frictionloss"] = 0.1
    return t


@pytest.mark.parametrize("graph", [False, True])
def test_live_parameters_act_as_cooked_ones(oracle_py, device, graph):
    E, steps = 128, 4
    cfg = nk.synthetic.config(2, E)
    t = driven_template(cfg)
    nl = t.link_count
    revolute = [l for l, link in enumerate(t.links) if link["joint_type"] == abi.JOINT_REVOLUTE]
    mass_link, damping_link, armature_link, friction_link, gain_link, limit_link = 0, revolute[1], revolute[2], revolute[4], revolute[5], revolute[7]
    changes = dict(mass=2.5 * t.links[mass_link]["mass"], damping=0.7, armature=0.05, frictionloss=0.3, gain=55.0, limit=12.0, gravity_z=-3.7, iterations=6)
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    world = nk.World(device, t, desc)
    rng = np.random.default_rng(41)
    gains = dict(drive_target=cfg.nominal_q[None, :] + rng.normal(0, 0.2, (E, nl)), drive_stiffness=rng.uniform(20, 80, (E, nl)),
                 drive_damping=rng.uniform(0.5, 3, (E, nl)), drive_force_limit=rng.uniform(5, 30, (E, nl)))
    state = cfg.state()
    world.set_state(state)
    for name in DRIVE_FIELDS:
        world.upload(name, gains[name].astype(np.float32))
    if graph:
        world.set_execution_mode(True)                      # the captured graph has to follow the changed options
        world.step(1); world.reset(); world.set_state(state)
        for name in DRIVE_FIELDS:
            world.upload(name, gains[name].astype(np.float32))
    world.set_link_mass(mass_link, changes["mass"])
    world.set_param("joint_damping", damping_link, changes["damping"])
    world.set_param("joint_armature", armature_link, changes["armature"])
    world.set_param("joint_frictionloss", friction_link, changes["frictionloss"])
    world.set_param("drive_stiffness", gain_link, changes["gain"])
    world.set_param("drive_force_limit", limit_link, changes["limit"])
    world.set_gravity_z(changes["gravity_z"])
    world.set_param("velocity_iterations", 0, changes["iterations"])
    # read back
    assert world.get_param("link_mass", mass_link) == pytest.approx(changes["mass"], rel=1e-6)
    assert world.get_param("joint_damping", damping_link) == pytest.approx(0.7) and world.get_param("joint_armature", armature_link) == pytest.approx(0.05)
    assert world.get_param("joint_frictionloss", friction_link) == pytest.approx(0.3) and world.get_param("drive_stiffness", gain_link) == 55.0
    assert world.get_param("drive_force_limit", limit_link) == 12.0 and world.get_param("gravity_z") == pytest.approx(-3.7)
    assert world.get_param("velocity_iterations") == 6.0

    cooked = copy.deepcopy(t)
    cooked.links[mass_link]["mass"] = changes["mass"]
    cooked.links[damping_link]["damping"] = changes["damping"]
    cooked.links[armature_link]["armature"] = changes["armature"]
    cooked.links[friction_link]["frictionloss"] = changes["frictionloss"]
    oracle = oracle_py.OracleWorld(cooked, abi.world_desc(E, cfg.dt, gravity=(0.0, 0.0, changes["gravity_z"]), vel_iters=changes["iterations"]), threads=8)
    oracle.set_state(state)
    gains["drive_stiffness"][:, gain_link] = changes["gain"]
    gains["drive_damping"][:, gain_link] = 2.0 * np.sqrt(np.float32(changes["gain"]))     # the damping the cook derives from a gain
    gains["drive_force_limit"][:, limit_link] = changes["limit"]
    for name in DRIVE_FIELDS:
        oracle.upload(name, gains[name].astype(np.float32))
    for name in ("drive_stiffness", "drive_damping", "drive_force_limit"):
        assert np.array_equal(world.download(name), oracle.download(name)), name

    world.step(steps); world.synchronize()
    oracle.step(steps)
    assert np.array_equal(world.download("env_status"), oracle.download("env_status")) and not world.download("env_status").any()
    assert np.array_equal(world.download("contact_count"), oracle.download("contact_count"))
    for name in ("q", "qdot", "base_pose", "link_pose", "actuator_effort"):
        error = relative_error(world.download(name), oracle.download(name))
        assert error <= steps * TOL, f"{name}: {error:.2e}"
    # the values are the world's from now on: a reset returns the state, not the parameters
    world.reset(); world.synchronize()
    assert world.get_param("link_mass", mass_link) == pytest.approx(changes["mass"], rel=1e-6)
    assert np.all(world.download("drive_stiffness").reshape(E, nl)[:, gain_link] == np.float32(55.0))
    assert world.download("link_inertia").reshape(nl, 6, 6)[mass_link, 3, 3] == np.float32(changes["mass"])
    assert world.download("joint_damping")[damping_link] == np.float32(0.7)
    world.close(); oracle.close()


def test_parameter_registry_and_refusals(device):
    cfg = nk.synthetic.config(3, 8)
    plain = nk.World(device, cfg.template, abi.world_desc(8, cfg.dt, vel_iters=cfg.vel_iters))
    infos = plain.param_infos()
    assert [i["key"] for i in infos] == list(nk.PARAMS)
    assert [i["count"] for i in infos] == [1, 1] + [cfg.template.link_count] * 6
    assert [i["unit"] for i in infos][:3] == ["m/s^2", "", "kg"] and infos[3]["scene_field"] == "joint.damping"
    assert infos[1]["type"] == 1 and infos[1]["min"] == 1.0 and infos[1]["max"] == 65535.0 and infos[0]["max"] == 1000.0
    assert infos[5]["tier"] == nk.PARAM_REBUILD and all(i["tier"] == nk.PARAM_LIVE for k, i in enumerate(infos) if k != 5)
    joint = next(l for l, link in enumerate(cfg.template.links) if link["joint_type"] == abi.JOINT_REVOLUTE)

    def refused(code, *args):
        with pytest.raises(nk.NukaError) as err:
            plain.set_param(*args)
        assert err.value.code == code, (args, err.value.code)

    refused(abi.RESULT_NOT_SUPPORTED, "joint_frictionloss", joint, 0.2)      # no friction rows were cooked
    refused(abi.RESULT_NOT_SUPPORTED, "joint_damping", 0, 0.2)               # the floating root has no joint record
    refused(abi.RESULT_NOT_SUPPORTED, "drive_stiffness", joint, 10.0)        # no drive rows in this world
    refused(abi.RESULT_INVALID_ARG, "link_mass", 1, 0.0)
    refused(abi.RESULT_INVALID_ARG, "link_mass", cfg.template.link_count, 1.0)
    refused(abi.RESULT_INVALID_ARG, "gravity_z", 0, 2000.0)
    refused(abi.RESULT_INVALID_ARG, "gravity_z", 1, -9.0)
    refused(abi.RESULT_INVALID_ARG, "velocity_iterations", 0, 2.5)
    refused(abi.RESULT_INVALID_ARG, "joint_armature", joint, float("nan"))
    refused(abi.RESULT_INVALID_ARG, "joint_damping", joint, -1.0)
    assert nk.lib().nuka_world_set_param(plain._h, 8, 0, 1.0) == abi.RESULT_INVALID_ARG
    assert plain.get_param("gravity_z") == pytest.approx(-9.81) and plain.get_param("link_mass", 1) == pytest.approx(cfg.template.links[1]["mass"])
    plain.close()
    driven = nk.World(device, driven_template(cfg), abi.world_desc(8, cfg.dt, vel_iters=cfg.vel_iters))
    assert driven.param_infos()[5]["tier"] == nk.PARAM_LIVE
    driven.set_param("joint_frictionloss", joint, 0.2)
    driven.close()


def test_pose_refresh_state_hash_and_checkpoint_equality(oracle_py, device):
    E = 64
    cfg = nk.synthetic.config(3, E)
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    world, twin, oracle = nk.World(device, cfg.template, desc), nk.World(device, cfg.template, desc), oracle_py.OracleWorld(cfg.template, desc, threads=8)
    state = cfg.state()
    for w in (world, twin, oracle):
        w.set_state(state)
    # poses follow the coordinates without a step
    world.forward_kinematics(); world.synchronize()
    oracle.op("fk_world_poses"); oracle.op("sync_link_body_pose")
    assert np.abs(world.download("link_pose")).max() > 0.1
    for name in ("link_pose", "body_pose"):
        assert relative_error(world.download(name), oracle.download(name)) <= TOL, name
    assert not world.download("qdot_flat").any()                      # nothing else ran
    twin.forward_kinematics()
    # one build, the same inputs: the same bits
    start = world.state_hash()
    assert start == twin.state_hash() and start != 0
    world.step(3); twin.step(3)
    after = world.state_hash()
    assert after != start and after == twin.state_hash()
    kept = world.checkpoint()
    world.step(2)
    assert world.state_hash() != after
    world.restore(kept); world.synchronize()
    assert world.state_hash() == after
    again = world.checkpoint()
    assert world.checkpoints_equal(kept, again)
    world.step(1)
    moved, other = world.checkpoint(), twin.checkpoint()
    assert not world.checkpoints_equal(kept, moved) and world.checkpoints_equal(kept, other)
    # drive fields and live parameters are state too: a change moves the hash and a restore takes it back
    base = world.checkpoint()
    before = world.state_hash()
    target = world.download("drive_target")
    world.upload("drive_target", target + 0.25)
    assert world.state_hash() != before
    world.restore(base); world.synchronize()
    assert world.state_hash() == before and np.array_equal(world.download("drive_target"), target)
    mass, damping = world.get_param("link_mass", 2), world.get_param("joint_damping", 3)
    world.set_param("link_mass", 2, 2.0 * mass)
    world.set_param("joint_damping", 3, damping + 0.5)
    changed = world.checkpoint()
    assert world.state_hash() != before and not world.checkpoints_equal(base, changed)
    world.restore(base); world.synchronize()
    assert world.get_param("link_mass", 2) == mass and world.get_param("joint_damping", 3) == damping
    assert world.state_hash() == before
    world.step(2)
    twin.restore(twin.checkpoint()); twin.set_state(state); twin.forward_kinematics()
    # a checkpoint of a world that is gone, or of another world, is refused by address and creation number
    stale = twin.checkpoint()
    twin.close()
    fresh = nk.World(device, cfg.template, desc)
    assert nk.lib().nuka_world_checkpoint_restore(fresh._h, stale) == abi.RESULT_INVALID_ARG
    assert nk.lib().nuka_world_checkpoint_restore(world._h, stale) == abi.RESULT_INVALID_ARG
    for handle in (kept, again, moved, other, base, changed, stale):
        nk.lib().nuka_checkpoint_destroy(handle)
    for w in (world, fresh, oracle):
        w.close()


def test_checkpoint_files_and_execution_info(device, tmp_path):
    E = 32
    cfg = nk.synthetic.config(2, E)
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    world, other = nk.World(device, cfg.template, desc), nk.World(device, cfg.template, desc)
    world.set_state(cfg.state())
    info = world.execution_info()
    assert (info.mode, info.graph_ready, info.capture_attempts, info.graph_replays, info.last_result) == (0, 0, 0, 0, 0)
    world.set_execution_mode(True)
    world.step(3); world.synchronize()
    info = world.execution_info()
    assert (info.mode, info.graph_ready, info.capture_attempts, info.graph_replays) == (1, 1, 1, 3)
    world.set_velocity_iterations(5)                       # a changed op sequence: the graph is captured again
    assert world.execution_info().capture_attempts == 2
    # a checkpoint written by one world, read by another of the same layout, continues bit for bit
    kept = world.checkpoint()
    path = tmp_path / "quadruped.ckpt"
    world.write_checkpoint(kept, path)
    size = C.c_uint64()
    nk.lib().nuka_checkpoint_byte_size(kept, C.byref(size))
    live_values = 2 + 6 * cfg.template.link_count            # gravity, sweeps, six per-link parameters
    assert path.stat().st_size == 32 + size.value + 8 * live_values
    read = other.read_checkpoint(path)
    other.restore(read); other.synchronize()               # the live parameters come with it: five sweeps
    assert other.get_param("velocity_iterations") == 5
    assert other.state_hash() == world.state_hash()
    world.restore(kept)                                    # a restore also clears the solver's carried history: both start from it
    world.step(2); other.step(2)
    assert other.state_hash() == world.state_hash() and np.array_equal(other.download("qdot"), world.download("qdot"))
    # files that are no checkpoint of this layout are refused
    bigger = nk.World(device, cfg.template, abi.world_desc(E + 1, cfg.dt))
    for reader, file in ((bigger, path), (other, tmp_path / "absent.ckpt")):
        with pytest.raises(nk.NukaError) as err:
            reader.read_checkpoint(file)
        assert err.value.code == abi.RESULT_INVALID_ARG
    (tmp_path / "short.ckpt").write_bytes(path.read_bytes()[:100])
    (tmp_path / "noise.ckpt").write_bytes(b"x" * 64)
    for name in ("short.ckpt", "noise.ckpt"):
        with pytest.raises(nk.NukaError) as err:
            other.read_checkpoint(tmp_path / name)
        assert err.value.code == abi.RESULT_INVALID_ARG
    for handle in (kept, read):
        nk.lib().nuka_checkpoint_destroy(handle)
    for w in (world, other, bigger):
        w.close()
