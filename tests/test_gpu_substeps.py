"""Steps of several substeps (nuka_world_desc_t::solver_substeps) through the C ABI on an MI355X: parity with the
oracle, whose substepping is pinned in test_oracle_substeps, and the same construction checked on the device itself -
n substeps of dt are n steps of dt / n, bit for bit.  fp32 fields to norm-wise relative error 1e-4 a substep."""
import copy

import numpy as np
import pytest

from conftest import nk, relative_error

pytestmark = pytest.mark.gpu
abi = nk.abi
TOL = 1e-4


def test_substepped_driven_humanoid_matches_the_oracle(oracle_py, device):
    E, substeps, steps = 96, 3, 2
    cfg = nk.synthetic.config(3, E)
    t = copy.deepcopy(cfg.template)
    t.drive_rows, t.drive_mode = True, abi.DRIVE_PD_POSITION
    for l, link in enumerate(t.links):
        if link["joint_type"] == abi.JOINT_REVOLUTE and l % 3 != 0:
            link["lower"], link["upper"] = float(cfg.nominal_q[l]) - 0.2, float(cfg.nominal_q[l]) + 0.25
    desc = abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters, substeps=substeps)
    world, oracle = nk.World(device, t, desc), oracle_py.OracleWorld(t, desc, threads=8)
    nl = t.link_count
    rng = np.random.default_rng(9)
    gains = dict(drive_target=cfg.nominal_q[None, :] + rng.normal(0, 0.2, (E, nl)), drive_stiffness=rng.uniform(20, 80, (E, nl)),
                 drive_damping=rng.uniform(0.5, 3, (E, nl)))
    state = cfg.state()
    for w in (world, oracle):
        w.set_state(state)
        for name, values in gains.items():
            w.upload(name, values.astype(np.float32))
    world.download("link_contact_wrench")              # a consumer asks for the contact readout: it joins every substep
    oracle.op("readout_contact_wrench")
    assert world.info.op_count > 3 * 15
    world.step(steps); world.synchronize()
    oracle.step(steps)
    assert np.array_equal(world.download("env_status"), oracle.download("env_status")) and not world.download("env_status").any()
    assert np.array_equal(world.download("contact_count"), oracle.download("contact_count"))
    assert np.abs(oracle.download("joint_limit_impulse")).max() > 1e-3 and np.abs(oracle.download("link_contact_wrench")).max() > 1.0
    for name in ("q", "qdot", "base_pose", "link_pose", "actuator_effort", "joint_limit_impulse"):
        error = relative_error(world.download(name), oracle.download(name))
        assert error <= substeps * steps * TOL, f"{name}: {error:.2e}"
    # contact forces of the humanoid after several intervals: the bar of the readout test in test_gpu_drives
    assert relative_error(world.download("link_contact_wrench"), oracle.download("link_contact_wrench")) <= 10 * TOL
    world.close(); oracle.close()


@pytest.mark.parametrize("graph", [False, True])
def test_two_substeps_are_two_half_steps_on_the_device(device, graph):
    E = 512
    cfg = nk.synthetic.config(2, E)
    whole = nk.World(device, cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters, substeps=2))
    halves = nk.World(device, cfg.template, abi.world_desc(E, cfg.dt * 0.5, vel_iters=cfg.vel_iters))
    state = cfg.state()
    for w in (whole, halves):
        w.set_state(state)
        w.set_execution_mode(graph)
    whole.step(2); halves.step(4)
    whole.synchronize(); halves.synchronize()
    assert whole.download("contact_count").max() >= 2
    for name in ("q", "qdot", "base_pose", "link_pose", "link_velocity", "lambda", "contact_count", "env_status"):
        assert np.array_equal(whole.download(name), halves.download(name)), name
    whole.close(); halves.close()


def test_substep_arguments_outside_the_path_are_refused(device):
    cfg = nk.synthetic.config(2, 4)
    shared = abi.world_desc(4, cfg.dt, substeps=2)
    shared.contact_detection_substeps = 2
    for desc, code in ((shared, abi.RESULT_NOT_SUPPORTED), (abi.world_desc(4, cfg.dt, substeps=65), abi.RESULT_INVALID_ARG)):
        with pytest.raises(nk.NukaError) as err:
            nk.World(device, cfg.template, desc)
        assert err.value.code == code
