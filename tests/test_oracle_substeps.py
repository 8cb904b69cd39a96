"""A step of several substeps in the oracle (nk/pipeline/pipeline.cpp:56-180, ops/readout.cu AccumulateStepKernel),
pinned without any running reference by what the construction fixes: n substeps of dt are n steps of dt / n for the
state, and the outputs of the step are the or, the sum and the time average of those n steps' outputs."""
import copy

import numpy as np
import pytest

from conftest import nk

abi = nk.abi


def limited_quadruped(E):
    cfg = nk.synthetic.config(2, E)
    t = copy.deepcopy(cfg.template)
    for l, link in enumerate(t.links):
        if link["joint_type"] == abi.JOINT_REVOLUTE:
            link["lower"], link["upper"] = float(cfg.nominal_q[l]) - 0.05, float(cfg.nominal_q[l]) + 0.05   # most joints start outside
    return cfg, t


def test_two_substeps_are_two_half_steps(oracle_py):
    E = 24
    cfg, t = limited_quadruped(E)
    whole = oracle_py.OracleWorld(t, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters, substeps=2), threads=8)
    halves = oracle_py.OracleWorld(t, abi.world_desc(E, cfg.dt * 0.5, vel_iters=cfg.vel_iters), threads=8)
    state = cfg.state()
    rng = np.random.default_rng(5)
    wrench = np.zeros((E, t.link_count, 6), np.float32)
    wrench[:, 0, :3] = rng.normal(0, 30.0, (E, 3))                     # a push on the trunk: the dynamics op consumes it
    for w in (whole, halves):
        w.set_state(state)
        w.upload("link_wrench", wrench)
        w.op("readout_contact_wrench")                                 # a consumer asks for the contact wrenches before stepping
    whole.step(1)
    limit, status, impulse, moment = np.zeros(E * t.link_count * 2), np.zeros(E, np.uint32), 0.0, 0.0
    half = np.float32(cfg.dt * 0.5)
    for _ in range(2):
        halves.step(1)
        limit = limit + halves.download("joint_limit_impulse").astype(np.float64)
        status |= halves.download("env_status")
        w6 = halves.download("link_contact_wrench").reshape(E, -1, 6).astype(np.float64)
        origin = halves.download("link_pose").reshape(E, -1, 7)[:, :, :3].astype(np.float64)
        impulse = impulse + w6[:, :, :3] * half
        moment = moment + w6[:, :, 3:] * half + np.cross(origin, w6[:, :, :3] * half)
    for name in ("q", "qdot", "base_pose", "link_pose", "link_velocity", "lambda", "contact_count"):
        assert np.array_equal(whole.download(name), halves.download(name)), name
    assert np.abs(limit).max() > 1e-3 and np.allclose(whole.download("joint_limit_impulse"), limit, rtol=1e-6, atol=1e-7)
    assert np.array_equal(whole.download("env_status"), status)
    got = whole.download("link_contact_wrench").reshape(E, -1, 6)
    force = impulse / cfg.dt
    torque = (moment - np.cross(origin, impulse)) / cfg.dt
    assert np.abs(force).max() > 1.0
    assert np.allclose(got[:, :, :3], force, rtol=1e-5, atol=1e-4) and np.allclose(got[:, :, 3:], torque, rtol=1e-5, atol=1e-4)
    # articulation.cu:600: the first dynamics op that integrates clears the applied wrench, in either world
    assert not whole.download("link_wrench").any() and not halves.download("link_wrench").any()
    whole.close(); halves.close()


def test_one_substep_is_the_plain_step(oracle_py):
    E = 8
    cfg = nk.synthetic.config(3, E)
    plain = oracle_py.OracleWorld(cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters), threads=8)
    one = oracle_py.OracleWorld(cfg.template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters, substeps=1), threads=8)
    state = cfg.state()
    for w in (plain, one):
        w.set_state(state)
        w.step(2)
    for name in ("q", "qdot", "base_pose", "lambda"):
        assert np.array_equal(plain.download(name), one.download(name)), name
    plain.close(); one.close()
