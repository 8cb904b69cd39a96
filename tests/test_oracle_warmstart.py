"""Pins of the oracle's contact cache (ContactWarmStart): what it must do by its own definition - seed a persisting
contact with last step's impulse, keep an absent contact for one step and drop it after two, place owners at their
own point and retained entries in the free points - and the profile terms its material key hashes."""
import ctypes as C

import numpy as np

from conftest import nk
from test_oracle_solver import ball, ball_state

abi = nk.abi
F = C.c_float


def step_ops(w, capture=None):
    w.op("fk_world_poses")
    w.op("articulation_dynamics", 1)
    for op in ("sync_link_body_pose", "build_aabbs", "query_pairs", "narrowphase", "assemble_rows"):
        w.op(op)
    w.op("contact_warm_start", 0)
    if capture is not None:
        capture["seed"] = w.download("lambda")
        capture["match"] = w.download("contact_warm_start_counts")
    w.op("block_descent_solve")
    w.op("contact_warm_start", 1)
    w.op("integrate_position")
    w.op("fk_world_poses")
    w.op("fk_link_velocities")
    w.op("sync_link_body_pose")


def test_resting_ball_is_seeded_with_last_steps_impulse(oracle_py):
    mass, radius, dt = 0.7, 0.05, 1.0 / 200.0
    w = oracle_py.OracleWorld(ball(mass, radius), abi.world_desc(1, dt, vel_iters=50))
    w.set_state(ball_state([radius - 1e-4], np.zeros((1, 6))))
    first = {}
    step_ops(w, first)
    assert first["match"].tolist() == [1, 0] and np.all(first["seed"] == 0)          # empty cache: nothing to seed
    solved = w.download("lambda")[0]
    assert abs(solved - mass * 9.81 * dt) < 1e-5
    assert w.download("contact_cache_age")[0] == 0 and w.download("contact_cache_pair")[0] != 0
    assert w.download("contact_cache_lambda")[0] == solved
    second = {}
    step_ops(w, second)
    assert second["match"].tolist() == [1, 1]
    assert second["seed"][0] == solved and np.all(second["seed"][1:3] == 0)        # the normal impulse came back
    assert w.download("vbd_velocity_sweep_count")[0] <= 2
    w.close()


def test_absent_contact_is_kept_one_step_and_dropped_after_two(oracle_py):
    radius, dt = 0.05, 1.0 / 200.0
    for absent_steps, expect_match in ((1, 1), (2, 0)):
        w = oracle_py.OracleWorld(ball(0.7, radius), abi.world_desc(1, dt, vel_iters=50))
        on, off = ball_state([radius - 1e-4], np.zeros((1, 6))), ball_state([radius + 0.5], np.zeros((1, 6)))
        w.set_state(on)
        step_ops(w)
        key = w.download("contact_cache_pair")[0]
        for k in range(absent_steps):
            w.set_state(off)
            step_ops(w)
            live = w.download("contact_cache_pair") != 0
            if k == 0:
                assert live.sum() == 1 and w.download("contact_cache_age")[live][0] == 1      # retained, one step old
                assert w.download("contact_cache_pair")[live][0] == key
            else:
                assert live.sum() == 0
        w.set_state(on)
        capture = {}
        step_ops(w, capture)
        assert capture["match"].tolist() == [1, expect_match]
        assert (capture["seed"][0] > 0) == bool(expect_match)
        w.close()


def test_cache_layout_invariants_over_steps(oracle_py):
    """Tilted boxes with feature-id corners: owners sit at their own point with age 0, everything else is a retained
    entry one step old, no key appears twice, and matched corners are seeded."""
    from test_gpu_properties import box_template
    E = 32
    t = box_template(True)
    g = np.random.default_rng(4)
    quat = np.array([1, 0, 0, 0]) + g.normal(0, 0.04, (E, 4))
    base = np.concatenate([g.normal(0, 0.2, (E, 2)), g.uniform(0.035, 0.05, (E, 1)), quat / np.linalg.norm(quat, axis=1, keepdims=True)], 1)
    zero = np.zeros((E, 1), np.float32)
    state = dict(q=np.concatenate([zero, g.uniform(-0.3, 0.6, (E, 1))], 1).astype(np.float32), qdot=np.zeros((E, 2), np.float32),
                 tau=np.zeros((E, 2), np.float32), base_pose=base.astype(np.float32), root_twist=np.zeros((E, 6), np.float32))
    w = oracle_py.OracleWorld(t, abi.world_desc(E, 1.0 / 200.0, vel_iters=20), threads=4)
    w.set_state(state)
    S = w.download("ucontact_count").size // E
    matched_total = 0
    for step in range(6):
        capture = {}
        step_ops(w, capture)
        matched_total += int(capture["match"].reshape(E, 2)[:, 1].sum())
        pair = w.download("contact_cache_pair").reshape(E, S * 4)
        feature = w.download("contact_cache_feature").reshape(E, S * 4)
        age = w.download("contact_cache_age").reshape(E, S * 4)
        owner = w.download("contact_cache_current_owner").reshape(E, S * 4) != 0
        cur_pair = w.download("ucontact_id_pair").reshape(E, S * 4)
        cur_feature = w.download("ucontact_id_feature").reshape(E, S * 4)
        assert np.array_equal(pair[owner], cur_pair[owner]) and np.array_equal(feature[owner], cur_feature[owner])
        assert np.all(age[owner] == 0) and np.all(age[~owner & (pair != 0)] == 1) and np.all(age[pair == 0] == 0)
        for e in range(E):
            keys = [(int(a), int(b)) for a, b in zip(pair[e], feature[e]) if a != 0]
            assert len(keys) == len(set(keys))
    assert matched_total > E          # box corners keep their feature ids from step to step
    w.close()


def test_material_key_hashes_the_merged_profile_terms(oracle_py, ref_lib):
    """The oracle hashes constants for every merged profile term but friction; they are what the reference's
    MergeContactParams yields for two default-authored profiles (the hash routine itself is device-only code)."""
    out = (F * 17)()
    for mu_a, mu_b in ((0.8, 0.8), (1.0, 0.5)):
        ref_lib.ref_merged_profile(F(mu_a), F(mu_b), out)
        expect = [max(mu_a, mu_b), max(mu_a, mu_b), 0.005, 0.0001, 0.02, 1.0, 0.9, 0.95, 0.001, 0.5, 2.0, 0.0, 0.0, 3.0, -1.0, 0.0, 0.0]
        assert [np.float32(v) for v in out] == [np.float32(v) for v in expect]
    L = oracle_py.lib()
    L.nko_contact_material.restype = C.c_uint64
    a, b = L.nko_contact_material(F(0.8), F(0.8), 2), L.nko_contact_material(F(1.0), F(1.0), 2)
    assert a != b and a != 0 and L.nko_contact_material(F(0.8), F(0.8), 0) != a
