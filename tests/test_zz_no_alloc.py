"""nuka_world_reset_envs_static, the masked reset that allocates nothing, against nuka_world_reset_envs: two calls in
a row through the C ABI, the second with fewer ids, must leave a world in exactly the state the allocating entry point
leaves its twin in.  Collected last: a failure here must not hide the tests before it."""
import ctypes as C

import numpy as np
import pytest

from conftest import nk

pytestmark = pytest.mark.gpu
FIELDS = ("q", "qdot", "qddot", "tau", "base_pose", "link_pose", "link_velocity", "body_pose", "lambda", "contact_cache_pair",
          "contact_cache_age", "contact_row_extent", "contact_cache_extent", "solver_velocity", "env_status")


def test_static_reset_equals_the_allocating_reset_on_two_calls_in_a_row(device):
    E = 256
    cfg = nk.synthetic.config(2, E)
    desc = nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    lib = nk.lib()
    lib.nuka_world_reset_envs_static.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32]
    lib.nuka_world_reset_envs_static.restype = C.c_int
    worlds = []
    for _ in range(2):
        w = nk.World(device, cfg.template, desc)
        w.set_state(cfg.state())
        w.step(3)
        w.synchronize()
        worlds.append(w)
    plain, static = worlds
    for n in FIELDS:
        assert np.array_equal(plain.download(n), static.download(n)), n
    g = np.random.default_rng(5)
    first = g.integers(0, E, 100).astype(np.uint32)          # with duplicates
    second = np.array([7, 200, 7, 31, 0], np.uint32)         # fewer ids than the call before: stale words stay behind them
    for ids in (first, second):
        assert lib.nuka_world_reset_envs(plain._h, ids.ctypes.data, ids.size) == 0
        assert lib.nuka_world_reset_envs_static(static._h, ids.ctypes.data, ids.size) == 0
        for n in FIELDS:
            assert np.array_equal(plain.download(n), static.download(n)), n
        for w in worlds:                                      # both go on from the reset state
            w.step(2)
            w.synchronize()
        for n in FIELDS:
            assert np.array_equal(plain.download(n), static.download(n)), n
    untouched = np.ones(E, bool)
    untouched[first] = False
    untouched[second] = False
    assert untouched.sum() > 100
    # the edges of the contract: nothing to do, a bad id, too many ids
    before = {n: static.download(n) for n in FIELDS}
    assert lib.nuka_world_reset_envs_static(static._h, None, 0) == 0
    bad = np.array([3, E], np.uint32)
    assert lib.nuka_world_reset_envs_static(static._h, bad.ctypes.data, bad.size) == 1
    many = np.zeros(nk.RESET_ENVS_STATIC_MAX + 1, np.uint32)
    assert lib.nuka_world_reset_envs_static(static._h, many.ctypes.data, many.size) == 1
    assert b"NUKA_RESET_ENVS_STATIC_MAX" in lib.nuka_last_error_message()
    assert lib.nuka_world_reset_envs_static(None, bad.ctypes.data, bad.size) == 2
    for n in FIELDS:
        assert np.array_equal(static.download(n), before[n]), n
    full = np.arange(E, dtype=np.uint32).repeat(nk.RESET_ENVS_STATIC_MAX // E)      # the maximum itself is accepted
    assert full.size == nk.RESET_ENVS_STATIC_MAX
    assert lib.nuka_world_reset_envs_static(static._h, full.ctypes.data, full.size) == 0
    assert lib.nuka_world_reset_envs(plain._h, full.ctypes.data, full.size) == 0
    for n in FIELDS:
        assert np.array_equal(plain.download(n), static.download(n)), n
    for w in worlds:
        w.close()
