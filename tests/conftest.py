import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

nk = entry.load_package()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs through the C ABI of libnuka_hip.so)")


@pytest.fixture(scope="session")
def oracle_py():
    mod = entry.load_oracle()
    mod.build()
    return mod


@pytest.fixture(scope="session")
def ref_lib(oracle_py):
    """The reference's own host headers behind extern "C" (oracle/_ref), when it has been built."""
    import ctypes as C
    if not os.path.exists(oracle_py.REF_PATH):
        pytest.skip("oracle/_ref/libnuka_ref.so not built (reference tree absent)")
    L = C.CDLL(oracle_py.REF_PATH)
    L.ref_cone_argument.restype = C.c_float
    L.ref_momentum_restart.restype = C.c_double
    L.ref_tangent_potential.restype = C.c_double
    L.ref_tangent_potential_change.restype = C.c_float
    L.ref_contact_projection_roundoff.restype = C.c_double
    L.ref_contact_query_reach.restype = C.c_float
    L.ref_contact_motion_radius.restype = C.c_float
    L.ref_rigid_contact_query_margin.restype = C.c_float
    return L


@pytest.fixture(scope="session")
def device():
    dev = nk.Device(0)
    yield dev
    dev.close()


def relative_error(a, b, floor=1e-30):
    """Norm-wise relative error max|a - b| / max|b| over the whole array."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), floor)) if a.size else 0.0


def per_env_error(a, b, env_count, floor=1e-6):
    """Per-environment norm-wise relative error."""
    a = np.asarray(a, np.float64).reshape(env_count, -1)
    b = np.asarray(b, np.float64).reshape(env_count, -1)
    return np.abs(a - b).max(1) / np.maximum(np.abs(b).max(1), floor)


def make_pair(oracle_py, device, index, env_count, **kw):
    cfg = nk.synthetic.config(index, env_count)
    desc = nk.abi.world_desc(env_count, cfg.dt, vel_iters=cfg.vel_iters, **kw)
    oracle = oracle_py.OracleWorld(cfg.template, desc, threads=8)
    world = nk.World(device, cfg.template, desc)
    state = cfg.state()
    oracle.set_state(state)
    world.set_state(state)
    return cfg, oracle, world, state
