"""The oracle's double-precision build (oracle/nko_double.h): the same sources with every scalar a double.  It is the
yardstick of the GPU tests' relaxed bars, so it is checked here for being what it claims: it loads, it computes in
double (its factorisation reconstructs the mass matrix to 1e-13 where the single-precision build stops at 1e-6), and it
is the same algorithm (integer outputs equal the single-precision build's, scalars agree to single-precision rounding)."""
import numpy as np
import pytest

from conftest import nk


@pytest.mark.parametrize("index,E", [(1, 64), (2, 64), (3, 48)])
def test_double_build_is_the_same_algorithm_in_double(oracle_py, index, E):
    cfg = nk.synthetic.config(index, E)
    desc = nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    single = oracle_py.OracleWorld(cfg.template, desc, threads=4)
    double = oracle_py.OracleWorld(cfg.template, desc, threads=4, double=True)
    assert oracle_py.lib64().nko_real_bytes() == 8 and oracle_py.lib().nko_real_bytes() == 4
    for w in (single, double):
        w.set_state(cfg.state())
        w.step()
    assert double.download("q").dtype == np.float64
    n = double.dof
    for w, bound in ((single, 2e-5), (double, 1e-12)):
        M = w.download("m").reshape(E, n, n).astype(np.float64)
        F = w.download("m_factor").reshape(E, n, n).astype(np.float64)
        L = np.tril(F, -1) + np.eye(n)[None]
        D = np.einsum("eii->ei", F)
        rebuilt = np.einsum("eik,ek,ejk->eij", L, D, L)
        error = np.abs(rebuilt - M).max() / np.abs(M).max()
        assert error < bound, (bound, error)
    for name in ("pair_count", "contact_count", "row_count", "env_status", "candidate_pairs") if single.rows_per_env else ():
        assert np.array_equal(single.download(name), double.download(name)), name
    for name, bound in (("link_pose", 1e-5), ("articulation_qdd", 1e-4), ("q", 1e-5)):
        a, b = single.download(name).astype(np.float64).reshape(E, -1), double.download(name).reshape(E, -1)
        error = (np.abs(a - b).max(1) / np.maximum(np.abs(b).max(1), 1e-9)).max()
        assert error < bound, (name, error)
    single.close()
    double.close()
