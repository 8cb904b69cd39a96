"""Pins of the oracle's contact solve.  The iterate path of the block descent has no independent check (the
reference's solver is device-only code): what is pinned here is its fixed point - closed-form impulses of small
scenes, momentum balance, and the Coulomb conditions at convergence."""
import numpy as np
import pytest

from conftest import nk

abi = nk.abi
ROW_WORDS = 26
ACTIVE, CONTACT_NORMAL = 1, 1 << 6
IDENTITY7 = np.array([0, 0, 0, 1, 0, 0, 0], np.float32)


def solve_once(oracle_py, template, desc, state):
    w = oracle_py.OracleWorld(template, desc, threads=4)
    w.set_state(state)
    w.op("fk_world_poses")
    w.op("articulation_dynamics", 1)
    for op in ("sync_link_body_pose", "build_aabbs", "query_pairs", "narrowphase", "assemble_rows"):
        w.op(op)
    E, n, R, nl = desc.env_count, w.dof, w.rows_per_env, template.link_count
    out = dict(n=n, R=R, free=w.download("qdot_flat").reshape(E, -1)[:, :n].astype(np.float64))
    w.op("contact_warm_start", 0)
    w.op("block_descent_solve")
    scalar = [i for i, l in enumerate(template.links) if l["joint_type"] in (abi.JOINT_REVOLUTE, abi.JOINT_PRISMATIC)]
    qdot, twist = w.download("qdot").reshape(E, nl), w.download("link_velocity").reshape(E, nl, 6)[:, 0, :]
    floating = template.links[0]["joint_type"] == abi.JOINT_FLOATING
    out["v"] = np.concatenate(([twist] if floating else []) + [qdot[:, scalar]], 1).astype(np.float64)
    out["M"] = w.download("m").reshape(E, n, n).astype(np.float64)
    out["J"] = (w.download("chain_jacobian").reshape(E, R, -1) + w.download("chain_jacobian_b").reshape(E, R, -1))[:, :, :n].astype(np.float64)
    out["lambda"] = w.download("lambda").reshape(E, R).astype(np.float64)
    out["rows"] = w.download("urows").reshape(E, R, ROW_WORDS)
    out["residual"] = w.download("solver_residual").reshape(E, 4)
    out["status"] = w.download("env_status")
    out["sweeps"] = w.download("vbd_velocity_sweep_count")
    w.close()
    return out


def ball(mass=0.7, radius=0.05, mu=0.5, inertia=None):
    t = abi.Template()
    inertia = 0.4 * mass * radius * radius if inertia is None else inertia
    t.add_link(abi.JOINT_FLOATING, None, mass=mass, diag_inertia=(inertia,) * 3)
    profile = t.add_profile(mu)
    t.add_body(abi.ROLE_STATIC, kind=abi.SHAPE_PLANE, contype=2, conaffinity=1, profile=profile)
    t.add_body(abi.ROLE_LINK_BODY, link=0, contype=0, conaffinity=0)
    t.add_body(abi.ROLE_PROXY, link=0, kind=abi.SHAPE_SPHERE, params=(radius, 0, 0, 0), contype=1, conaffinity=2,
               profile=profile)
    return t


def ball_state(heights, twists):
    E = len(heights)
    base = np.tile(IDENTITY7, (E, 1))
    base[:, 2] = heights
    z = np.zeros((E, 1), np.float32)
    return dict(q=z, qdot=z, tau=z, base_pose=base, root_twist=np.asarray(twists, np.float32))


def test_resting_and_falling_ball_closed_form(oracle_py):
    """One sphere over the plane z = 0.  Touching: the impulse stops the fall, lambda = m (g dt - v_z).  Hovering over
    a gap (beyond the 5e-4 separation band): the speculative row lets it close the gap and no more, v_z' = max(v_z, depth / dt)."""
    mass, radius, dt, g = 0.7, 0.05, 1.0 / 200.0, 9.81
    heights = [radius - 1e-3, radius - 1e-4, radius + 8e-4, radius + 9.5e-4]   # the surface sits 5e-4 proud
    twists = np.zeros((4, 6))
    twists[1, 5] = -0.3
    twists[2, 5] = -0.5
    out = solve_once(oracle_py, ball(mass, radius), abi.world_desc(4, dt, vel_iters=50), ball_state(heights, twists))
    lam, v, rows = out["lambda"], out["v"], out["rows"]
    assert np.all(out["status"] == 0) and np.all(out["residual"] < 2e-5)
    for e in range(4):
        normal = np.nonzero(rows.view(np.uint32)[e, :, 0] & CONTACT_NORMAL)[0]
        assert len(normal) == 1
        r = normal[0]
        free_vz = twists[e, 5] - g * dt
        allowed = rows[e, r, 4] * dt                  # rhs dt: 0 when touching, depth / dt over a gap (negative)
        # side B (the ball) moves along -n = +z: J v = v_z; the row asks J v >= rhs dt
        expect_vz = max(free_vz, allowed)
        assert abs(v[e, 5] - expect_vz) < 2e-5
        assert abs(lam[e, r] - mass * (expect_vz - free_vz)) < 2e-5 * mass
        assert np.abs(v[e, :5]).max() < 1e-6 and abs(lam[e, r + 1]) < 1e-6 and abs(lam[e, r + 2]) < 1e-6
    assert rows[0, 0, 4] == 0 and rows[1, 0, 4] == 0 and rows[2, 0, 4] < 0 and rows[3, 0, 4] < 0
    assert lam[2, 0] > 0 and lam[3, 0] == 0     # the fast one is slowed to the allowance, the slow one is left alone


def test_sliding_and_rolling_ball_coulomb_law(oracle_py):
    """A ball pressed on the plane with sideways speed.  The inverse contact-point mass along a tangent is
    1/m + l^2/I with l the lever from the centre to the contact point (midway between the two surfaces).  Sticking
    needs |lambda_t| = v_t / (1/m + l^2/I) <= mu lambda_n; otherwise it slides with mu lambda_n."""
    mass, radius, dt, g, mu = 0.7, 0.05, 1.0 / 200.0, 9.81, 0.5
    speeds = [0.01, 0.05, 1.0, 3.0]
    twists = np.zeros((4, 6))
    twists[:, 3] = speeds
    out = solve_once(oracle_py, ball(mass, radius, mu), abi.world_desc(4, dt, vel_iters=100),
                     ball_state([radius - 1e-3] * 4, twists))
    lam, v = out["lambda"], out["v"]
    assert np.all(out["residual"] < 2e-5)
    normal = mass * g * dt
    height = radius - 1e-3
    lever = height - 0.5 * (height - radius)
    point_mass = 1.0 / (1.0 / mass + lever * lever / (0.4 * mass * radius * radius))
    for e, speed in enumerate(speeds):
        assert abs(lam[e, 0] - normal) < 2e-5 * mass
        tangent = np.hypot(lam[e, 1], lam[e, 2])
        stick = point_mass * speed
        if stick <= mu * normal:
            assert abs(tangent - stick) < 1e-4 * stick + 1e-7
            point_speed = v[e, 3] - lever * v[e, 1]           # v_x + (omega x r)_x with r = (0, 0, -lever)
            assert abs(point_speed) < 2e-5
        else:
            assert abs(tangent - mu * lam[e, 0]) < 1e-5 * normal and abs(tangent - mu * normal) < 2e-4 * normal
            assert abs(v[e, 3] - (speed - mu * normal / mass)) < 2e-5     # friction opposes the slide
    assert stick > mu * normal and point_mass * speeds[0] < mu * normal     # both regimes were exercised


@pytest.mark.parametrize("index", [2, 3])
def test_converged_solve_satisfies_momentum_balance_and_coulomb_conditions(oracle_py, index):
    E = 32
    cfg = nk.synthetic.config(index, E)
    out = solve_once(oracle_py, cfg.template, abi.world_desc(E, cfg.dt, vel_iters=100), cfg.state())
    lam, v, J, M, rows = out["lambda"], out["v"], out["J"], out["M"], out["rows"]
    assert np.all(out["status"] == 0) and np.all(out["residual"] < 2e-5)
    words = rows.view(np.uint32)
    impulse = np.einsum("eri,er->ei", J, lam)
    balance = np.einsum("eij,ej->ei", M, v - out["free"]) - impulse
    assert np.abs(balance).max() < 2e-5 * np.abs(impulse).max()
    rate = np.einsum("eri,ei->er", J, v)
    tol = 5e-5
    contacts = pressed = sliding = 0
    for e in range(E):
        for r in np.nonzero(words[e, :, 0] & CONTACT_NORMAL)[0]:
            P, mu = words[e, r, 2], rows[e, r, 8]
            ln, lt = lam[e, r], np.array([lam[e, r + P], lam[e, r + 2 * P]])
            gap_rate = rate[e, r] - rows[e, r, 4] * cfg.dt
            vt = np.array([rate[e, r + P], rate[e, r + 2 * P]])
            contacts += 1
            assert ln >= 0 and gap_rate > -tol                        # no pull, no approach beyond the allowance
            assert ln * abs(gap_rate) < tol * max(ln, 1e-3)            # complementarity
            assert np.linalg.norm(lt) <= mu * ln * (1 + 1e-4) + 1e-7   # cone
            if ln > 1e-6:
                pressed += 1
                if np.linalg.norm(lt) < mu * ln * (1 - 1e-3):
                    assert np.linalg.norm(vt) < tol                    # strictly inside the cone: the point sticks
                else:
                    sliding += 1
                    if np.linalg.norm(vt) > 10 * tol:                  # on the cone: friction opposes the slide
                        cosine = lt @ vt / (np.linalg.norm(lt) * np.linalg.norm(vt))
                        assert cosine < -1 + 1e-3
    assert contacts > E and pressed > E // 2


def test_iteration_budget_is_respected_and_reported(oracle_py):
    E = 32
    cfg = nk.synthetic.config(3, E)
    few = solve_once(oracle_py, cfg.template, abi.world_desc(E, cfg.dt, vel_iters=8), cfg.state())
    many = solve_once(oracle_py, cfg.template, abi.world_desc(E, cfg.dt, vel_iters=100), cfg.state())
    assert few["sweeps"].max() == 8 and np.all(few["sweeps"] <= 8)
    early = few["sweeps"] < 8
    assert early.any() and (~early).any()
    # environments that met the tolerance inside the budget are untouched by a larger budget
    assert np.array_equal(few["lambda"][early], many["lambda"][early]) and np.array_equal(few["sweeps"][early], many["sweeps"][early])


@pytest.mark.parametrize("n", [7, 18, 32, 33, 36, 48, 64])
def test_block_factor_follows_the_route_of_its_width(oracle_py, n):
    """Up to 32 coordinates the block is factored L L^T from the first coordinate (block_descent_tile.cuh:1622-1645);
    past them U U^T from the last one (FactorTileColumns :209-252).  Either factor must reproduce the matrix and
    solve the system; which triangle it fills tells the order of elimination."""
    import ctypes as C
    L = oracle_py.lib()
    L.nko_tile_cholesky_solve.restype = C.c_int
    rng = np.random.default_rng(n)
    a = rng.normal(size=(n, n + 5))
    h = (a @ a.T + 0.5 * np.eye(n)).astype(np.float32)
    g = rng.normal(size=n).astype(np.float32)
    factor = np.zeros((n, n), np.float32)
    d = np.zeros(n, np.float32)
    ok = L.nko_tile_cholesky_solve(h.ctypes.data_as(C.c_void_p), C.c_uint32(n), g.ctypes.data_as(C.c_void_p),
                                   factor.ctypes.data_as(C.c_void_p), d.ctypes.data_as(C.c_void_p))
    assert ok == 1
    f = factor.astype(np.float64)
    if n > 32:
        assert np.all(np.tril(f, -1) == 0.0) and np.all(np.diag(f) > 0.0)
    else:
        assert np.all(np.triu(f, 1) == 0.0) and np.all(np.diag(f) > 0.0)
    assert np.abs(f @ f.T - h).max() <= 2e-6 * np.abs(h).max()
    exact = np.linalg.solve(h.astype(np.float64), g.astype(np.float64))
    assert np.abs(d - exact).max() <= 1e-4 * np.abs(exact).max()
    # an indefinite matrix is refused on either route
    h[n // 2, n // 2] = -1.0
    assert L.nko_tile_cholesky_solve(h.ctypes.data_as(C.c_void_p), C.c_uint32(n), g.ctypes.data_as(C.c_void_p),
                                     factor.ctypes.data_as(C.c_void_p), d.ctypes.data_as(C.c_void_p)) == 0
