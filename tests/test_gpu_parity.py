"""Parity of the HIP path (through the C ABI of libnuka_hip.so) with the CPU oracle, on an MI355X.

Bars, as used below:
  * integer and index outputs (pairs, counts, row ranges, row flags, contact ids, sweep counts where the solve
    converged, status words): bit-exact;
  * fp32 outputs upstream of the contact solve and the step's resulting poses and velocities: norm-wise relative
    error max|a - b| / max|b| <= 1e-4 (TOL);
  * contact impulses: the generalised impulse J^T lambda and the post-solve velocity to TOL.  The split of that
    impulse over the individual rows of several spheres on one rigid foot is statically indeterminate to first
    order, so a one-ulp change of the inputs moves the oracle's own lambda by more than TOL on the humanoid; the
    per-row lambda is therefore held to max(TOL, 4 x the oracle's own one-ulp sensitivity), the sensitivity being
    measured in the test by running the oracle on inputs moved by one ulp."""
import numpy as np
import pytest

from conftest import make_pair, nk, per_env_error, relative_error

pytestmark = pytest.mark.gpu
TOL = 1e-4
ROW_WORDS = 26
ORACLE_OPS = {"FkWorldPoses": ("fk_world_poses",), "ArticulationDynamics": ("articulation_dynamics", 1),
              "SyncLinkBodyPose": ("sync_link_body_pose",), "BuildAabbs": ("build_aabbs",),
              "LbvhQueryPairs": ("query_pairs",), "NarrowphasePrimitives": ("narrowphase",),
              "AssembleRows": ("assemble_rows",), "BlockDescentSolve": ("block_descent_solve",),
              "IntegratePosition": ("integrate_position",), "FkLinkVelocities": ("fk_link_velocities",)}
UPSTREAM = ["FkWorldPoses", "ArticulationDynamics", "SyncLinkBodyPose", "BuildAabbs", "LbvhQueryPairs",
            "NarrowphasePrimitives", "AssembleRows"]


def both(oracle, world, name):
    oracle.op(*ORACLE_OPS[name])
    world.op(name)
    world.synchronize()


def close(world, oracle, name, tol=TOL):
    """Norm-wise relative error of a field, environment by environment: no environment may hide behind another's
    larger values."""
    E = world.env_count
    got, expect = world.download(name), oracle.download(name)
    if got.size == 0 and expect.size == 0:
        return 0.0
    errors = per_env_error(got, expect, E)
    worst = float(errors.max()) if errors.size else 0.0
    assert worst <= tol, f"{name}: {int((errors > tol).sum())} of {E} environments above {tol:.1e}, worst {worst:.3e}"
    return worst


def close_masked(got, expect, mask, E, tol, what):
    """Per-environment relative error over the entries `mask` selects (leading axis = environment)."""
    got, expect = np.where(mask, got, 0.0).reshape(E, -1), np.where(mask, expect, 0.0).reshape(E, -1)
    errors = per_env_error(got, expect, E)
    assert errors.max() <= tol, f"{what}: {int((errors > tol).sum())} of {E} environments above {tol:.1e}, worst {errors.max():.3e}"


def equal(world, oracle, name):
    assert np.array_equal(world.download(name), oracle.download(name)), f"{name}: integer field differs"


def generalized_impulse(w, E):
    R = w.rows_per_env
    J = w.download("chain_jacobian").reshape(E, R, -1) + w.download("chain_jacobian_b").reshape(E, R, -1)
    return np.einsum("eri,er->ei", J.astype(np.float64), w.download("lambda").reshape(E, R).astype(np.float64))


def oracle_sensitivity(oracle_py, index, E, fields, steps=1, **kw):
    """How far the oracle's own outputs move when q, qdot and tau move by one ulp."""
    cfg = nk.synthetic.config(index, E)
    desc = nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters, **kw)
    outputs = []
    for perturb in (False, True):
        w = oracle_py.OracleWorld(cfg.template, desc, threads=8)
        state = cfg.state()
        if perturb:
            g = np.random.default_rng(99)
            for key in ("q", "qdot", "tau"):
                toward = state[key] + g.choice([-1.0, 1.0], state[key].shape).astype(np.float32)
                state[key] = np.nextafter(state[key], toward).astype(np.float32)
        w.set_state(state)
        w.step(steps)
        outputs.append({f: w.download(f) for f in fields})
        w.close()
    return {f: relative_error(outputs[1][f], outputs[0][f]) for f in fields}


def velocity_scale(world, oracle, E):
    """Per-environment size of the velocities the solve works with: the free velocity it starts from, or the result.
    A body that the contacts bring to rest ends near zero; its error is measured against what the solve removed."""
    free = np.abs(oracle.download("qdot_flat")).reshape(E, -1).max(1)
    return np.maximum(free, 1e-6)


def scaled_errors(got, expect, scale, E):
    return np.abs(np.asarray(got, np.float64).reshape(E, -1) - np.asarray(expect, np.float64).reshape(E, -1)).max(1) / scale


def one_ulp_sensitivity(oracle_py, template, desc, state, threads=8):
    """How far the oracle's own outputs move when q, qdot and tau move by one ulp: the worst environment's relative
    change of the joint accelerations, of the generalized contact impulse and of the post-solve velocity (against the
    free velocity), and the batch-wide relative change of lambda.  An ill-conditioned mass matrix or Newton block
    shows here, and no other fp32 evaluation of the same formulas can be expected to agree more closely than this."""
    E = desc.env_count
    runs = []
    for perturb in (False, True):
        w = oracle_py.OracleWorld(template, desc, threads=threads)
        moved = {k: v.copy() for k, v in state.items()}
        if perturb:
            g = np.random.default_rng(99)
            for key in ("q", "qdot", "tau"):
                toward = moved[key] + g.choice([-1.0, 1.0], moved[key].shape).astype(np.float32)
                moved[key] = np.nextafter(moved[key], toward).astype(np.float32)
        w.set_state(moved)
        for name in UPSTREAM if w.rows_per_env else UPSTREAM[:2]:
            w.op(*ORACLE_OPS[name])
        out = {"qdd": w.download("articulation_qdd").reshape(E, -1).astype(np.float64)}
        if w.rows_per_env:
            out["free"] = np.abs(w.download("qdot_flat")).reshape(E, -1).max(1)
            w.op("block_descent_solve")
            out["impulse"] = generalized_impulse(w, E)
            out["velocity"] = w.download("qdot_flat").reshape(E, -1).astype(np.float64)
            out["lambda"] = w.download("lambda")
        w.op("integrate_position")       # with the push-out of the position pass, a block descent of its own
        out["q"] = w.download("q").reshape(E, -1).astype(np.float64)
        runs.append(out)
        w.close()
    a, b = runs
    sens = {"qdd": float((np.abs(b["qdd"] - a["qdd"]).max(1) / np.maximum(np.abs(a["qdd"]).max(1), 1e-6)).max()),
            "q": float((np.abs(b["q"] - a["q"]).max(1) / np.maximum(np.abs(a["q"]).max(1), 1e-6)).max())}
    if "impulse" in a:
        sens["impulse"] = float((np.abs(b["impulse"] - a["impulse"]).max(1) / np.maximum(np.abs(a["impulse"]).max(1), 1e-9)).max())
        sens["velocity"] = float((np.abs(b["velocity"] - a["velocity"]).max(1) / np.maximum(a["free"], 1e-6)).max())
        sens["lambda"] = relative_error(b["lambda"], a["lambda"])
    return sens


def bar(sens, key):
    """The stated tolerance, or four times the oracle's own one-ulp sensitivity where that is larger."""
    return max(TOL, 4.0 * sens.get(key, 0.0)) if sens else TOL


def acceleration_residual(w, state, E):
    """Backward error of the joint accelerations: |M qdd + bias - tau| against |M||qdd| + |bias| + |tau|, per environment."""
    n = w.dof
    M = w.download("m").reshape(E, n, n).astype(np.float64)
    qdd = w.download("articulation_qdd").reshape(E, -1)[:, :n].astype(np.float64)
    bias = w.download("articulation_bias").reshape(E, -1)[:, :n].astype(np.float64)
    nl = state["tau"].shape[1]
    tau = np.zeros((E, n))
    tau[:, n - (nl - 1):] = state["tau"][:, 1:]          # joint torques follow the root's coordinates
    residual = np.abs(np.einsum("eij,ej->ei", M, qdd) + bias - tau).max(1)
    scale = (np.einsum("eij,ej->ei", np.abs(M), np.abs(qdd)) + np.abs(bias) + np.abs(tau)).max(1)
    return residual / np.maximum(scale, 1e-30)


def compare_ops(oracle, world, E, sens=None, state=None):
    """Every op of one step on both sides, outputs compared after each.  Returns the per-environment errors of the
    solve's outputs (generalized impulse, velocity) for the caller's report."""
    both(oracle, world, "FkWorldPoses")
    close(world, oracle, "link_pose")
    both(oracle, world, "ArticulationDynamics")
    for name in ("m", "articulation_bias"):
        close(world, oracle, name)
    # the accelerations solve M qdd = tau - bias: forward to the bar the oracle's own conditioning allows, and
    # backward (the residual of the device's own solution) to 1e-5 whatever the conditioning
    for name in ("m_factor", "articulation_qdd", "qddot", "qdot", "link_acceleration"):
        close(world, oracle, name, tol=bar(sens, "qdd"))
    if state is not None:
        residual = acceleration_residual(world, state, E)
        assert residual.max() <= 1e-5, f"M qdd + bias - tau: worst environment {residual.max():.2e}"
    report = {}
    if world.rows_per_env:
        R, S = world.rows_per_env, world.info.contact_slots_per_env
        for name in UPSTREAM[2:]:
            both(oracle, world, name)
        close(world, oracle, "body_pose")
        for name in ("pair_count", "ucontact_count", "ucontact_row_range", "contact_row_extent", "row_count",
                     "contact_count", "row_cj_link", "row_cj_link_b"):
            equal(world, oracle, name)
        live = oracle.download("pair_count")
        gp, op = world.download("candidate_pairs").reshape(E, S, 2), oracle.download("candidate_pairs").reshape(E, S, 2)
        assert all(np.array_equal(gp[e, :live[e]], op[e, :live[e]]) for e in range(E))
        points = oracle.download("ucontact_count").reshape(E, S)
        mask = np.arange(4)[None, None, :] < points[:, :, None]
        for name, width in (("ucontact_point", 3), ("ucontact_normal", 3), ("ucontact_depth", 1)):
            g, o = world.download(name).reshape(E, S, 4, width), oracle.download(name).reshape(E, S, 4, width)
            close_masked(g, o, mask[..., None], E, TOL, name)
        for name in ("ucontact_a", "ucontact_b"):
            g, o = world.download(name).reshape(E, S, 4), oracle.download(name).reshape(E, S, 4)
            assert np.array_equal(g[mask], o[mask]), name
        grow, orow = world.download("urows").reshape(E, R, ROW_WORDS), oracle.download("urows").reshape(E, R, ROW_WORDS)
        gw, ow = grow.view(np.uint32), orow.view(np.uint32)
        assert np.array_equal(gw[:, :, 0], ow[:, :, 0])                     # flags of every row, live or not
        active = (ow[:, :, 0] & 1) != 0
        for word in (1, 2, 3, 10, 11, 18, 19):                             # group, env, side kinds and indices
            assert np.array_equal(gw[:, :, word][active], ow[:, :, word][active]), f"row word {word}"
        for lo, hi in ((4, 10), (12, 18), (20, 26)):                       # rhs..mu, both sides' directions
            close_masked(grow[:, :, lo:hi], orow[:, :, lo:hi], active[..., None], E, TOL, f"row words {lo}..{hi}")
        for name in ("chain_jacobian", "chain_jacobian_b"):
            g, o = world.download(name).reshape(E, R, -1), oracle.download(name).reshape(E, R, -1)
            close_masked(g, o, active[..., None], E, TOL, name)
        g, o = world.download("row_penetration").reshape(E, R), oracle.download("row_penetration").reshape(E, R)
        close_masked(g, o, active, E, TOL, "row_penetration")
        close(world, oracle, "qdot_flat", tol=bar(sens, "qdd"))
        scale = velocity_scale(world, oracle, E)
        both(oracle, world, "BlockDescentSolve")
        assert np.array_equal(world.download("env_status"), oracle.download("env_status"))
        impulse_o = generalized_impulse(oracle, E)
        impulse = scaled_errors(generalized_impulse(world, E), impulse_o, np.maximum(np.abs(impulse_o).max(1), 1e-9), E)
        velocity = scaled_errors(world.download("qdot_flat"), oracle.download("qdot_flat"), scale, E)
        report = {"impulse": impulse, "velocity": velocity}
        for what, errors in report.items():
            assert errors.max() <= bar(sens, what), \
                f"{what} after the solve: {int((errors > bar(sens, what)).sum())} of {E} environments above {bar(sens, what):.1e}, worst {errors.max():.3e}"
    for name in ("IntegratePosition", "FkWorldPoses", "FkLinkVelocities"):
        both(oracle, world, name)
    for name in ("q", "base_pose", "link_pose"):
        close(world, oracle, name, tol=bar(sens, "q"))
    return report


@pytest.mark.parametrize("index,E", [(1, 64), (2, 256), (3, 256)])
def test_every_op_matches_the_oracle(oracle_py, device, index, E):
    cfg, oracle, world, state = make_pair(oracle_py, device, index, E)
    desc = nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    sens = one_ulp_sensitivity(oracle_py, cfg.template, desc, state)
    print(cfg.name, "one-ulp sensitivity of the oracle:", {k: f"{v:.2e}" for k, v in sens.items()})
    report = compare_ops(oracle, world, E, sens, state)
    print(cfg.name, "worst environment:", {k: f"{v.max():.2e}" for k, v in report.items()},
          "environments above 1e-4:", {k: int((v > TOL).sum()) for k, v in report.items()})
    close(world, oracle, "link_velocity", tol=bar(sens, "velocity"))
    world.close()
    oracle.close()


@pytest.mark.parametrize("index,E", [(1, 64), (2, 512), (3, 512)])
def test_whole_step_matches_the_oracle(oracle_py, device, index, E):
    cfg, oracle, world, state = make_pair(oracle_py, device, index, E)
    sens = one_ulp_sensitivity(oracle_py, cfg.template, nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters), state)
    world.step()
    world.synchronize()
    oracle.step()
    errors = {n: close(world, oracle, n) for n in ("articulation_qdd", "link_pose", "q", "base_pose", "body_pose")}
    errors.update({n: close(world, oracle, n, tol=bar(sens, "velocity")) for n in ("qdot", "link_velocity")})
    print(cfg.name, "worst environment:", {k: f"{v:.2e}" for k, v in errors.items()})
    if world.rows_per_env:
        assert np.array_equal(world.download("env_status"), oracle.download("env_status"))
        impulse_o = generalized_impulse(oracle, E)
        impulse = scaled_errors(generalized_impulse(world, E), impulse_o, np.maximum(np.abs(impulse_o).max(1), 1e-9), E)
        print(cfg.name, f"J^T lambda: worst environment {impulse.max():.2e}, {int((impulse > TOL).sum())} of {E} above 1e-4; "
              f"the oracle's own one-ulp sensitivity {sens['impulse']:.2e}")
        assert impulse.max() <= bar(sens, "impulse")
        bound = bar(sens, "lambda")
        lam_error = relative_error(world.download("lambda"), oracle.download("lambda"))
        print(cfg.name, f"lambda error {lam_error:.2e} against bound {bound:.2e}")
        assert lam_error <= bound
        # environments whose solve met the tolerance inside the budget took the same number of sweeps
        budget = cfg.vel_iters
        gs, os_ = world.download("vbd_velocity_sweep_count"), oracle.download("vbd_velocity_sweep_count")
        assert np.mean(gs == os_) > 0.97 and np.all(gs <= budget)
        per_env = per_env_error(world.download("lambda"), oracle.download("lambda"), E)
        print(cfg.name, "environments with lambda error above 1e-4:", int((per_env > TOL).sum()), "of", E)
    world.close()
    oracle.close()


def distances_to_double(oracle_py, device, index, E):
    """Per environment, how far the device's and the single-precision oracle's results of one solve lie from those
    of the oracle's double-precision build (the same algorithm with every scalar a double: the answer that the
    single-precision arithmetic approximates).  Accelerations against the environment's largest, the post-solve
    velocity against its free velocity, multipliers and the generalized contact impulse against their largest.
    Environments whose integer outputs differ between the builds (a pair at the edge of its query band) are left out."""
    cfg = nk.synthetic.config(index, E)
    desc = nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    state = cfg.state()
    exact = oracle_py.OracleWorld(cfg.template, desc, threads=8, double=True)
    single = oracle_py.OracleWorld(cfg.template, desc, threads=8)
    world = nk.World(device, cfg.template, desc)
    for w in (exact, single, world):
        w.set_state(state)
    for name in UPSTREAM:
        for w in (exact, single):
            w.op(*ORACLE_OPS[name])
        world.op(name)
    world.synchronize()
    free = np.maximum(np.abs(exact.download("qdot_flat")).reshape(E, -1).max(1), 1e-6)
    for w in (exact, single):
        w.op("block_descent_solve")
    world.op("BlockDescentSolve")
    world.synchronize()
    same = np.ones(E, bool)
    for name in ("contact_count", "row_count", "pair_count"):
        same &= (exact.download(name) == single.download(name)) & (exact.download(name) == world.download(name))
    def per_env(w):
        return {"qdd": w.download("articulation_qdd").reshape(E, -1).astype(np.float64), "velocity": w.download("qdot_flat").reshape(E, -1).astype(np.float64),
                "lambda": w.download("lambda").reshape(E, -1).astype(np.float64), "impulse": generalized_impulse(w, E)}
    truth, out = per_env(exact), {}
    for label, w in (("device", world), ("oracle", single)):
        got = per_env(w)
        out[label] = {k: (np.abs(got[k] - truth[k]).max(1) / (free if k == "velocity" else np.maximum(np.abs(truth[k]).max(1), 1e-9)))[same] for k in truth}
    sweeps = {label: w.download("vbd_velocity_sweep_count")[same] for label, w in (("device", world), ("oracle", single), ("double", exact))}
    for w in (exact, single, world):
        w.close()
    return out, sweeps, int(same.sum())


@pytest.mark.parametrize("index,E", [(2, 512), (3, 512)])
def test_the_kernels_line_rule_in_the_oracle_changes_nothing_that_is_compared(oracle_py, device, index, E):
    """The kernels' line search stops by a rule that is not the reference's (its rounding magnitude also counts the
    heads' residuals).  The oracle switched to that rule must stand to the device as the oracle under the reference's
    rule does: sweep counts equal on at least 99 % of the environments either way, velocities within the bar either way."""
    cfg = nk.synthetic.config(index, E)
    desc = nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    state = cfg.state()
    world = nk.World(device, cfg.template, desc)
    world.set_state(state)
    for name in UPSTREAM + ["BlockDescentSolve"]:
        world.op(name)
    world.synchronize()
    got, sweeps = world.download("qdot_flat").reshape(E, -1), world.download("vbd_velocity_sweep_count").astype(int)
    for rule in (0, 1):
        oracle = oracle_py.OracleWorld(cfg.template, desc, threads=8)
        oracle.set_line_rule(rule)
        oracle.set_state(state)
        for name in UPSTREAM + ["BlockDescentSolve"]:
            oracle.op(*ORACLE_OPS[name])
        expect, taken = oracle.download("qdot_flat").reshape(E, -1), oracle.download("vbd_velocity_sweep_count").astype(int)
        equal = sweeps == taken
        error = np.abs(got - expect).max(1) / np.maximum(np.abs(expect).max(1), 1e-6)
        print(f"config {index}, line rule {rule}: sweep counts equal on {equal.mean():.4f}, velocity worst {error[equal].max():.2e}")
        assert equal.mean() >= 0.99 and np.abs(sweeps - taken).max() <= 1
        assert error[equal].max() <= TOL
        oracle.close()
    world.close()


@pytest.mark.parametrize("index,E", [(2, 512), (3, 512), (5, 64)])
def test_the_device_is_as_close_to_the_double_precision_answer_as_the_oracle(oracle_py, device, index, E):
    """The bars above that exceed 1e-4 rest on the single-precision oracle's own sensitivity; this is the measure
    behind them.  The oracle built in double gives the answer both single-precision evaluations approximate.  Where the
    problem is well posed both lie within 1e-4 of it; where it is not (six coplanar spheres on one rigid foot, the
    rope's Newton block), the oracle itself lies further away, and the device must not lie further than twice as far.
    The distances of single environments are two draws of rounding noise, so they are compared as distributions:
    median, 95th percentile and largest over the batch, each against twice the oracle's or the tolerance."""
    out, sweeps, counted = distances_to_double(oracle_py, device, index, E)
    assert counted >= 0.95 * E
    report = []
    for key in ("qdd", "velocity", "lambda", "impulse"):
        dev, ora = out["device"][key], out["oracle"][key]
        for what, measure in (("median", np.median), ("95th percentile", lambda v: np.percentile(v, 95)), ("largest", np.max)):
            d, o = float(measure(dev)), float(measure(ora))
            assert d <= max(TOL, 2.0 * o), f"{key} {what}: device {d:.2e} from the double-precision answer, oracle {o:.2e}"
        report.append(f"{key}: device {np.max(dev):.1e} (median {np.median(dev):.1e}), oracle {np.max(ora):.1e} (median {np.median(ora):.1e})")
    print(f"config {index}, {counted} environments, largest distance to the double-precision answer - " + "; ".join(report))
    print("sweep counts equal to the double build's: device %.3f, oracle %.3f" % (np.mean(sweeps["device"] == sweeps["double"]), np.mean(sweeps["oracle"] == sweeps["double"])))


def test_quadruped_impulses_meet_the_plain_tolerance(oracle_py, device):
    """Four separate feet, one sphere each: the impulse split is well determined and lambda itself meets 1e-4."""
    E = 512
    _, oracle, world, _ = make_pair(oracle_py, device, 2, E)
    world.step()
    world.synchronize()
    oracle.step()
    assert relative_error(world.download("lambda"), oracle.download("lambda")) <= TOL
    same = world.download("vbd_velocity_sweep_count") == oracle.download("vbd_velocity_sweep_count")
    assert same.mean() > 0.98        # a residual within rounding of the tolerance can take one sweep more or less
    world.close()
    oracle.close()


def test_several_steps_stay_with_the_oracle(oracle_py, device):
    E, steps = 128, 4
    cfg, oracle, world, _ = make_pair(oracle_py, device, 2, E)
    world.step(steps)
    world.synchronize()
    oracle.step(steps)
    sensitivity = oracle_sensitivity(oracle_py, 2, E, ["q", "qdot", "link_pose"], steps=steps)
    for name in ("q", "qdot", "link_pose"):
        error = relative_error(world.download(name), oracle.download(name))
        print(name, f"{error:.2e}", f"one-ulp sensitivity {sensitivity[name]:.2e}")
        assert error <= max(TOL, 4.0 * sensitivity[name])
    world.close()
    oracle.close()


def test_rope_step_matches_the_oracle(oracle_py, device):
    """Config 5 through every op, the block descent included.  The 64-link rope's mass matrix has a condition number
    of about 2e4 (with its joint armature) and its Newton block about 1e6, so accelerations and the solve's outputs
    move by more than 1e-4 under a one-ulp change of the inputs in the oracle itself; their bar is max(1e-4, 4 x that
    measured sensitivity), and the accelerations are also held by their residual.  The resulting joint angles carry
    the push-out of the position pass, one more block descent over 64 one-sided rows that stops at its Newton-step
    budget in a few environments: they get the same kind of bar.  Everything else - poses, M, the bias, the contact
    integers, rows and Jacobians, status words - is held as on the other configurations."""
    E = 64
    cfg, oracle, world, state = make_pair(oracle_py, device, 5, E)
    sens = one_ulp_sensitivity(oracle_py, cfg.template, nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters), state)
    print("rope one-ulp sensitivity of the oracle:", {k: f"{v:.2e}" for k, v in sens.items()})
    report = compare_ops(oracle, world, E, sens, state)
    status = oracle.download("env_status")
    assert np.all(status == 0) and np.all(oracle.download("contact_count") == 64)
    gs, os_ = world.download("vbd_velocity_sweep_count"), oracle.download("vbd_velocity_sweep_count")
    lam = relative_error(world.download("lambda"), oracle.download("lambda"))
    print("rope sweeps (oracle)", np.bincount(os_), "same count on", float(np.mean(gs == os_)), "worst environment:",
          {k: f"{v.max():.2e}" for k, v in report.items()}, f"lambda {lam:.2e}")
    assert np.mean(gs == os_) >= 0.9 and np.all(gs <= cfg.vel_iters)
    assert lam <= bar(sens, "lambda")
    world.close()
    oracle.close()


def test_graph_replays_equal_eager_steps(oracle_py, device):
    E = 256
    cfg = nk.synthetic.config(3, E)
    desc = nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters)
    names = ("q", "qdot", "link_pose", "lambda", "link_velocity", "vbd_velocity_sweep_count")
    results = []
    for graph in (False, True):
        world = nk.World(device, cfg.template, desc)
        world.set_state(cfg.state())
        world.set_execution_mode(graph)
        per_step = []
        for _ in range(4):                     # every replay is checked, with host reads in between
            world.step()
            world.synchronize()
            per_step.append({n: world.download(n) for n in names})
        results.append(per_step)
        world.close()
    for eager, replay in zip(*results):
        for n in names:
            assert np.array_equal(eager[n], replay[n]), n


def test_steps_are_deterministic_and_reset_restores(oracle_py, device):
    E = 256
    cfg = nk.synthetic.config(3, E)
    world = nk.World(device, cfg.template, nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters))
    runs = []
    for _ in range(2):
        world.reset()
        world.set_state(cfg.state())
        world.step(3)
        world.synchronize()
        runs.append({n: world.download(n) for n in ("q", "qdot", "lambda", "link_pose")})
    for n in runs[0]:
        assert np.array_equal(runs[0][n], runs[1][n]), n
    world.close()


def test_velocity_iteration_budget_can_change(oracle_py, device):
    """nuka_world_set_velocity_iterations raises the sweep budget of an existing world; the result is the oracle's
    at that budget, including which environments still miss the tolerance."""
    E = 128
    cfg = nk.synthetic.config(3, E)
    world = nk.World(device, cfg.template, nk.abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters))
    oracle = oracle_py.OracleWorld(cfg.template, nk.abi.world_desc(E, cfg.dt, vel_iters=100), threads=8)
    state = cfg.state()
    world.set_state(state)
    oracle.set_state(state)
    world.set_velocity_iterations(100)
    world.step()
    world.synchronize()
    oracle.step()
    sweeps, expect = world.download("vbd_velocity_sweep_count"), oracle.download("vbd_velocity_sweep_count")
    assert sweeps.max() > cfg.vel_iters and sweeps.max() <= 100
    assert np.mean(sweeps == expect) > 0.9        # a residual within rounding of the tolerance can take one sweep more
    converged = oracle.download("solver_residual").reshape(E, 4).max(1) < 2e-5
    assert converged.mean() > 0.95
    assert np.array_equal(world.download("solver_residual").reshape(E, 4).max(1) < 2e-5, converged)
    assert relative_error(world.download("qdot"), oracle.download("qdot")) <= TOL
    world.close()
    oracle.close()


def test_checkpoint_restore_replays_the_same_step(oracle_py, device):
    """nuka_world_checkpoint_capture / restore: a step taken from a restored checkpoint equals, bit for bit, the
    step taken from the state itself - after other steps have run in between - and matches the oracle."""
    E = 128
    cfg, oracle, world, _ = make_pair(oracle_py, device, 3, E)
    seeded = world.checkpoint()
    import ctypes
    size = ctypes.c_uint64()
    assert nk.lib().nuka_checkpoint_byte_size(seeded, ctypes.byref(size)) == 0 and size.value > E * 1000
    world.step()
    world.synchronize()
    first = {n: world.download(n) for n in ("q", "qdot", "lambda", "link_pose", "base_pose", "contact_row_extent")}
    world.step(7)
    world.step_from(seeded, 2)
    world.synchronize()
    for n, expect in first.items():
        assert np.array_equal(world.download(n), expect), n
    oracle.step()
    close(world, oracle, "qdot")
    other = nk.World(device, cfg.template, nk.abi.world_desc(E, cfg.dt))
    assert nk.lib().nuka_world_checkpoint_restore(other._h, seeded) == 1          # a checkpoint of another world
    other.close()
    nk.lib().nuka_checkpoint_destroy(seeded)
    world.close()
    oracle.close()


def test_contact_cache_follows_the_oracle_over_steps(oracle_py, device):
    """ContactWarmStart over several steps of tilted boxes (feature-id corners persist, so the cache matches and
    seeds): keys, ages, owners, retained entries, extents and match counts bit-exact; cached impulses to TOL."""
    from test_gpu_properties import box_template
    E = 64
    t = box_template(True)
    g = np.random.default_rng(4)
    quat = np.array([1, 0, 0, 0]) + g.normal(0, 0.04, (E, 4))
    base = np.concatenate([g.normal(0, 0.2, (E, 2)), g.uniform(0.035, 0.05, (E, 1)), quat / np.linalg.norm(quat, axis=1, keepdims=True)], 1)
    zero = np.zeros((E, 1), np.float32)
    state = dict(q=np.concatenate([zero, g.uniform(-0.3, 0.6, (E, 1))], 1).astype(np.float32), qdot=np.zeros((E, 2), np.float32),
                 tau=np.zeros((E, 2), np.float32), base_pose=base.astype(np.float32), root_twist=np.zeros((E, 6), np.float32))
    desc = nk.abi.world_desc(E, 1.0 / 200.0, vel_iters=30)
    world, oracle = nk.World(device, t, desc), oracle_py.OracleWorld(t, desc, threads=4)
    world.set_state(state)
    oracle.set_state(state)
    matched = 0
    for step in range(5):
        world.step()
        world.synchronize()
        oracle.step()
        for name in ("contact_material", "contact_cache_current_owner", "contact_cache_old_keep", "contact_cache_extent",
                     "contact_warm_start_counts", "contact_cache_age"):
            assert np.array_equal(world.download(name), oracle.download(name)), f"step {step}: {name}"
        same = world.download("contact_cache_pair") == oracle.download("contact_cache_pair")
        assert same.all()
        # sphere points hash a quantised position into their feature word; box corners carry exact ids
        assert np.mean(world.download("contact_cache_feature") == oracle.download("contact_cache_feature")) > 0.99
        assert relative_error(world.download("contact_cache_lambda"), oracle.download("contact_cache_lambda")) <= TOL
        assert relative_error(world.download("contact_cache_normal"), oracle.download("contact_cache_normal")) <= TOL
        assert relative_error(world.download("qdot"), oracle.download("qdot")) <= TOL
        matched += int(oracle.download("contact_warm_start_counts").reshape(E, 2)[:, 1].sum())
    assert matched > E
    # the seeding itself: phase 0 on both sides from the same cache
    for name, oname in (("FkWorldPoses", "fk_world_poses"), ("ArticulationDynamics", "articulation_dynamics")):
        oracle.op(oname, *((1,) if oname == "articulation_dynamics" else ()))
        world.op(name)
    for name in UPSTREAM[2:]:
        both(oracle, world, name)
    oracle.op("contact_warm_start", 0)
    world.op("ContactWarmStart", 0)
    world.synchronize()
    seeds = oracle.download("lambda")
    assert np.count_nonzero(seeds) > E
    assert relative_error(world.download("lambda"), seeds) <= TOL
    world.close()
    oracle.close()
