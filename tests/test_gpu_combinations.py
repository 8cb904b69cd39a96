"""Features that other tests cover one at a time, here together and at widths the benchmark configurations do not reach:
joint rows (unit heads) in the wide one-wave-per-SIMD kernels, the MuJoCo contact law with either cone at wide widths,
MuJoCo-sourced joint rows with the integrator's damping pass, the split-impulse position pass at narrow and wide widths.
Every case steps the device world and the CPU oracle side by side from one seeded state."""
import copy

import numpy as np
import pytest

from conftest import nk, per_env_error
from test_gpu_parity import TOL
from trees import tree_case

pytestmark = pytest.mark.gpu
abi = nk.abi

# coordinates, floating root, branched, features
CASES = [
    (20, True, True, dict(drive=abi.DRIVE_PD_POSITION, limits=True, friction=0.1)),
    (44, True, True, dict(drive=abi.DRIVE_PD_POSITION, limits=True, friction=0.1)),
    (60, True, True, dict(drive=abi.DRIVE_TORQUE, limits=True, friction=0.05)),
    # a 64-link serial chain moves its own accelerations by 3e-3 under one ulp of input and doubles that every step: one step
    (64, False, False, dict(drive=abi.DRIVE_TORQUE, limits=True, friction=0.05, steps=1)),
    (40, True, True, dict(cone=abi.CONE_ELLIPTIC)),
    (48, True, False, dict(cone=abi.CONE_PYRAMIDAL)),
    (28, True, True, dict(cone=abi.CONE_ELLIPTIC, limits=True, friction=0.1, joint_law=True, integrator=abi.INTEGRATOR_MUJOCO_EULER, damping=0.4)),
    (56, True, True, dict(limits=True, friction=0.1, pos_iters=2)),
    # the position pass at widths whose block assembly updates the Hessian row by the written-out column groups: its
    # contact heads are single rows, with and without joint rows beside them
    (20, True, True, dict(pos_iters=2)),
    (32, False, True, dict(limits=True, friction=0.1, pos_iters=3)),
    (36, False, True, dict(cone=abi.CONE_PYRAMIDAL, drive=abi.DRIVE_VELOCITY, limits=True)),
]


def featured(tree, feats, seed):
    """The tree's template with the case's features switched on."""
    t = copy.deepcopy(tree.template)
    g = np.random.default_rng(seed)
    if "drive" in feats:
        t.drive_rows, t.drive_mode = True, feats["drive"]
    for l, link in enumerate(t.links):
        if link["joint_type"] != abi.JOINT_REVOLUTE:
            continue
        if feats.get("limits") and l % 3 != 0:
            link["lower"], link["upper"] = -0.25, 0.3          # the seeded angles (sigma 0.3) leave some joints outside
        if feats.get("friction") and l % 2 == 0:
            link["frictionloss"] = feats["friction"]
        if feats.get("damping"):
            link["damping"] = float(g.uniform(0.0, feats["damping"]))
        if feats.get("joint_law"):
            link["law"] = abi.LAW_MUJOCO
            link["limit_margin"] = 0.01
    if "cone" in feats:
        for profile in t.profiles:
            profile["law"] = abi.LAW_MUJOCO
        t.contact_cone = feats["cone"]
    if "integrator" in feats:
        t.integrator = feats["integrator"]
    return t


def drive_fields(feats, E, nl, seed):
    g = np.random.default_rng(seed)
    mode = feats.get("drive")
    if mode is None:
        return {}
    return dict(
        drive_target=g.normal(0, 0.2, (E, nl)) if mode == abi.DRIVE_PD_POSITION else g.normal(0, 1.5, (E, nl)),
        drive_stiffness=g.uniform(5, 30, (E, nl)), drive_damping=g.uniform(0.2, 1.0, (E, nl)),
        drive_force_limit=np.where(g.uniform(size=(E, nl)) < 0.5, g.uniform(2, 10, (E, nl)), 0.0),
        velocity_target=g.normal(0, 0.5, (E, nl)), joint_f=g.normal(0, 0.3, (E, nl)))


FIELDS = ("q", "qdot", "link_pose", "base_pose", "link_velocity")


def one_ulp_sensitivity(oracle_py, template, desc, state, extras, steps):
    """How far the oracle's own outputs move, step by step, when q, qdot and tau start one ulp away: the worst
    environment's relative change of every compared field.  No other fp32 evaluation of the same formulas can be held
    closer than a few times this (a 64-link serial chain moves its joint accelerations by 3e-3)."""
    E = desc.env_count
    runs = []
    for perturb in (False, True):
        w = oracle_py.OracleWorld(template, desc, threads=8)
        moved = {k: v.copy() for k, v in state.items()}
        if perturb:
            g = np.random.default_rng(99)
            for key in ("q", "qdot", "tau"):
                toward = moved[key] + g.choice([-1.0, 1.0], moved[key].shape).astype(np.float32)
                moved[key] = np.nextafter(moved[key], toward).astype(np.float32)
        w.set_state(moved)
        for name, values in extras.items():
            w.upload(name, values.astype(np.float32))
        out = []
        for _ in range(steps):
            w.step()
            out.append({name: w.download(name).copy() for name in FIELDS})
        runs.append(out)
        w.close()
    return [{name: float(per_env_error(runs[1][s][name], runs[0][s][name], E).max()) for name in FIELDS} for s in range(steps)]


@pytest.mark.parametrize("dof,floating,branched,feats", CASES, ids=lambda v: "-".join(sorted(v)) if isinstance(v, dict) else str(v))
def test_features_together_stay_with_the_oracle(oracle_py, device, dof, floating, branched, feats):
    E, steps = 32, feats.get("steps", 3)
    seed = dof + 11 * len(feats)
    tree, desc, state = tree_case(oracle_py, dof, floating, branched, seed=seed, E=E)
    template = featured(tree, feats, seed)
    desc = abi.world_desc(E, 1.0 / 240.0, vel_iters=8, pos_iters=feats.get("pos_iters", 0), contact_margin=0.1)
    oracle = oracle_py.OracleWorld(template, desc, threads=8)
    world = nk.World(device, template, desc)
    assert world.dof == dof and world.rows_per_env == oracle.rows_per_env
    extras = drive_fields(feats, E, template.link_count, seed)
    for w in (oracle, world):
        w.set_state(state)
        for name, values in extras.items():
            w.upload(name, values.astype(np.float32))
    sens = one_ulp_sensitivity(oracle_py, template, desc, state, extras, steps)
    report = []
    for step in range(steps):
        world.step()
        world.synchronize()
        oracle.step()
        assert np.array_equal(world.download("env_status"), oracle.download("env_status")), f"step {step}: env_status"
        for name in ("contact_count", "row_count"):
            assert np.array_equal(world.download(name), oracle.download(name)), f"step {step}: {name}"
        sweeps_g, sweeps_o = world.download("vbd_velocity_sweep_count"), oracle.download("vbd_velocity_sweep_count")
        assert (sweeps_g == sweeps_o).mean() >= 0.9 and np.abs(sweeps_g.astype(int) - sweeps_o.astype(int)).max() <= 1, f"step {step}: sweeps"
        for name in FIELDS:
            # the stated tolerance (later steps compound the first step's last-place differences), or four times the
            # oracle's own one-ulp sensitivity where that is larger
            tol = max(TOL if step == 0 else 3 * TOL, 4.0 * sens[step][name])
            errors = per_env_error(world.download(name), oracle.download(name), E)
            report.append((step, name, float(errors.max())))
            assert errors.max() <= tol, f"step {step}, {name}: {int((errors > tol).sum())} of {E} environments above {tol:.1e}, worst {errors.max():.3e}"
    assert (oracle.download("contact_count") > 0).mean() >= 0.3, "the case must keep contacts"
    print(f"{dof} coordinates, {feats}: worst per-environment error " + ", ".join(f"{n}@{s} {e:.1e}" for s, n, e in report if s == steps - 1)
          + "; oracle one-ulp sensitivity " + ", ".join(f"{n} {v:.1e}" for n, v in sens[-1].items()))
    world.close()
    oracle.close()
