"""Every compiled width of the device kernels against the CPU oracle: the benchmark configurations reach 8, 20, 36 and
64 padded coordinates only, so seeded trees fill in the rest, in particular the widths past 36 that run one wavefront
per SIMD and, past 32, factor the Newton block from the leaves (the reference's wide route)."""
import numpy as np
import pytest

from conftest import nk
from test_gpu_parity import TOL, bar, close, compare_ops, one_ulp_sensitivity
from trees import tree_case

pytestmark = pytest.mark.gpu

CASES = [  # coordinates, floating root, branched
    (33, True, True), (40, True, True), (40, False, False), (44, True, True), (48, True, False), (48, False, True),
    (52, True, True), (56, True, True), (56, False, False), (60, True, True), (64, True, True), (64, False, True),
    (24, True, True), (28, False, False), (32, True, True), (13, True, False),
]


@pytest.mark.parametrize("dof,floating,branched", CASES)
def test_every_op_at_every_width_matches_the_oracle(oracle_py, device, dof, floating, branched):
    E = 48
    tree, desc, state = tree_case(oracle_py, dof, floating, branched, seed=dof + 7 * floating + 3 * branched, E=E)
    oracle = oracle_py.OracleWorld(tree.template, desc, threads=8)
    world = nk.World(device, tree.template, desc)
    assert world.dof == dof
    oracle.set_state(state)
    world.set_state(state)
    sens = one_ulp_sensitivity(oracle_py, tree.template, desc, state)
    report = compare_ops(oracle, world, E, sens, state)
    contacts = oracle.download("contact_count")
    assert (contacts > 0).mean() >= 0.4, "the case must exercise the contact solve"
    print(f"dof {dof} floating {floating} branched {branched}: contacts per env {contacts.mean():.1f}, worst environment "
          + ", ".join(f"{k} {v.max():.2e}" for k, v in report.items()) + "; oracle one-ulp sensitivity "
          + ", ".join(f"{k} {v:.1e}" for k, v in sens.items()))
    close(world, oracle, "link_velocity", tol=bar(sens, "velocity"))
    world.close()
    oracle.close()


@pytest.mark.parametrize("dof,floating,branched", [(40, True, True), (56, False, False), (64, True, True)])
def test_steps_at_wide_widths_stay_with_the_oracle(oracle_py, device, dof, floating, branched):
    """Three whole steps (contact cache and carried solver velocities included) through the graph-less pipeline."""
    E = 32
    tree, desc, state = tree_case(oracle_py, dof, floating, branched, seed=dof, E=E)
    oracle = oracle_py.OracleWorld(tree.template, desc, threads=8)
    world = nk.World(device, tree.template, desc)
    oracle.set_state(state)
    world.set_state(state)
    for step in range(3):
        world.step()
        world.synchronize()
        oracle.step()
        assert np.array_equal(world.download("env_status"), oracle.download("env_status")), f"step {step}"
        for name in ("q", "link_pose", "base_pose"):
            close(world, oracle, name, tol=TOL if step == 0 else 3 * TOL)
    world.close()
    oracle.close()


@pytest.mark.parametrize("dof,floating,limb_joints", [(48, True, 3), (40, True, 2), (64, True, 4)])
def test_trees_wider_than_a_sweep_pass_match_the_oracle(oracle_py, device, dof, floating, limb_joints):
    """Bushy trees: more links at one depth (14, 17 and 15) than a pass of the dynamics' tree sweeps holds (ten), so a depth
    takes several passes; every op against the oracle as above."""
    E = 32
    tree, desc, state = tree_case(oracle_py, dof, floating, True, seed=5 * dof + limb_joints, E=E, limb_joints=limb_joints)
    oracle = oracle_py.OracleWorld(tree.template, desc, threads=8)
    world = nk.World(device, tree.template, desc)
    assert world.dof == dof
    oracle.set_state(state)
    world.set_state(state)
    sens = one_ulp_sensitivity(oracle_py, tree.template, desc, state)
    compare_ops(oracle, world, E, sens, state)
    close(world, oracle, "link_velocity", tol=bar(sens, "velocity"))
    close(world, oracle, "link_acceleration", tol=bar(sens, "qdd"))
    world.close()
    oracle.close()
