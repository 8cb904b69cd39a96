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


@pytest.mark.parametrize("dof,floating,limb_joints", [(44, True, 7), (64, False, 16), (28, True, 7)])
def test_wide_blocks_with_rows_between_links_match_the_oracle(oracle_py, device, dof, floating, limb_joints):
    """Worlds whose spheres also collide with one another: some contact rows have the articulation on both sides, so a
    wide block keeps its rows staged instead of deriving them from the links, and takes the heads' curvature by way of
    the links only in environments where every live row happens to be one-sided."""
    E = 48
    tree, desc, state = tree_case(oracle_py, dof, floating, True, seed=3 * dof + 1, E=E, limb_joints=limb_joints, sphere_pairs=True)
    oracle = oracle_py.OracleWorld(tree.template, desc, threads=8)
    world = nk.World(device, tree.template, desc)
    assert world.dof == dof
    oracle.set_state(state)
    world.set_state(state)
    sens = one_ulp_sensitivity(oracle_py, tree.template, desc, state)
    compare_ops(oracle, world, E, sens, state)
    rows = oracle.download("urows").reshape(E, -1, 26).view(np.uint32)
    active = (rows[:, :, 0] & 1) != 0
    two_sided = active & (rows[:, :, 10] == 1) & (rows[:, :, 18] == 1)
    print(f"dof {dof}: environments with a row between two links {int(two_sided.any(1).sum())} of {E}, contacts per env "
          f"{oracle.download('contact_count').mean():.1f}")
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


# (coordinates, floating root, joints a limb, limbs that carry spheres, width of the sweeps): every compiled pair of a
# full and a reduced width
REDUCED = [(24, True, 6, 1, 12), (28, True, 7, 1, 16), (32, True, 7, 1, 16), (36, True, 7, 2, 20), (40, True, 7, 2, 20), (44, True, 7, 2, 24),
           (48, True, 7, 2, 24), (52, True, 7, 3, 28), (56, True, 7, 3, 28), (60, True, 7, 3, 32), (64, True, 7, 3, 32), (48, False, 8, 3, 24)]


@pytest.mark.parametrize("dof,floating,limb_joints,sphere_limbs,width", REDUCED)
def test_reduced_blocks_match_the_oracle(oracle_py, device, dof, floating, limb_joints, sphere_limbs, width):
    """Worlds whose contacts reach only the first limbs: the solve eliminates the other coordinates once and sweeps at
    the reduced width (the oracle solves the full block, as the reference does).  Every op of a step against the oracle,
    then the momentum balance of all coordinates, the eliminated ones included."""
    E = 48
    tree, desc, state = tree_case(oracle_py, dof, floating, True, seed=11 * dof + sphere_limbs, E=E, limb_joints=limb_joints,
                                  sphere_limbs=sphere_limbs)
    oracle = oracle_py.OracleWorld(tree.template, desc, threads=8)
    world = nk.World(device, tree.template, desc)
    assert world.dof == dof and world.info.solver_width == width
    oracle.set_state(state)
    world.set_state(state)
    sens = one_ulp_sensitivity(oracle_py, tree.template, desc, state)
    report = compare_ops(oracle, world, E, sens, state)
    contacts = oracle.download("contact_count")
    assert (contacts > 0).mean() >= 0.4, "the case must exercise the contact solve"
    close(world, oracle, "link_velocity", tol=bar(sens, "velocity"))
    print(f"dof {dof} sweeps at {width}: contacts per env {contacts.mean():.1f}, worst environment "
          + ", ".join(f"{k} {v.max():.2e}" for k, v in report.items()))
    world.close()
    oracle.close()
    # the momentum balance of all coordinates with the device's own M and J: M (v - v_free) = J^T lambda, measured in
    # velocity units, on the environments that met the tolerance; the eliminated coordinates hold it as the others do
    world = nk.World(device, tree.template, desc)
    world.set_state(state)
    for name in ("FkWorldPoses", "ArticulationDynamics", "SyncLinkBodyPose", "BuildAabbs", "LbvhQueryPairs", "NarrowphasePrimitives", "AssembleRows"):
        world.op(name)
    world.synchronize()
    free = world.download("qdot_flat").reshape(E, -1)[:, :dof].astype(np.float64)
    world.op("BlockDescentSolve")
    world.synchronize()
    R = world.rows_per_env
    M = world.download("m").reshape(E, dof, dof).astype(np.float64)
    J = (world.download("chain_jacobian").reshape(E, R, -1) + world.download("chain_jacobian_b").reshape(E, R, -1))[:, :, :dof].astype(np.float64)
    lam = world.download("lambda").reshape(E, R).astype(np.float64)
    v = world.download("qdot_flat").reshape(E, -1)[:, :dof].astype(np.float64)
    balance = np.einsum("eij,ej->ei", M, v - free) - np.einsum("eri,er->ei", J, lam)
    imbalance = np.abs(np.linalg.solve(M, balance[:, :, None])[:, :, 0])
    converged = world.download("vbd_velocity_sweep_count") < 8
    assert converged.sum() >= E // 4
    assert imbalance[converged].max() < 1.2e-5, imbalance[converged].max()
    assert imbalance[converged][:, width:].max() < 1.2e-5
    world.close()


@pytest.mark.parametrize("dof,floating,limb_joints,sphere_limbs", [(36, True, 7, 2), (64, True, 7, 3)])
def test_steps_of_reduced_blocks_stay_with_the_oracle(oracle_py, device, dof, floating, limb_joints, sphere_limbs):
    E = 32
    tree, desc, state = tree_case(oracle_py, dof, floating, True, seed=3 * dof, E=E, limb_joints=limb_joints, sphere_limbs=sphere_limbs)
    oracle = oracle_py.OracleWorld(tree.template, desc, threads=8)
    world = nk.World(device, tree.template, desc)
    assert world.info.solver_width < dof
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
