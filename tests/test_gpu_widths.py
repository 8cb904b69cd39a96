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


# (coordinates, floating root, joints a limb, limbs that carry spheres or None, width of the sweeps): every kernel of
# the dense build, full blocks up to 20 coordinates and the reduced blocks that sweep at up to 20
DENSE = [(4, False, 7, None, 4), (8, True, 7, None, 8), (11, True, 7, None, 11), (16, False, 7, None, 16), (20, True, 7, None, 20),
         (24, True, 6, 1, 12), (28, True, 7, 1, 16), (32, True, 7, 1, 16), (36, True, 7, 2, 20), (40, True, 7, 2, 20)]


@pytest.mark.parametrize("dof,floating,limb_joints,sphere_limbs,width", DENSE)
def test_large_batches_take_the_dense_kernels_and_give_the_same_bits(oracle_py, device, dof, floating, limb_joints, sphere_limbs, width):
    """From 6144 environments on, worlds of contact heads only whose sweeps are at most 20 wide run the kernels compiled
    for three waves a SIMD (twelve blocks a compute unit instead of eight).  They are the same arithmetic in fewer
    registers: a batch of 6144 made of 128 copies of 48 seeded environments must give, in every copy, the bits the 48
    give alone with the two-wave kernel, and those stay with the oracle."""
    E, copies = 48, 128
    tree, desc, state = tree_case(oracle_py, dof, floating, True, seed=5 * dof + 1, E=E, limb_joints=limb_joints, sphere_limbs=sphere_limbs)
    small = nk.World(device, tree.template, desc)
    assert small.dof == dof and small.info.solver_width == width and small.info.solver_blocks_per_cu == 8
    small.set_state(state)
    small.step()
    small.synchronize()
    big_desc = nk.abi.world_desc(E * copies, 1.0 / 240.0, vel_iters=8, contact_margin=0.1)
    big = nk.World(device, tree.template, big_desc)
    assert big.info.solver_width == width and big.info.solver_blocks_per_cu > 8, big.info.solver_blocks_per_cu
    big.set_state({k: np.tile(v, (copies, 1)) for k, v in state.items()})
    big.step()
    big.synchronize()
    assert (small.download("contact_count") > 0).mean() >= 0.4, "the case must exercise the contact solve"
    for name in ("qdot", "q", "lambda", "link_velocity", "vbd_velocity_sweep_count", "env_status"):
        alone = small.download(name).reshape(1, -1)
        batch = big.download(name).reshape(copies, -1)
        assert np.array_equal(np.broadcast_to(alone, batch.shape), batch), name
    small.close()
    small = nk.World(device, tree.template, desc)       # and the two-wave kernel's results against the oracle's, op by op
    small.set_state(state)
    oracle = oracle_py.OracleWorld(tree.template, desc, threads=8)
    oracle.set_state(state)
    compare_ops(oracle, small, E, one_ulp_sensitivity(oracle_py, tree.template, desc, state), state)
    small.close()
    big.close()
    oracle.close()
