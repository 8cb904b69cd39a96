"""Parity of the HIP contact path beyond shape-against-plane pairs with the CPU oracle, through the C ABI on an
MI355X: every analytic pair of sphere, capsule, box, plane and cylinder (the oracle's manifolds are pinned bit-exact
against the reference's own header), rows whose two sides both move, and the excluded-pair list.  Bars as in
test_gpu_parity: integer words bit-exact, fp32 norm-wise relative error <= 1e-4."""
import numpy as np
import pytest

from conftest import nk, relative_error
from test_gpu_parity import one_ulp_sensitivity
from test_oracle_pairs import box_on_slab, floating, floating_state, rail_state, rails

pytestmark = pytest.mark.gpu
abi = nk.abi
TOL = 1e-4
ROW_WORDS = 26
CONTACT_NORMAL = 1 << 6
SPHERE, CAPSULE, BOX, PLANE, CYLINDER = abi.SHAPE_SPHERE, abi.SHAPE_CAPSULE, abi.SHAPE_BOX, abi.SHAPE_PLANE, abi.SHAPE_CYLINDER
SHAPE_PARAMS = {SPHERE: (0.05, 0, 0, 0), CAPSULE: (0.035, 0.08, 0, 0), BOX: (0.06, 0.04, 0.05, 0), CYLINDER: (0.04, 0.07, 0, 0),
                PLANE: (0, 0, 0, 0)}


def carriage(t, kind, profile):
    """Six links on the fixed root - three sliders, three hinges - whose last one carries the shape: a collidable
    that the coordinates place anywhere."""
    parent = 0
    for joint, axis in ((abi.JOINT_PRISMATIC, (1, 0, 0)), (abi.JOINT_PRISMATIC, (0, 1, 0)), (abi.JOINT_PRISMATIC, (0, 0, 1)),
                        (abi.JOINT_REVOLUTE, (1, 0, 0)), (abi.JOINT_REVOLUTE, (0, 1, 0)), (abi.JOINT_REVOLUTE, (0, 0, 1))):
        parent = t.add_link(joint, parent, axis=axis, mass=0.3, diag_inertia=(0.002, 0.003, 0.0025))
        t.add_body(abi.ROLE_LINK_BODY, link=parent, contype=0, conaffinity=0)
    return parent, dict(role=abi.ROLE_PROXY, link=parent, kind=kind, params=SHAPE_PARAMS[kind], contype=1, conaffinity=1, profile=profile)


def pair_template(ka, kb):
    """Collidable rows in the order (ka, kb): the lower row is side A of the pair."""
    t = abi.Template()
    t.add_link(abi.JOINT_FIXED, None, mass=1.0)
    profile = t.add_profile(0.7)
    shapes = []
    for kind in (ka, kb):
        if kind == PLANE:
            shapes.append(dict(role=abi.ROLE_STATIC, kind=PLANE, contype=1, conaffinity=1, profile=profile))
        else:
            shapes.append(carriage(t, kind, profile)[1])
    for shape in shapes:
        t.add_body(**shape)
    return t


def pair_state(t, E, seed, kinds):
    """Coordinates that bring the two shapes within a few centimetres of touching in about half the environments."""
    g = np.random.default_rng(seed)
    nl = t.link_count
    q = np.zeros((E, nl), np.float32)
    moving = [k for k in kinds if k != PLANE]
    for c, kind in enumerate(moving):
        first = 1 + 6 * c
        q[:, first:first + 3] = g.normal(0, 0.045, (E, 3))
        q[:, first + 3:first + 6] = g.uniform(-np.pi, np.pi, (E, 3))
        if PLANE in kinds:
            q[:, first + 2] = g.uniform(-0.01, 0.13, E)
            flat = np.nonzero(g.uniform(size=E) < 0.4)[0]    # cylinders standing on a cap, capsules lying down: the many-point cases
            turn = g.choice([0.0, np.pi], len(flat)) if kind == CYLINDER else np.full(len(flat), 0.5 * np.pi)
            q[flat, first + 3] = turn + g.normal(0, 0.05, len(flat))
            q[flat, first + 4] = g.normal(0, 0.05, len(flat))
            q[flat, first + 2] = g.uniform(0.0, 0.09, len(flat))
    qdot = g.normal(0, 0.5, (E, nl)).astype(np.float32)
    qdot[:, 0] = 0
    return dict(q=q, qdot=qdot, tau=np.zeros((E, nl), np.float32), base_pose=np.tile([0, 0, 0, 1, 0, 0, 0], (E, 1)).astype(np.float32),
                root_twist=np.zeros((E, 6), np.float32))


PAIRS = [(SPHERE, SPHERE), (SPHERE, BOX), (BOX, SPHERE), (CAPSULE, PLANE), (PLANE, CAPSULE), (CAPSULE, SPHERE), (SPHERE, CAPSULE),
         (CAPSULE, CAPSULE), (CYLINDER, PLANE), (PLANE, CYLINDER), (CYLINDER, SPHERE), (SPHERE, CYLINDER), (BOX, BOX)]


@pytest.mark.parametrize("ka,kb", PAIRS)
def test_every_analytic_pair_matches_the_oracle(oracle_py, device, ka, kb):
    E = 256
    t = pair_template(ka, kb)
    desc = abi.world_desc(E, 1.0 / 200.0, vel_iters=30)
    state = pair_state(t, E, 100 + 10 * ka + kb, (ka, kb))
    world, oracle = nk.World(device, t, desc), oracle_py.OracleWorld(t, desc, threads=8)
    world.set_state(state)
    oracle.set_state(state)
    oracle.op("fk_world_poses"); world.op("FkWorldPoses")
    oracle.op("articulation_dynamics", 1); world.op("ArticulationDynamics")
    for name, oname in (("SyncLinkBodyPose", "sync_link_body_pose"), ("BuildAabbs", "build_aabbs"), ("LbvhQueryPairs", "query_pairs"),
                        ("NarrowphasePrimitives", "narrowphase"), ("AssembleRows", "assemble_rows")):
        oracle.op(oname); world.op(name)
    world.synchronize()
    exact = ("pair_count", "candidate_pairs") if (ka, kb) == (BOX, BOX) else ("pair_count", "candidate_pairs", "ucontact_count", "ucontact_row_range", "ucontact_id_pair", "row_count")
    for name in exact:
        assert np.array_equal(world.download(name), oracle.download(name)), name
    counts = oracle.download("ucontact_count").reshape(E, -1)
    assert (counts > 0).sum() >= E // 5 and (counts == 0).sum() >= E // 10          # touching and apart both occur
    if PLANE in (ka, kb) and CAPSULE in (ka, kb):
        assert counts.max() == 2
    if PLANE in (ka, kb) and CYLINDER in (ka, kb):
        assert counts.max() == 4
    # Two of the manifolds are not continuous in their inputs: a cylinder cap keeps four of nine candidates by
    # distances that tie by symmetry, and the closest points of two capsule axes jump where the axes run parallel
    # or cross.  Poses that differ in their last bits can then give a different, equally valid manifold; such
    # environments (few) are set aside by their point keys or a coarse test on the points, and everything else -
    # manifolds, rows, Jacobians and the solve on them - has to meet the tolerance.
    S = world.info.contact_slots_per_env
    assert S == 1
    keys_g, keys_o = world.download("ucontact_id_feature").reshape(E, 4), oracle.download("ucontact_id_feature").reshape(E, 4)
    point_g, point_o = world.download("ucontact_point").reshape(E, 4, 3), oracle.download("ucontact_point").reshape(E, 4, 3)
    live = np.arange(4)[None, :] < counts.reshape(E, 1)
    same = np.ones(E, bool)
    if CYLINDER in (ka, kb) and PLANE in (ka, kb):
        same &= ~((keys_g != keys_o) & live).any(1)
    if (ka, kb) == (BOX, BOX):       # the winning axis of fifteen, and the clipped polygon's vertices, change with the last bits
        same &= ~(((keys_g != keys_o) | (np.abs(point_g - point_o).max(2) > 1e-4)) & live).any(1)
        same &= world.download("ucontact_count") == counts.reshape(-1)
    if (ka, kb) == (CAPSULE, CAPSULE):
        same &= ~((np.abs(point_g - point_o).max(2) > 1e-4) & live).any(1)
        # the normal is the difference of the closest axis points over its length: within two centimetres the
        # rounding of the poses (1e-6) shows in it at the tolerance itself
        axis_distance = 2 * SHAPE_PARAMS[CAPSULE][0] - (oracle.download("ucontact_depth").reshape(E, 4)[:, 0] - 5e-4)
        same &= ~((axis_distance < 0.02) & live[:, 0])
    assert same.mean() >= 0.8, same.mean()
    live = live & same[:, None]
    for name, width in (("ucontact_point", 3), ("ucontact_normal", 3), ("ucontact_depth", 1)):
        got, want = world.download(name).reshape(E, 4, width)[live], oracle.download(name).reshape(E, 4, width)[live]
        assert relative_error(got, want) <= TOL, name
    assert np.mean(keys_g[live] == keys_o[live]) > 0.98         # featureless points hash a quantised position
    R = world.rows_per_env
    grow, orow = world.download("urows").reshape(E, R, ROW_WORDS)[same], oracle.download("urows").reshape(E, R, ROW_WORDS)[same]
    assert np.array_equal(grow.view(np.uint32)[:, :, 0], orow.view(np.uint32)[:, :, 0])      # flags
    active = (orow.view(np.uint32)[:, :, 0] & 1) != 0
    for word in (1, 2, 3, 10, 11, 18, 19):                                                    # group, env, side kinds and owners
        assert np.array_equal(grow.view(np.uint32)[:, :, word][active], orow.view(np.uint32)[:, :, word][active]), word
    assert relative_error(grow[active][:, 4:10], orow[active][:, 4:10]) <= TOL                # rhs, compliance, bounds, friction
    for name in ("chain_jacobian", "chain_jacobian_b", "row_penetration"):
        assert relative_error(world.download(name).reshape(E, -1)[same], oracle.download(name).reshape(E, -1)[same]) <= TOL, name
    # the whole solve on those rows
    oracle.op("contact_warm_start", 0); world.op("ContactWarmStart", 0)
    oracle.op("block_descent_solve"); world.op("BlockDescentSolve")
    world.synchronize()
    assert np.array_equal(world.download("env_status")[same], oracle.download("env_status")[same])
    # A manifold of several points on one rigid body splits its impulse over the points indeterminately to first
    # order: the multipliers and the velocities are held to the tolerance, or to four times what the oracle's own answer
    # moves by when its inputs move by one ulp where that is more.
    # An environment whose residual sits at the solve's tolerance after some sweep stops there or a sweep later depending
    # on the last bits, and a sweep more moves what the contacts constrain weakly (a cylinder's spin) by more than the
    # tolerance: such environments (a few in a hundred at most) are compared on their sweep counts only.
    sens = one_ulp_sensitivity(oracle_py, t, desc, state)
    sweeps_agree = world.download("vbd_velocity_sweep_count") == oracle.download("vbd_velocity_sweep_count")
    assert sweeps_agree[same].mean() >= 0.97, sweeps_agree[same].mean()
    assert np.abs(world.download("vbd_velocity_sweep_count").astype(int) - oracle.download("vbd_velocity_sweep_count").astype(int)).max() <= 1
    same &= sweeps_agree
    for name, bound in (("qdot", max(TOL, 4.0 * sens["velocity"])), ("lambda", max(TOL, 4.0 * sens["lambda"]))):
        error = relative_error(world.download(name).reshape(E, -1)[same], oracle.download(name).reshape(E, -1)[same])
        assert error <= bound, (name, error, bound)
    world.close()
    oracle.close()


def test_two_spheres_collide_and_keep_their_momentum(device):
    m1, m2, radius, dt = 0.8, 2.0, 0.05, 1.0 / 200.0
    touching = 2 * radius - 1e-3
    state = rail_state([[0.0, touching], [0.0, touching], [0.0, touching + 0.05]], [[1.0, -0.5], [-0.2, 0.3], [1.0, -0.5]])
    world = nk.World(device, rails(m1, m2, radius), abi.world_desc(3, dt, gravity=(0, 0, 0), vel_iters=50))
    world.set_state(state)
    world.step()
    world.synchronize()
    qdot = world.download("qdot").reshape(3, 3).astype(np.float64)
    common = (m1 * 1.0 + m2 * -0.5) / (m1 + m2)
    assert list(world.download("pair_count")) == [1, 1, 0] and np.all(world.download("env_status") == 0)
    assert np.abs(qdot[0, 1:] - common).max() < 2e-5
    assert np.abs(qdot[1, 1:] - [-0.2, 0.3]).max() < 1e-6 and np.abs(qdot[2, 1:] - [1.0, -0.5]).max() < 1e-6
    world.close()


def test_rows_of_one_link_and_excluded_rows_never_pair(device):
    state = rail_state([[0.0, 0.05]], [[0.0, 0.0]])
    desc = abi.world_desc(1, 1.0 / 200.0, gravity=(0, 0, 0))
    for template, pairs in ((rails(1, 1, 0.05), 1), (rails(1, 1, 0.05, exclude=True), 0), (rails(1, 1, 0.05, same_link=True), 0)):
        template.max_contacts_per_env = 2
        world = nk.World(device, template, desc)
        world.set_state(state)
        world.step()
        world.synchronize()
        assert world.download("pair_count")[0] == pairs
        world.close()


@pytest.mark.parametrize("shape", ["capsule_lying", "cylinder_standing", "box_on_box"])
def test_supports_carry_the_weight(oracle_py, device, shape):
    """A capsule lying on the plane (two points), a cylinder standing on it (four) and a box on a static box (four):
    the normal impulses add up to the weight, the body stays at rest, and the device agrees with the oracle."""
    mass, radius, half, dt, g = 1.3, 0.04, 0.1, 1.0 / 200.0, 9.81
    if shape == "capsule_lying":
        kind, pose, points = CAPSULE, [0, 0, radius - 1e-3, np.sqrt(0.5), 0, np.sqrt(0.5), 0], 2
    elif shape == "cylinder_standing":
        kind, pose, points = CYLINDER, [0, 0, half - 1e-3, 1, 0, 0, 0], 4
    else:
        kind, pose, points = BOX, [0.02, -0.01, 0.05 - 1e-3, np.cos(0.15), 0, 0, np.sin(0.15)], 4
    t = box_on_slab(mass) if kind == BOX else floating(kind, (radius, half, 0, 0), mass, (0.01, 0.01, 0.01))
    desc = abi.world_desc(1, dt, vel_iters=100)
    world, oracle = nk.World(device, t, desc), oracle_py.OracleWorld(t, desc, threads=1)
    for w in (world, oracle):
        w.set_state(floating_state(pose))
        w.step()
    world.synchronize()
    assert world.download("ucontact_count")[0] == points and world.download("env_status")[0] == 0
    rows = world.download("urows").reshape(-1, ROW_WORDS).view(np.uint32)
    lam = world.download("lambda")[(rows[:, 0] & CONTACT_NORMAL) != 0].astype(np.float64)
    assert len(lam) == points and abs(lam.sum() - mass * g * dt) < 3e-5 * mass
    assert np.abs(world.download("link_velocity").reshape(-1, 6)[0]).max() < 3e-5
    for name in ("lambda", "link_pose"):
        assert relative_error(world.download(name), oracle.download(name)) <= TOL, name
    world.close()
    oracle.close()


def test_single_point_dispatch_gives_the_general_dispatch_its_manifolds(device):
    """A world whose admitted pairs give one point at most runs the narrowphase on its own dispatch of those manifolds.
    The same world with one box added far above everything (its pair with the plane is admitted, so the general dispatch
    runs, and never in reach) must report the same contacts for the pairs both worlds have, bit for bit."""
    E = 256
    cfg = nk.synthetic.config(3, E)
    import copy
    plain = cfg.template
    boxed = copy.deepcopy(plain)
    boxed.add_body(abi.ROLE_PROXY, link=0, kind=BOX, params=SHAPE_PARAMS[BOX], local_pos=(0.0, 0.0, 5.0), contype=1, conaffinity=2,
                   profile=0)
    boxed.max_contacts_per_env = plain.max_contacts_per_env + 1
    results = []
    for template in (plain, boxed):
        world = nk.World(device, template, abi.world_desc(E, cfg.dt, vel_iters=cfg.vel_iters))
        world.set_state(cfg.state())
        for op in ("FkWorldPoses", "SyncLinkBodyPose", "BuildAabbs", "LbvhQueryPairs", "NarrowphasePrimitives"):
            world.op(op)
        world.synchronize()
        S = world.info.contact_slots_per_env
        live = world.download("pair_count")
        pairs = world.download("candidate_pairs").reshape(E, S, 2)
        fields = {name: world.download(name).reshape(E, S, 4, -1) for name in ("ucontact_point", "ucontact_normal", "ucontact_depth",
                                                                              "ucontact_id_feature", "ucontact_id_pair")}
        counts = world.download("ucontact_count").reshape(E, S)
        found = {}
        for e in range(E):
            for s in range(live[e]):
                found[(e, int(pairs[e, s, 0]), int(pairs[e, s, 1]))] = (int(counts[e, s]),) + tuple(fields[n][e, s, 0].tobytes() for n in fields)
        results.append(found)
        world.close()
    plain_found, boxed_found = results
    assert len(plain_found) > 4 * E and sum(v[0] for v in plain_found.values()) > 2 * E, "the batch must hold contacts"
    nb = len(plain.bodies)
    shared = {k: v for k, v in boxed_found.items() if k[1] < nb and k[2] < nb}
    assert shared.keys() == plain_found.keys()
    differing = [k for k in plain_found if plain_found[k][0] != shared[k][0] or (plain_found[k][0] and plain_found[k][1:] != shared[k][1:])]
    assert not differing, f"{len(differing)} pairs differ between the two dispatches, first {differing[:3]}"
