"""Pins of the oracle's row math and contact geometry against the reference's own host headers (oracle/_ref) and
the known answers of the reference's tests/math/test_contact_tangent.cpp."""
import ctypes as C

import numpy as np
import pytest

F = C.c_float


def farr(values):
    return (F * len(values))(*[float(v) for v in values])


def test_scalar_impulse_matches_reference(oracle_py, ref_lib):
    L, g = oracle_py.lib(), np.random.default_rng(1)
    for _ in range(2000):
        dual, residual = g.normal(0, 2), g.normal(0, 1)
        rho = float(np.exp(g.normal(0, 3)))
        compliance = float(g.choice([0.0, 1e-3, 0.1, 5.0]))
        lower, upper = g.choice([(0.0, 3.4e38), (-3.4e38, 3.4e38), (-1.0, 2.0), (1.0, 1.0)])
        a, b = (F * 2)(), (F * 2)()
        L.nko_scalar_impulse(F(dual), F(rho), F(residual), F(compliance), F(lower), F(upper), a)
        ref_lib.ref_scalar_impulse(F(dual), F(rho), F(residual), F(compliance), F(lower), F(upper), b)
        assert list(a) == list(b)


def test_tangent_impulse_matches_reference_bitwise(oracle_py, ref_lib):
    L, g = oracle_py.lib(), np.random.default_rng(2)
    for _ in range(3000):
        dual, residual = farr(g.normal(0, 1, 3)), farr(g.normal(0, 0.5, 3))
        rho = float(np.exp(g.normal(0, 2)))
        normal = float(g.choice([0.0, -1.0, abs(g.normal(0, 1))]))
        mu1, mu2 = float(g.choice([0.0, 0.5, 1.0, 2.0])), float(g.choice([0.5, 1.0, 1.1e-5]))
        fa, ca, fb, cb = (F * 3)(), (F * 6)(), (F * 3)(), (F * 6)()
        L.nko_tangent_impulse(dual, F(rho), residual, F(normal), F(mu1), F(mu2), fa, ca)
        ref_lib.ref_tangent_impulse(dual, F(rho), residual, F(normal), F(mu1), F(mu2), fb, cb)
        assert list(fa) == list(fb) and list(ca) == list(cb)


def test_relaxation_matches_reference_and_known_root(oracle_py, ref_lib):
    L, g = oracle_py.lib(), np.random.default_rng(3)
    for _ in range(500):
        sa, wa, pa = farr(g.normal(0, 1, 3)), F(float(g.choice([0.0, 0.5, 1.0]))), farr(g.normal(0, 1, 3))
        sb, wb, pb = farr(list(sa)), F(wa.value), farr(list(pa))
        dual, nxt = farr(g.normal(0, 1, 3)), farr(g.normal(0, 1, 3))
        oa, ob = (F * 3)(), (F * 3)()
        L.nko_relax_contact_impulse(dual, nxt, sa, C.byref(wa), pa, oa)
        ref_lib.ref_relax_contact_impulse(dual, nxt, sb, C.byref(wb), pb, ob)
        assert list(oa) == list(ob) and wa.value == wb.value and list(sa) == list(sb) and list(pa) == list(pb)
    # tests/math/test_contact_tangent.cpp:22-38: the secant finds the linear root with weight 1/3
    for beta in (0.0, 0.5):
        step, weight, point = farr([0, 0, 0]), F(0.0), farr([0, 0, 0])
        first = (F * 3)()
        L.nko_relax_contact_impulse(farr([10, 1, 0]), farr([10, -2, 0]), step, C.byref(weight), point, first)
        p = [first[i] + (first[i] - [10, 1, 0][i]) * beta for i in range(3)]
        root = (F * 3)()
        L.nko_relax_contact_impulse(farr(p), farr([10, -2 * np.float32(p[1]), 0]), step, C.byref(weight), point, root)
        assert root[0] == 10.0 and abs(root[1]) < 5e-7 and root[2] == 0.0
        assert abs(weight.value - 1.0 / 3.0) < 1e-7


def test_friction_known_answers(oracle_py):
    # tests/math/test_contact_tangent.cpp:40-63, 65-90: collapsed cones respond with zero; inside the cone the
    # curvature is rho and the impulse follows the residual; outside it saturates at mu * normal.
    L = oracle_py.lib()
    for mu in (1.1e-5, 0.5, 2.0):
        f, c = (F * 3)(), (F * 6)()
        L.nko_tangent_impulse(farr([0, 0, 0]), F(10.0), farr([0, 0.1, -0.1]), F(0.0), F(mu), F(mu), f, c)
        assert list(f) == [0, 0, 0] and list(c) == [0] * 6
        normal, rho = 0.05, 10.0
        radius = mu * normal
        for fraction in (0.25, 2.0):
            residual = farr([0, 0.6 * fraction * radius / rho, 0.8 * fraction * radius / rho])
            L.nko_tangent_impulse(farr([0, 0, 0]), F(rho), residual, F(normal), F(mu), F(mu), f, c)
            magnitude = radius * min(fraction, 1.0)
            assert abs(f[1] - 0.6 * magnitude) <= radius * 2e-6 and abs(f[2] - 0.8 * magnitude) <= radius * 2e-6
            if fraction < 1.0:
                assert abs(c[1] - rho) <= 2e-5 and abs(c[2] - rho) <= 2e-5


def rotation_matrix(q):
    w, x, y, z = [float(v) for v in q]
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


def test_prim_frame_is_the_rotation_matrix(oracle_py):
    # The pipeline bakes frames in a device-only helper (narrowphase_prims.cu:34-46), out of reach of the host
    # build of the reference, so the frame is pinned by the closed form: columns of R(q), then the position.
    L, g = oracle_py.lib(), np.random.default_rng(9)
    for _ in range(300):
        q = g.normal(0, 1, 4)
        q /= np.linalg.norm(q)
        pose = np.concatenate([g.normal(0, 1, 3), q]).astype(np.float32)
        frame = (F * 12)()
        L.nko_prim_frame(farr(pose), frame)
        f = np.array(frame).reshape(4, 3)
        assert np.abs(f[:3].T - rotation_matrix(pose[3:])).max() < 5e-7
        assert list(f[3]) == list(pose[:3])


@pytest.mark.parametrize("kinds", [(0, 3), (3, 0), (2, 3), (3, 2)])
def test_manifolds_match_reference_bitwise(oracle_py, ref_lib, kinds):
    L, g = oracle_py.lib(), np.random.default_rng(10 + kinds[0])
    hits = 0
    for _ in range(1500):
        q = g.normal(0, 1, 4)
        q /= np.linalg.norm(q)
        shape_pose = farr(list(g.normal(0, 0.05, 2)) + [g.uniform(-0.03, 0.08)] + list(q))
        pq = np.array([1, 0, 0, 0]) + g.normal(0, 0.05, 4)
        pq /= np.linalg.norm(pq)
        plane_pose = farr([0, 0, g.uniform(-0.01, 0.01)] + list(pq))
        params = farr([0.02, 0, 0, 0]) if 0 in kinds else farr(list(g.uniform(0.01, 0.05, 3)) + [0])
        zero = farr([0, 0, 0, 0])
        query = float(g.choice([0.0, 1e-3, 5e-4]))
        shape_frame, plane_frame = (F * 12)(), (F * 12)()
        L.nko_prim_frame(shape_pose, shape_frame)
        L.nko_prim_frame(plane_pose, plane_frame)
        pts, nrm, pen, keys = (F * 12)(), (F * 12)(), (F * 4)(), (C.c_uint64 * 4)()
        ka, kb = kinds
        pa, pb = (shape_frame, plane_frame) if kb == 3 else (plane_frame, shape_frame)
        sa, sb = (params, zero) if kb == 3 else (zero, params)
        n_ref = ref_lib.ref_primitive_pair_frames(ka, pa, sa, kb, pb, sb, F(query), pts, nrm, pen, keys)
        opts, onrm, open_, feat = (F * 12)(), (F * 3)(), (F * 4)(), (C.c_uint32 * 4)()
        if 0 in kinds:
            n = L.nko_sphere_plane(shape_pose, F(0.02), plane_pose, F(query), opts, onrm, open_)
        else:
            n = L.nko_box_plane(shape_pose, params, plane_pose, F(query), opts, onrm, open_, feat)
        assert n == n_ref
        hits += n > 0
        # the oracle's helpers report the normal of the (shape, plane) order; the reference flips it for (plane, shape)
        sign = 1.0 if kb == 3 else -1.0
        for i in range(n):
            assert [opts[3 * i + k] for k in range(3)] == [pts[3 * i + k] for k in range(3)]
            assert [sign * onrm[k] for k in range(3)] == [nrm[3 * i + k] for k in range(3)]
            assert open_[i] == pen[i]
            if 2 in kinds:
                assert feat[i] == keys[i]
    assert hits > 200


def test_constants_and_small_helpers_match_reference(oracle_py, ref_lib):
    assert ref_lib.ref_rigid_contact_query_margin() == np.float32(0.0005)
    assert ref_lib.ref_contact_query_reach(F(0.0), F(0.0)) == np.float32(0.02)
    out = (F * 4)()
    ref_lib.ref_discretize_zero_row(F(1.0 / 200.0), out)
    assert out[0] == 0.0 and out[1] == 0.0          # the speculative rows' R and bias the oracle hard-codes
    for a, b in ((0.8, 0.8), (1.0, 0.5), (0.5, 1.0)):
        ref_lib.ref_merge_friction(F(a), F(b), out)
        assert out[0] == np.float32(max(a, b)) and out[2] == 3.0 and out[3] == 0.0   # max mixing, condim 3, margin 0
    # filter used by the oracle's pair enumeration
    assert ref_lib.ref_shape_filter_admits(1, 2, 0, 2, 1, 0) == 1
    assert ref_lib.ref_shape_filter_admits(1, 2, 0, 1, 2, 0) == 0
    assert ref_lib.ref_shape_filter_admits(0, 0, 0, 2, 1, 0) == 0


def test_tangent_basis_is_orthonormal_and_right_handed(oracle_py):
    L, g = oracle_py.lib(), np.random.default_rng(5)
    for _ in range(200):
        n = g.normal(0, 1, 3)
        n /= np.linalg.norm(n)
        t1, t2 = (F * 3)(), (F * 3)()
        L.nko_contact_tangent_basis(farr(n), t1, t2)
        a, b = np.array(t1), np.array(t2)
        assert abs(a @ n) < 1e-6 and abs(b @ n) < 1e-6 and abs(a @ b) < 1e-6
        assert abs(np.linalg.norm(a) - 1) < 1e-6 and np.allclose(np.cross(n, a), b, atol=1e-6)


def test_cone_argument_and_momentum_restart_match_reference(oracle_py, ref_lib):
    L, g = oracle_py.lib(), np.random.default_rng(6)
    L.nko_cone_argument.restype = C.c_float
    L.nko_momentum_restart.restype = C.c_double
    for _ in range(2000):
        dual, residual = float(g.normal(0, 1)), float(g.normal(0, 1))
        rho, mu = float(np.exp(g.normal(0, 2))), float(g.choice([2.0, 0.5, 1.0, 1.1e-5]))   # callers never pass mu = 0
        assert L.nko_cone_argument(F(dual), F(rho), F(mu), F(residual)) == ref_lib.ref_cone_argument(F(dual), F(rho), F(mu), F(residual))
        v = [farr(g.normal(0, 1, 3)) for _ in range(3)] + [farr(np.abs(g.normal(0, 1, 3)) * g.integers(0, 2, 3))]
        assert L.nko_momentum_restart(*v) == ref_lib.ref_momentum_restart(*v)
    # tests/math/test_contact_tangent.cpp:92-104: sign of the restart test in the scaled metric
    scale = farr([2, 4, 0])
    assert L.nko_momentum_restart(farr([1, 2, 0]), farr([0.8, 1.8, 0]), farr([1.1, 2.1, 0]), scale) < 0
    assert L.nko_momentum_restart(farr([0.4, 1.4, 0]), farr([0.5, 1.5, 0]), farr([0.8, 1.8, 0]), scale) > 0
    assert L.nko_momentum_restart(farr([1, 2, 0]), farr([1, 2, 0]), farr([1.1, 2.1, 0]), scale) == 0


def test_contact_query_helpers_match_reference(oracle_py, ref_lib):
    L, g = oracle_py.lib(), np.random.default_rng(7)
    L.nko_contact_projection_roundoff.restype = C.c_double
    L.nko_contact_query_reach.restype = C.c_float
    L.nko_contact_motion_radius.restype = C.c_float
    for _ in range(1000):
        s, e, a = farr(g.normal(0, 1, 3)), farr(g.normal(0, 1, 3)), farr(g.normal(0, 1, 3))
        assert L.nko_contact_projection_roundoff(s, e, a) == ref_lib.ref_contact_projection_roundoff(s, e, a)
        t, m = F(abs(g.normal(0, 0.01))), F(abs(g.normal(0, 0.01)))
        assert L.nko_contact_query_reach(t, m) == ref_lib.ref_contact_query_reach(t, m)
        args = [F(abs(g.normal(0, 0.01))), F(1.0 / g.integers(60, 1000)), F(abs(g.normal())), F(abs(g.normal())), F(0.9)]
        assert L.nko_contact_motion_radius(*args) == ref_lib.ref_contact_motion_radius(*args)
        bits = [int(x) for x in g.integers(0, 4, 6)]
        assert L.nko_shape_filter_admits(*bits) == ref_lib.ref_shape_filter_admits(*bits)


def test_compose_transform_matches_reference_bitwise(oracle_py, ref_lib):
    L, g = oracle_py.lib(), np.random.default_rng(8)
    for _ in range(2000):
        poses = []
        for _k in range(2):
            q = g.normal(0, 1, 4)
            q /= np.linalg.norm(q)
            poses.append(farr(list(g.normal(0, 1, 3)) + list(q)))
        a, b = (F * 7)(), (F * 7)()
        L.nko_compose_transform(poses[0], poses[1], a)
        ref_lib.ref_compose_transform(poses[0], poses[1], b)
        assert list(a) == list(b)


def test_contact_id_matches_reference(oracle_py, ref_lib):
    L, g = oracle_py.lib(), np.random.default_rng(11)
    for _ in range(2000):
        a = int(g.integers(0, 100))
        b = a + 1 + int(g.integers(0, 100))
        la, lb, n = farr(g.normal(0, 0.3, 3)), farr(g.normal(0, 0.3, 3)), farr([0, 0, 1])
        feature = int(g.choice([0xFFFFFFFF, 0, 3, 7]))
        slot = int(g.integers(0, 4))
        x, y = (C.c_uint64 * 2)(), (C.c_uint64 * 2)()
        L.nko_make_contact_id(a, b, la, lb, feature, slot, x)
        ref_lib.ref_make_contact_id(a, b, la, lb, n, feature, slot, y)
        assert list(x) == list(y)


# the hand-evaluated table of tests/constraint/test_solref_solimp.cpp: solref, solimp, pos_imp, pos_aref, vel, invweight, dt,
# then the expected k, b, imp, D, R, aref
COMPLIANT_TABLE = [
    ((0.02, 1.0), (0.9, 0.95, 0.001, 0.5, 2.0), -0.001, -0.001, 0.0, 1.0, 0.005, (2770.0835, 105.26316, 0.95, 18.999996, 0.05263159, 2.6315794)),
    ((0.02, 1.0), (0.9, 0.95, 0.001, 0.5, 2.0), -0.0003, -0.0003, -0.1, 1.0, 0.005, (2770.0835, 105.26316, 0.909, 9.989008, 0.10011004, 11.281718)),
    ((0.02, 1.0), (0.9, 0.95, 0.001, 0.5, 2.0), -0.0007, -0.0007, 0.2, 1.0, 0.005, (2770.0835, 105.26316, 0.941, 15.949148, 0.06269927, -19.22798)),
    ((0.02, 1.0), (0.9, 0.95, 0.001, 0.5, 2.0), -0.002, -0.002, 0.5, 2.0, 0.005, (2770.0835, 105.26316, 0.95, 9.499998, 0.10526318, -47.368423)),
    ((0.02, 1.0), (0.9, 0.95, 0.001, 0.5, 1.0), -0.0004, -0.0004, 0.0, 1.0, 0.005, (2770.0835, 105.26316, 0.92, 11.499993, 0.086956576, 1.0193907)),
    ((-50.0, 1.0), (0.9, 0.95, 0.001, 0.5, 2.0), -0.0005, -0.0005, 0.3, 1.0, 0.005, (55.401665, 210.52632, 0.92499995, 12.333324, 0.08108114, -63.132275)),
    ((0.02, -10.0), (0.9, 0.95, 0.001, 0.5, 2.0), -0.0005, -0.0005, 0.4, 1.0, 0.005, (27.700834, 10.526316, 0.92499995, 12.333324, 0.08108114, -4.197715)),
    ((0.005, 1.0), (0.9, 0.95, 0.001, 0.5, 2.0), -0.0006, -0.0006, 0.0, 1.0, 0.01, (2770.0835, 105.26316, 0.934, 14.151519, 0.070663795, 1.5523549)),
    ((0.02, 1.0), (0.9, 0.95, 0.001, 0.5, 2.0), -1.0e-7, -1.0e-7, 0.0, 1.0, 0.005, (2770.0835, 105.26316, 0.9, 8.999997, 0.11111115, 0.00024930752)),
]


def test_compliant_row_terms_match_the_hand_evaluated_table(oracle_py):
    """ComputeCompliantRowTerms against the reference test's own table, with that test's tolerances; R D = 1 and a deeper
    contact is stiffer (its DAndRNotSwapped case)."""
    L = oracle_py.lib()
    for solref, solimp, pos_imp, pos_aref, vel, invweight, dt, expect in COMPLIANT_TABLE:
        out = (F * 6)()
        L.nko_compliant_row_terms(farr(solref), farr(solimp), F(pos_imp), F(pos_aref), F(vel), F(invweight), F(dt), 1, out)
        k, b, imp, D, R, aref = list(out)
        assert abs(k - expect[0]) <= 1e-3 * (1 + abs(expect[0])) and abs(b - expect[1]) <= 1e-3 * (1 + abs(expect[1]))
        assert abs(imp - expect[2]) <= 1e-5 and abs(D - expect[3]) <= 1e-3 * (1 + abs(expect[3])) and abs(R - expect[4]) <= 1e-5
        assert abs(aref - expect[5]) <= 1e-3 * (1 + abs(expect[5]))
    shallow, deep = (F * 6)(), (F * 6)()
    default = (farr((0.02, 1.0)), farr((0.9, 0.95, 0.001, 0.5, 2.0)))
    L.nko_compliant_row_terms(*default, F(-0.0002), F(-0.0002), F(0.0), F(1.0), F(0.005), 1, shallow)
    L.nko_compliant_row_terms(*default, F(-0.0009), F(-0.0009), F(0.0), F(1.0), F(0.005), 1, deep)
    assert abs(shallow[3] * shallow[4] - 1) < 1e-4 and abs(deep[3] * deep[4] - 1) < 1e-4
    assert deep[2] > shallow[2] and deep[4] < shallow[4] and deep[3] > shallow[3]


def test_compliant_rows_and_elliptic_cone_match_reference_bitwise(oracle_py, ref_lib):
    L, g = oracle_py.lib(), np.random.default_rng(12)
    for _ in range(1500):
        solref = (float(g.choice([0.02, 0.005, -50.0, 0.1])), float(g.choice([1.0, 0.5, -10.0])))
        solimp = (g.uniform(0.5, 0.95), g.uniform(0.9, 0.999), float(g.choice([0.001, 0.01])), g.uniform(0.2, 0.8), float(g.choice([1.0, 2.0, 3.0])))
        args = (farr(solref), farr(solimp), F(-abs(g.normal(0, 0.002))), F(g.normal(0, 0.002)), F(g.normal(0, 0.5)), F(g.uniform(0.1, 5)),
                F(float(g.choice([0.005, 0.002]))), int(g.integers(0, 2)))
        a, b = (F * 6)(), (F * 6)()
        L.nko_compliant_row_terms(*args, a)
        ref_lib.ref_compliant_row_terms(*args, b)
        assert list(a) == list(b)
        c, d = (F * 3)(), (F * 3)()
        L.nko_discretize_compliant_row(F(a[4]), F(a[5]), F(a[1]), args[6], c)
        ref_lib.ref_discretize_row(F(a[4]), F(a[5]), F(a[1]), args[6], d)
        assert list(c) == list(d)
    inside = projected = polar = 0
    for _ in range(3000):
        dual, residual = farr(g.normal(0, 1, 3)), farr(g.normal(0, 1, 3))
        cap, mu = F(float(np.exp(g.normal(0, 2)))), F(g.uniform(0.1, 1.5))
        compliance = farr(np.exp(g.normal(-3, 2, 3)))
        a, b = (F * 9)(), (F * 9)()
        L.nko_elliptic_impulse(dual, cap, residual, compliance, mu, a)
        ref_lib.ref_elliptic_impulse(dual, cap, residual, compliance, mu, b)
        assert list(a) == list(b)
        inside += a[6] == 0 and a[3] != 0
        polar += not any(a)
        projected += a[6] != 0 or a[7] != 0
        nxt, c, d = farr(g.normal(0, 1, 3)), (F * 3)(), (F * 3)()
        L.nko_elliptic_multiplier_step(dual, nxt, cap, compliance, c)
        ref_lib.ref_elliptic_multiplier_step(dual, nxt, cap, compliance, d)
        assert list(c) == list(d)
    assert inside > 300 and projected > 300 and polar > 100
