"""Writes tests/golden/rowmath_vectors.npz: inputs and outputs of the reference's own host-compilable headers
(augmented_row.hpp, analytical_manifold.hpp, contact_identity.hpp, contact_query.hpp), called through the
extern "C" wrapper built under oracle/_ref.  Runs only where the reference tree is mounted; the vectors it writes
are what travels.  Usage: python tests/golden/make_rowmath_vectors.py"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
import oracle_py  # noqa: E402

F = C.c_float


def farr(values):
    return (F * len(values))(*[float(v) for v in values])


def unit_quat(g):
    q = g.normal(0, 1, 4)
    return q / np.linalg.norm(q)


def frame(pose):
    """cx, cy, cz, t from the closed-form rotation matrix, rounded to float32: the frames the manifold cases use."""
    w, x, y, z = [float(v) for v in np.asarray(pose[3:], np.float32)]
    R = np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                  [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                  [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])
    return np.concatenate([R[:, 0], R[:, 1], R[:, 2], pose[:3]]).astype(np.float32)


# every ordered kind pair PrimitivePair answers analytically beyond those of the first block (sphere 0, capsule 1, box 2,
# plane 3, cylinder 7); box x box twice over, for its many branches
PAIR_ORDERS = [(0, 0), (0, 2), (2, 0), (1, 3), (3, 1), (1, 0), (0, 1), (1, 1), (7, 3), (3, 7), (7, 0), (0, 7), (2, 2), (2, 2)]


def pair_shape(g, kind):
    if kind == 0:
        return [g.uniform(0.02, 0.06), 0, 0, 0]
    if kind in (1, 7):
        return [g.uniform(0.02, 0.05), g.uniform(0.03, 0.1), 0, 0]
    if kind == 2:
        return list(g.uniform(0.02, 0.08, 3)) + [0]
    return [0, 0, 0, 0]


def pair_case(g, ka, kb):
    """Two poses a few centimetres apart, so that about half the cases touch, and the shapes' parameters."""
    pose = np.zeros((2, 7), np.float32)
    for side, kind in enumerate((ka, kb)):
        if kind == 3:
            q = np.array([1, 0, 0, 0]) + g.normal(0, 0.05, 4)
            pose[side] = np.concatenate([[0, 0, g.uniform(-0.01, 0.01)], q / np.linalg.norm(q)])
        else:
            q = unit_quat(g)
            if kind == 7 and g.uniform() < 0.5:   # a cylinder standing on a cap, or nearly
                q = np.array([1, 0, 0, 0]) + g.normal(0, 0.08, 4)
                q /= np.linalg.norm(q)
                if g.uniform() < 0.5:
                    q = np.array([-q[1], q[0], q[3], -q[2]])   # turned over
            if (ka, kb) == (2, 2) and g.uniform() < 0.5:   # boxes nearly aligned, or aligned: faces meet faces
                q = np.array([1, 0, 0, 0]) + g.normal(0, g.choice([0.0, 0.02]), 4)
                q /= np.linalg.norm(q)
            pose[side] = np.concatenate([g.normal(0, 0.04, 3), q])
            if 3 in (ka, kb):
                pose[side, 2] = g.uniform(-0.02, 0.12)
    return pose, np.array([pair_shape(g, ka), pair_shape(g, kb)], np.float32), g.choice([0.0, 1e-3, 5e-4])


def pair_cases(L, g):
    m = 100 * len(PAIR_ORDERS)
    kinds = np.zeros((m, 2), np.uint32)
    poses, params, query = np.zeros((m, 2, 7), np.float32), np.zeros((m, 2, 4), np.float32), np.zeros(m, np.float32)
    count = np.zeros(m, np.uint32)
    points, normals, pen, keys = np.zeros((m, 12), np.float32), np.zeros((m, 12), np.float32), np.zeros((m, 4), np.float32), np.zeros((m, 4), np.uint64)
    for i in range(m):
        ka, kb = PAIR_ORDERS[i % len(PAIR_ORDERS)]
        kinds[i] = (ka, kb)
        poses[i], params[i], query[i] = pair_case(g, ka, kb)
        p, nr, pe, ke = (F * 12)(), (F * 12)(), (F * 4)(), (C.c_uint64 * 4)()
        count[i] = L.ref_primitive_pair_frames(ka, farr(frame(poses[i, 0])), farr(params[i, 0]), kb, farr(frame(poses[i, 1])),
                                               farr(params[i, 1]), F(float(query[i])), p, nr, pe, ke)
        points[i], normals[i], pen[i], keys[i] = list(p), list(nr), list(pe), list(ke)
    return dict(pair_kinds=kinds, pair_poses=poses, pair_params=params, pair_query=query, pair_count=count,
                pair_points=points, pair_normals=normals, pair_penetration=pen, pair_keys=keys)


def main():
    oracle_py.build()
    L = C.CDLL(oracle_py.REF_PATH)
    L.ref_cone_argument.restype = C.c_float
    L.ref_momentum_restart.restype = C.c_double
    L.ref_contact_projection_roundoff.restype = C.c_double
    g = np.random.default_rng(20240607)
    out = {}

    n = 400
    cases, results = np.zeros((n, 6), np.float32), np.zeros((n, 2), np.float32)
    bounds = [(0.0, 3.0e38), (-3.0e38, 3.0e38), (-1.0, 2.0), (1.0, 1.0)]
    for i in range(n):
        lower, upper = bounds[g.integers(0, 4)]
        cases[i] = [g.normal(0, 2), np.exp(g.normal(0, 3)), g.normal(0, 1), g.choice([0.0, 1e-3, 0.1, 5.0]), lower, upper]
        r = (F * 2)()
        L.ref_scalar_impulse(*[F(float(v)) for v in cases[i]], r)
        results[i] = list(r)
    out["scalar_in"], out["scalar_out"] = cases, results

    cases, results = np.zeros((n, 10), np.float32), np.zeros((n, 9), np.float32)
    for i in range(n):
        cases[i] = list(g.normal(0, 1, 3)) + [np.exp(g.normal(0, 2))] + list(g.normal(0, 0.5, 3)) + \
            [g.choice([0.0, -1.0, abs(g.normal(0, 1))]), g.choice([0.0, 0.5, 1.0, 2.0]), g.choice([0.5, 1.0, 1.1e-5])]
        c = cases[i]
        f, cv = (F * 3)(), (F * 6)()
        L.ref_tangent_impulse(farr(c[0:3]), F(float(c[3])), farr(c[4:7]), F(float(c[7])), F(float(c[8])), F(float(c[9])), f, cv)
        results[i] = list(f) + list(cv)
    out["tangent_in"], out["tangent_out"] = cases, results

    cases, results = np.zeros((n, 13), np.float32), np.zeros((n, 10), np.float32)
    for i in range(n):
        cases[i] = list(g.normal(0, 1, 3)) + list(g.normal(0, 1, 3)) + list(g.normal(0, 1, 3)) + [g.choice([0.0, 0.5, 1.0])] + list(g.normal(0, 1, 3))
        c = cases[i]
        step, weight, point, res = farr(c[6:9]), F(float(c[9])), farr(c[10:13]), (F * 3)()
        L.ref_relax_contact_impulse(farr(c[0:3]), farr(c[3:6]), step, C.byref(weight), point, res)
        results[i] = list(res) + list(step) + [weight.value] + list(point)
    out["relax_in"], out["relax_out"] = cases, results

    cases, results = np.zeros((n, 4), np.float32), np.zeros(n, np.float32)
    for i in range(n):
        cases[i] = [g.normal(0, 1), np.exp(g.normal(0, 2)), g.choice([2.0, 0.5, 1.0, 1.1e-5]), g.normal(0, 1)]
        results[i] = L.ref_cone_argument(*[F(float(v)) for v in cases[i]])
    out["cone_in"], out["cone_out"] = cases, results

    cases, results = np.zeros((n, 12), np.float32), np.zeros(n, np.float64)
    for i in range(n):
        cases[i] = list(g.normal(0, 1, 9)) + list(np.abs(g.normal(0, 1, 3)) * g.integers(0, 2, 3))
        c = cases[i]
        results[i] = L.ref_momentum_restart(farr(c[0:3]), farr(c[3:6]), farr(c[6:9]), farr(c[9:12]))
    out["restart_in"], out["restart_out"] = cases, results

    # manifolds: kind pair, two poses, shape params, query -> count, points, normals, penetration, keys
    m = 600
    kinds = np.zeros((m, 2), np.uint32)
    poses, params, query = np.zeros((m, 2, 7), np.float32), np.zeros((m, 4), np.float32), np.zeros(m, np.float32)
    count = np.zeros(m, np.uint32)
    points, normals, pen, keys = np.zeros((m, 12), np.float32), np.zeros((m, 12), np.float32), np.zeros((m, 4), np.float32), np.zeros((m, 4), np.uint64)
    orders = [(0, 3), (3, 0), (2, 3), (3, 2)]
    for i in range(m):
        ka, kb = orders[i % 4]
        shape_pose = np.concatenate([g.normal(0, 0.05, 2), [g.uniform(-0.03, 0.08)], unit_quat(g)])
        pq = np.array([1, 0, 0, 0]) + g.normal(0, 0.05, 4)
        plane_pose = np.concatenate([[0, 0, g.uniform(-0.01, 0.01)], pq / np.linalg.norm(pq)])
        shape = [0.02, 0, 0, 0] if 0 in (ka, kb) else list(g.uniform(0.01, 0.05, 3)) + [0]
        kinds[i], params[i], query[i] = (ka, kb), shape, g.choice([0.0, 1e-3, 5e-4])
        poses[i] = (shape_pose, plane_pose) if kb == 3 else (plane_pose, shape_pose)
        zero = farr([0, 0, 0, 0])
        sa, sb = (farr(shape), zero) if kb == 3 else (zero, farr(shape))
        p, nr, pe, ke = (F * 12)(), (F * 12)(), (F * 4)(), (C.c_uint64 * 4)()
        count[i] = L.ref_primitive_pair_frames(ka, farr(frame(poses[i, 0])), sa, kb, farr(frame(poses[i, 1])), sb,
                                               F(float(query[i])), p, nr, pe, ke)
        points[i], normals[i], pen[i], keys[i] = list(p), list(nr), list(pe), list(ke)
    out.update(manifold_kinds=kinds, manifold_poses=poses, manifold_params=params, manifold_query=query,
               manifold_count=count, manifold_points=points, manifold_normals=normals, manifold_penetration=pen,
               manifold_keys=keys)

    cases, results = np.zeros((n, 14), np.float32), np.zeros((n, 7), np.float32)
    for i in range(n):
        cases[i] = list(g.normal(0, 1, 3)) + list(unit_quat(g)) + list(g.normal(0, 1, 3)) + list(unit_quat(g))
        r = (F * 7)()
        L.ref_compose_transform(farr(cases[i, :7]), farr(cases[i, 7:]), r)
        results[i] = list(r)
    out["compose_in"], out["compose_out"] = cases, results

    ids, locals_, results = np.zeros((n, 4), np.uint32), np.zeros((n, 6), np.float32), np.zeros((n, 2), np.uint64)
    for i in range(n):
        a = int(g.integers(0, 100))
        ids[i] = [a, a + 1 + int(g.integers(0, 100)), g.choice([0xFFFFFFFF, 0, 3, 7]), g.integers(0, 4)]
        locals_[i] = g.normal(0, 0.3, 6)
        r = (C.c_uint64 * 2)()
        L.ref_make_contact_id(int(ids[i, 0]), int(ids[i, 1]), farr(locals_[i, :3]), farr(locals_[i, 3:]), farr([0, 0, 1]),
                              int(ids[i, 2]), int(ids[i, 3]), r)
        results[i] = list(r)
    out["id_in"], out["id_local"], out["id_out"] = ids, locals_, results

    cases, results = np.zeros((n, 9), np.float32), np.zeros(n, np.float64)
    for i in range(n):
        cases[i] = g.normal(0, 1, 9)
        results[i] = L.ref_contact_projection_roundoff(farr(cases[i, :3]), farr(cases[i, 3:6]), farr(cases[i, 6:]))
    out["roundoff_in"], out["roundoff_out"] = cases, results

    out.update(pair_cases(L, g))

    # compliant-row terms and their discretisation: solref[2], solimp[5], pos_imp, pos_aref, vel, invweight, dt, refsafe
    n = 300
    cases, results = np.zeros((n, 13), np.float32), np.zeros((n, 9), np.float32)
    for i in range(n):
        cases[i] = [g.choice([0.02, 0.005, -50.0, 0.1]), g.choice([1.0, 0.5, -10.0]), g.uniform(0.5, 0.95), g.uniform(0.9, 0.999),
                    g.choice([0.001, 0.01]), g.uniform(0.2, 0.8), g.choice([1.0, 2.0, 3.0]), -abs(g.normal(0, 0.002)), g.normal(0, 0.002),
                    g.normal(0, 0.5), g.uniform(0.1, 5), g.choice([0.005, 0.002]), g.integers(0, 2)]
        c = cases[i]
        terms, discrete = (F * 6)(), (F * 3)()
        L.ref_compliant_row_terms(farr(c[0:2]), farr(c[2:7]), F(float(c[7])), F(float(c[8])), F(float(c[9])), F(float(c[10])), F(float(c[11])), int(c[12]), terms)
        L.ref_discretize_row(F(terms[4]), F(terms[5]), F(terms[1]), F(float(c[11])), discrete)
        results[i] = list(terms) + list(discrete)
    out["compliant_in"], out["compliant_out"] = cases, results

    # elliptic cone: dual[3], cap, residual[3], compliance[3], mu, next[3] -> impulse[3], curvature[6], multiplier step[3]
    cases, results = np.zeros((n, 14), np.float32), np.zeros((n, 12), np.float32)
    for i in range(n):
        cases[i] = list(g.normal(0, 1, 3)) + [np.exp(g.normal(0, 2))] + list(g.normal(0, 1, 3)) + list(np.exp(g.normal(-3, 2, 3))) + [g.uniform(0.1, 1.5)] + list(g.normal(0, 1, 3))
        c = cases[i]
        impulse, step = (F * 9)(), (F * 3)()
        L.ref_elliptic_impulse(farr(c[0:3]), F(float(c[3])), farr(c[4:7]), farr(c[7:10]), F(float(c[10])), impulse)
        L.ref_elliptic_multiplier_step(farr(c[0:3]), farr(c[11:14]), F(float(c[3])), farr(c[7:10]), step)
        results[i] = list(impulse) + list(step)
    out["elliptic_in"], out["elliptic_out"] = cases, results

    np.savez_compressed(os.path.join(HERE, "rowmath_vectors.npz"), **out)
    print("wrote", os.path.join(HERE, "rowmath_vectors.npz"))


if __name__ == "__main__":
    main()
