"""The oracle against the committed vectors of the reference's host headers (tests/golden/rowmath_vectors.npz,
written by tests/golden/make_rowmath_vectors.py from oracle/_ref).  Bit-exact: both sides are plain fp32 host code."""
import ctypes as C
import os

import numpy as np
import pytest

from conftest import ROOT

F = C.c_float
sys_path = os.path.join(ROOT, "tests", "golden")


def farr(values):
    return (F * len(values))(*[float(v) for v in values])


@pytest.fixture(scope="module")
def vectors():
    return np.load(os.path.join(sys_path, "rowmath_vectors.npz"), allow_pickle=False)


def same(a, b):
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    return np.array_equal(a.view(np.uint32) | (a == 0) * 0x80000000, b.view(np.uint32) | (b == 0) * 0x80000000)   # -0 == +0


def test_scalar_rows(oracle_py, vectors):
    L = oracle_py.lib()
    for c, expect in zip(vectors["scalar_in"], vectors["scalar_out"]):
        out = (F * 2)()
        L.nko_scalar_impulse(*[F(float(v)) for v in c], out)
        assert same(list(out), expect)


def test_tangent_rows(oracle_py, vectors):
    L = oracle_py.lib()
    for c, expect in zip(vectors["tangent_in"], vectors["tangent_out"]):
        f, cv = (F * 3)(), (F * 6)()
        L.nko_tangent_impulse(farr(c[0:3]), F(float(c[3])), farr(c[4:7]), F(float(c[7])), F(float(c[8])), F(float(c[9])), f, cv)
        assert same(list(f) + list(cv), expect)


def test_relaxation(oracle_py, vectors):
    L = oracle_py.lib()
    for c, expect in zip(vectors["relax_in"], vectors["relax_out"]):
        step, weight, point, res = farr(c[6:9]), F(float(c[9])), farr(c[10:13]), (F * 3)()
        L.nko_relax_contact_impulse(farr(c[0:3]), farr(c[3:6]), step, C.byref(weight), point, res)
        assert same(list(res) + list(step) + [weight.value] + list(point), expect)


def test_cone_argument_and_restart(oracle_py, vectors):
    L = oracle_py.lib()
    L.nko_cone_argument.restype = C.c_float
    L.nko_momentum_restart.restype = C.c_double
    for c, expect in zip(vectors["cone_in"], vectors["cone_out"]):
        assert same([L.nko_cone_argument(*[F(float(v)) for v in c])], [expect])
    for c, expect in zip(vectors["restart_in"], vectors["restart_out"]):
        assert L.nko_momentum_restart(farr(c[0:3]), farr(c[3:6]), farr(c[6:9]), farr(c[9:12])) == expect


def test_manifolds(oracle_py, vectors):
    from golden.make_rowmath_vectors import frame
    L = oracle_py.lib()
    hits = 0
    for i in range(len(vectors["manifold_count"])):
        ka, kb = [int(k) for k in vectors["manifold_kinds"][i]]
        shape, zero = farr(vectors["manifold_params"][i]), farr([0, 0, 0, 0])
        sa, sb = (shape, zero) if kb == 3 else (zero, shape)
        p, n, pe, ke = (F * 12)(), (F * 12)(), (F * 4)(), (C.c_uint64 * 4)()
        count = L.nko_primitive_pair_frames(ka, farr(frame(vectors["manifold_poses"][i, 0])), sa, kb,
                                            farr(frame(vectors["manifold_poses"][i, 1])), sb,
                                            F(float(vectors["manifold_query"][i])), p, n, pe, ke)
        assert count == vectors["manifold_count"][i]
        hits += count > 0
        assert same(list(p)[:3 * count], vectors["manifold_points"][i, :3 * count])
        assert same(list(n)[:3 * count], vectors["manifold_normals"][i, :3 * count])
        assert same(list(pe)[:count], vectors["manifold_penetration"][i, :count])
        assert list(ke)[:count] == list(vectors["manifold_keys"][i, :count])
    assert hits > 100


def test_every_analytic_pair(oracle_py, vectors):
    """Sphere, capsule, box, plane and cylinder pairs of the reference's PrimitivePair, both orders."""
    from golden.make_rowmath_vectors import frame
    L = oracle_py.lib()
    hits = {}
    for i in range(len(vectors["pair_count"])):
        ka, kb = [int(k) for k in vectors["pair_kinds"][i]]
        p, n, pe, ke = (F * 12)(), (F * 12)(), (F * 4)(), (C.c_uint64 * 4)()
        count = L.nko_primitive_pair_frames(ka, farr(frame(vectors["pair_poses"][i, 0])), farr(vectors["pair_params"][i, 0]), kb,
                                            farr(frame(vectors["pair_poses"][i, 1])), farr(vectors["pair_params"][i, 1]),
                                            F(float(vectors["pair_query"][i])), p, n, pe, ke)
        assert count == vectors["pair_count"][i], (ka, kb, i)
        hits[(ka, kb)] = hits.get((ka, kb), 0) + int(count > 0)
        assert same(list(p)[:3 * count], vectors["pair_points"][i, :3 * count]), (ka, kb, i)
        assert same(list(n)[:3 * count], vectors["pair_normals"][i, :3 * count]), (ka, kb, i)
        assert same(list(pe)[:count], vectors["pair_penetration"][i, :count]), (ka, kb, i)
        assert list(ke)[:count] == list(vectors["pair_keys"][i, :count]), (ka, kb, i)
    assert len(hits) == 13 and min(hits.values()) >= 15, hits


def test_compliant_rows_and_elliptic_cone(oracle_py, vectors):
    """The compliant-row terms, their discretisation and the elliptic cone projection (no device counterpart)."""
    L = oracle_py.lib()
    for c, expect in zip(vectors["compliant_in"], vectors["compliant_out"]):
        terms, discrete = (F * 6)(), (F * 3)()
        L.nko_compliant_row_terms(farr(c[0:2]), farr(c[2:7]), F(float(c[7])), F(float(c[8])), F(float(c[9])), F(float(c[10])), F(float(c[11])), int(c[12]), terms)
        L.nko_discretize_compliant_row(F(terms[4]), F(terms[5]), F(terms[1]), F(float(c[11])), discrete)
        assert same(list(terms) + list(discrete), expect)
    for c, expect in zip(vectors["elliptic_in"], vectors["elliptic_out"]):
        impulse, step = (F * 9)(), (F * 3)()
        L.nko_elliptic_impulse(farr(c[0:3]), F(float(c[3])), farr(c[4:7]), farr(c[7:10]), F(float(c[10])), impulse)
        L.nko_elliptic_multiplier_step(farr(c[0:3]), farr(c[11:14]), F(float(c[3])), farr(c[7:10]), step)
        assert same(list(impulse) + list(step), expect)


def test_compose_contact_id_and_roundoff(oracle_py, vectors):
    L = oracle_py.lib()
    L.nko_contact_projection_roundoff.restype = C.c_double
    for c, expect in zip(vectors["compose_in"], vectors["compose_out"]):
        out = (F * 7)()
        L.nko_compose_transform(farr(c[:7]), farr(c[7:]), out)
        assert same(list(out), expect)
    for ids, local, expect in zip(vectors["id_in"], vectors["id_local"], vectors["id_out"]):
        out = (C.c_uint64 * 2)()
        L.nko_make_contact_id(int(ids[0]), int(ids[1]), farr(local[:3]), farr(local[3:]), int(ids[2]), int(ids[3]), out)
        assert list(out) == list(expect)
    for c, expect in zip(vectors["roundoff_in"], vectors["roundoff_out"]):
        assert L.nko_contact_projection_roundoff(farr(c[:3]), farr(c[3:6]), farr(c[6:])) == expect
