"""Pins of the oracle's leaf functions (CPU only).

Splines: the reference's own object code (oracle/_ref, built from
cubic_spline_set.cpp / cubic_spline.cpp / tools.cpp / zbl.cpp) where present,
and scipy.interpolate.CubicSpline with the reference's own test function
(symmetrix/test/test_cubic_spline_set.py:10-68).  Harmonics: scipy's
sph_harm_y, sum rule, tangency, central differences.  Polynomial: brute-force
monomial sums on the reference's own example monomials
(symmetrix/test/test_multivariate_polynomial.py:12,23).  MLP: numpy closed
form + central differences (symmetrix/test/test_multilayer_perceptron.py).
ZBL: the two known answers of symmetrix/test/test_zbl.py:25,42.
"""
import ctypes as C

import numpy as np
import pytest
from scipy.interpolate import CubicSpline
from scipy.special import sph_harm_y

from oracle import oracle as O


def pd(a):
    return a.ctypes.data_as(C.POINTER(C.c_double))


def _spline_data(n=20, r_cut=5.0):
    r, h = np.linspace(0, r_cut, n, retstep=True)
    fs = [np.sin(r) * r**2 * (r_cut - r) ** 2, np.cos(r) * r**2 * (r_cut - r) ** 2,
          np.sin(r) * np.cos(r) * r**2 * (r_cut - r) ** 2]
    spl = [CubicSpline(r, f) for f in fs]
    vals = np.array(fs)
    ders = np.array([s.derivative()(r) for s in spl])
    return r, h, spl, vals, ders


def test_spline_set_matches_scipy():
    r, h, spl, vals, ders = _spline_data()
    L = O.lib()
    c = np.zeros(4 * 3 * (len(r) - 1))
    L.orc_spline_set_build(C.c_double(h), 3, len(r), pd(vals), pd(ders), pd(c))
    rr = np.linspace(0, 5.0, 1000, endpoint=False)
    v = np.zeros(3); d = np.zeros(3)
    for x in rr:
        L.orc_spline_set_evaluate_derivs(C.c_double(h), 3, pd(c), C.c_double(x), pd(v), pd(d))
        for j in range(3):
            assert v[j] == pytest.approx(float(spl[j](x)), rel=1e-9, abs=1e-9)
            assert d[j] == pytest.approx(float(spl[j].derivative()(x)), rel=1e-8, abs=1e-8)


def test_spline_hermite_identities():
    """Value and derivative are reproduced exactly at the left knot of every interval."""
    r, h, spl, vals, ders = _spline_data()
    L = O.lib()
    c = np.zeros(4 * 3 * (len(r) - 1))
    L.orc_spline_set_build(C.c_double(h), 3, len(r), pd(vals), pd(ders), pd(c))
    v = np.zeros(3); d = np.zeros(3)
    for i in range(len(r) - 1):
        x = h * i * (1 + 1e-15) + 1e-13
        L.orc_spline_set_evaluate_derivs(C.c_double(h), 3, pd(c), C.c_double(x), pd(v), pd(d))
        assert np.allclose(v, vals[:, i], rtol=0, atol=1e-9)
        assert np.allclose(d, ders[:, i], rtol=0, atol=1e-9)


def test_spline_set_matches_reference_object_code():
    R = O.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(0)
    n, ns, h = 33, 7, 0.13
    vals = rng.normal(size=(ns, n)); ders = rng.normal(size=(ns, n))
    L = O.lib()
    c = np.zeros(4 * ns * (n - 1))
    L.orc_spline_set_build(C.c_double(h), ns, n, pd(vals), pd(ders), pd(c))
    s = C.c_void_p(R.ref_spline_set_create(C.c_double(h), ns, n, pd(vals), pd(ders)))
    v = np.zeros(ns); d = np.zeros(ns); v2 = np.zeros(ns); d2 = np.zeros(ns)
    for x in rng.uniform(0, h * (n - 1) * 0.999, size=500):
        L.orc_spline_set_evaluate_derivs(C.c_double(h), ns, pd(c), C.c_double(x), pd(v), pd(d))
        R.ref_spline_set_evaluate_derivs(s, C.c_double(x), pd(v2), pd(d2))
        assert np.array_equal(v, v2) and np.array_equal(d, d2)   # same arithmetic, bit for bit
    R.ref_spline_set_free(s)


def test_single_spline_matches_reference_and_bounds():
    R = O.ref_lib()
    rng = np.random.default_rng(1)
    n, h = 20, 0.25
    vals = rng.normal(size=n); ders = rng.normal(size=n)
    L = O.lib()
    c = np.zeros(4 * (n - 1))
    L.orc_spline_build(C.c_double(h), n, pd(vals), pd(ders), pd(c))
    f = C.c_double(); d = C.c_double()
    # out of bounds where the reference throws (cubic_spline.cpp:19-20)
    assert L.orc_spline_evaluate_deriv(C.c_double(h), n - 1, pd(c), C.c_double(h * (n - 1) + 1e-9), C.byref(f), C.byref(d)) == -1
    assert L.orc_spline_evaluate_deriv(C.c_double(h), n - 1, pd(c), C.c_double(-0.3), C.byref(f), C.byref(d)) in (0, -1)
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    s = C.c_void_p(R.ref_spline_create(C.c_double(h), n, pd(vals), pd(ders)))
    f2 = C.c_double(); d2 = C.c_double()
    for x in rng.uniform(0, h * (n - 1) * 0.999, size=300):
        assert L.orc_spline_evaluate_deriv(C.c_double(h), n - 1, pd(c), C.c_double(x), C.byref(f), C.byref(d)) == 0
        assert R.ref_spline_evaluate_deriv(s, C.c_double(x), C.byref(f2), C.byref(d2)) == 0
        assert f.value == f2.value and d.value == d2.value
    assert R.ref_spline_evaluate_deriv(s, C.c_double(h * (n - 1) + 1e-9), C.byref(f2), C.byref(d2)) == -1
    R.ref_spline_free(s)


# ---------------------------------------------------------------------------
def _oracle_Y(xyz):
    L = O.lib()
    Y = np.zeros(16); dY = np.zeros((3, 16))
    v = np.ascontiguousarray(xyz, dtype=np.float64)
    L.orc_sph_harm_l3(pd(v), pd(Y), pd(dY))
    return Y, dY


def test_harmonics_match_scipy():
    rng = np.random.default_rng(0)
    for _ in range(50):
        v = rng.normal(size=3) * rng.uniform(0.5, 3.0)
        Y, _ = _oracle_Y(v)
        u = v / np.linalg.norm(v)
        th = np.arccos(u[2]); ph = np.arctan2(u[1], u[0])
        for l in range(4):
            for m in range(-l, l + 1):
                if m < 0:
                    ref = np.sqrt(2) * (-1) ** m * sph_harm_y(l, -m, th, ph).imag
                elif m == 0:
                    ref = sph_harm_y(l, 0, th, ph).real
                else:
                    ref = np.sqrt(2) * (-1) ** m * sph_harm_y(l, m, th, ph).real
                assert Y[l * l + l + m] == pytest.approx(ref, abs=1e-13)


def test_harmonics_invariants_and_gradient():
    rng = np.random.default_rng(1)
    for _ in range(20):
        v = rng.normal(size=3) * rng.uniform(0.5, 3.0)
        Y, dY = _oracle_Y(v)
        for l in range(4):   # sum rule of orthonormal harmonics
            assert np.sum(Y[l * l:(l + 1) ** 2] ** 2) == pytest.approx((2 * l + 1) / (4 * np.pi), rel=1e-13)
        assert np.abs(v @ dY).max() < 1e-13            # functions of the direction only
        Ym, _ = _oracle_Y(-v)
        for l in range(4):                              # parity (-1)^l
            assert np.allclose(Ym[l * l:(l + 1) ** 2], (-1) ** l * Y[l * l:(l + 1) ** 2], atol=1e-14)
        h = 1e-6
        for a in range(3):
            e = np.zeros(3); e[a] = h
            fd = (_oracle_Y(v + e)[0] - _oracle_Y(v - e)[0]) / (2 * h)
            assert np.allclose(fd, dY[a], atol=1e-8)


def test_compute_Y_engine_convention():
    """mace.cpp:118-148: harmonics at (z,x,y), times 2 sqrt(pi): l=1 block is sqrt(3) (x,y,z)/r."""
    from tests.helpers import tiny_model
    orc = O.OracleMACE(tiny_model(K=2, L_max=0))
    rng = np.random.default_rng(2)
    xyz = rng.normal(size=(6, 3))
    orc.compute_Y(xyz.reshape(-1))
    Y = orc.Y.reshape(6, 16); G = orc.Y_grad.reshape(6, 3, 16)
    u = xyz / np.linalg.norm(xyz, axis=1, keepdims=True)
    assert np.allclose(Y[:, 0], 1.0)
    assert np.allclose(Y[:, 1:4], np.sqrt(3) * u, atol=1e-14)
    assert np.allclose(Y[:, 4], np.sqrt(15) * u[:, 0] * u[:, 2], atol=1e-14)          # sqrt15 xz
    assert np.allclose(Y[:, 6], np.sqrt(5) * (u[:, 1] ** 2 - 0.5 * (u[:, 0] ** 2 + u[:, 2] ** 2)), atol=1e-14)
    for l in range(4):   # component normalisation
        assert np.allclose(np.sum(Y[:, l * l:(l + 1) ** 2] ** 2, axis=1), 2 * l + 1)
    h = 1e-6
    for a in range(3):
        xp = xyz.copy(); xp[:, a] += h
        xm = xyz.copy(); xm[:, a] -= h
        orc.compute_Y(xp.reshape(-1)); Yp = orc.Y.reshape(6, 16)
        orc.compute_Y(xm.reshape(-1)); Ym = orc.Y.reshape(6, 16)
        assert np.allclose((Yp - Ym) / (2 * h), G[:, a, :], atol=1e-8)


# ---------------------------------------------------------------------------
def _brute_force(coefs, monos, x):
    f = 0.0
    g = np.zeros(len(x))
    for c, m in zip(coefs, monos):
        f += c * np.prod([x[i] for i in m])
        for j in range(len(m)):
            g[m[j]] += c * np.prod([x[m[k]] for k in range(len(m)) if k != j])
    return f, g


@pytest.mark.parametrize("nv,monos", [
    (5, [[0], [0, 1], [1, 1, 2], [0, 1, 2, 4]]),
    (8, [[7], [0, 1], [1, 3], [1, 1, 2], [0, 1, 2, 4], [4, 5, 6, 7]]),
    (6, [[2, 2, 2], [0, 0], [5], [1, 2, 3], [0, 5], [3, 3, 4, 4, 5]]),
])
def test_polynomial_graph_vs_brute_force(nv, monos):
    rng = np.random.default_rng(len(monos))
    coefs = rng.normal(size=len(monos))
    nodes, edges, nc, n_aux = O.build_product_graph(nv, coefs, monos)
    # every non-leaf node is the product of two earlier nodes
    for e, (i0, i1) in enumerate(edges):
        assert i0 < nv + e and i1 < nv + e
        assert sorted(nodes[i0] + nodes[i1]) == sorted(nodes[nv + e])
    # shorter first, then lexicographic
    assert nodes == sorted(nodes, key=lambda t: (len(t), t))
    L = O.lib()
    x = rng.normal(size=nv)
    ed = np.ascontiguousarray(np.array(edges, dtype=np.int32).reshape(-1))
    nv_ = np.zeros(len(nodes)); na_ = np.zeros(len(nodes)); g = np.zeros(nv)
    f = L.orc_poly_evaluate_gradient(nv, len(nodes), ed.ctypes.data_as(C.POINTER(C.c_int)), pd(np.ascontiguousarray(nc)),
                                     pd(x), pd(nv_), pd(na_), pd(g))
    f0, g0 = _brute_force(coefs, monos, x)
    assert f == pytest.approx(f0, rel=1e-12)
    assert np.allclose(g, g0, rtol=1e-12, atol=1e-14)


def test_two_part_partitions_vs_reference():
    counts = [len(O.two_part_partitions(list(range(n)))) for n in range(1, 8)]
    assert counts == [0, 1, 3, 7, 15, 31, 63]          # symmetrix/test/test_tools.py:29-34
    R = O.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    assert [R.ref_num_partitions(n) for n in range(1, 8)] == [1, 2, 5, 15, 52, 203, 877]   # test_tools.py:22-27
    for v in ([0, 1], [1, 1, 2], [0, 1, 2, 4], [3, 3, 4, 4, 5], [0, 2, 5, 7, 9, 11]):
        mine = O.two_part_partitions(v)
        buf = (C.c_int * 4096)()
        arr = (C.c_int * len(v))(*v)
        n = R.ref_two_part_partitions(arr, len(v), buf, 4096)
        assert n == len(mine)
        ref = []
        pos = 0
        for _ in range(n):
            part = []
            for _ in range(2):
                ln = buf[pos]
                part.append(list(buf[pos + 1:pos + 1 + ln]))
                pos += 1 + ln
            ref.append(part)
        if len(mine) <= 16:
            # std::sort on at most 16 equal keys is an insertion sort, hence stable: same order
            assert ref == mine
        else:
            # beyond that the reference's order is whatever libstdc++'s introsort leaves
            # (every key is equal); only the set is defined.  MACE monomials have degree <= 3.
            assert sorted(ref) == sorted(mine)


# ---------------------------------------------------------------------------
def test_mlp_vs_numpy_and_finite_differences():
    rng = np.random.default_rng(3)
    K = 6
    shape = np.array([K, 16, 1], dtype=np.int32)
    W1 = rng.normal(size=(16, K)); W2 = rng.normal(size=16)
    scale = 1.679
    x = rng.normal(size=K)
    L = O.lib()
    ptrs = (C.POINTER(C.c_double) * 2)(pd(W1), pd(W2))
    g = np.zeros(K)
    f = L.orc_mlp_evaluate_gradient(3, shape.ctypes.data_as(C.POINTER(C.c_int)), ptrs, C.c_double(scale), pd(x), pd(g))

    def ref(x):
        hpre = W1 @ x
        return W2 @ (scale * hpre / (1 + np.exp(-hpre)))
    assert f == pytest.approx(ref(x), rel=1e-13)
    h = 1e-6
    fd = np.array([(ref(x + h * np.eye(K)[i]) - ref(x - h * np.eye(K)[i])) / (2 * h) for i in range(K)])
    assert np.allclose(g, fd, atol=1e-8)


def test_zbl_known_answers():
    L = O.lib()
    R = O.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    c = np.array([0.1818, 0.5099, 0.2802, 0.02817]); radii = np.zeros(20); radii[5] = 0.84; radii[10] = 0.58
    z = C.c_void_p(R.ref_zbl_create(C.c_double(0.3), C.c_double(0.4543), pd(c), pd(radii), 20, 6))
    assert R.ref_zbl_envelope(z, C.c_double(1.0), C.c_double(0.84 + 0.58), 6) == pytest.approx(0.4374788794430078, rel=1e-12)
    assert R.ref_zbl_compute(z, 5, 10, C.c_double(1.0)) == pytest.approx(0.3166652764835175, rel=1e-12)

    class Z(C.Structure):
        _fields_ = [("a_exp", C.c_double), ("a_prefactor", C.c_double), ("c", C.c_double * 4),
                    ("radii", C.POINTER(C.c_double)), ("n", C.c_int), ("p", C.c_int)]
    zz = Z(0.3, 0.4543, (C.c_double * 4)(*c), pd(radii), 20, 6)
    f = C.c_double(); d = C.c_double()
    for r in (0.3, 0.7, 1.0, 1.3):
        L.orc_zbl_compute(C.byref(zz), 5, 10, C.c_double(r), C.byref(f), C.byref(d))
        assert f.value == pytest.approx(R.ref_zbl_compute(z, 5, 10, C.c_double(r)), rel=1e-14)
        assert d.value == pytest.approx(R.ref_zbl_compute_gradient(z, 5, 10, C.c_double(r)), rel=1e-13)
    R.ref_zbl_free(z)
