"""Index conventions of the oracle's forward stages, pinned by hand-made models (CPU only).

Finite differences and invariances cannot see a weight matrix that is read transposed in the
forward stage and in its adjoint alike, a wrong pair-table index, a sender/receiver mix-up or a
permuted polynomial map: with random weights all of those give another valid model.  Every test
here uses weights whose effect the reference's own call arguments fix (the BLAS layout and
transposition flags, the index expressions of libsymmetrix/source/mace.cpp), so the expected
output is a plain selection of inputs and not a re-evaluation of the oracle's formula.  Each
docstring names the mistake the test fails under; where it is cheap the test also asserts that
the mistaken variant of the expectation does NOT match (negative control).
"""
import copy

import numpy as np
import pytest

from oracle.oracle import OracleMACE
from tests import helpers as H

K = 5  # channels; odd and != 16 so that a [16][K] / [K][16] mix-up cannot go unnoticed


def _system(model, n=9, seed=11):
    pos, cell, sp = H.small_system(n, seed=seed)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    assert len(set(ea["node_types"].tolist())) == 3 and ea["num_neigh"].min() > 0
    return nl, ea


def _pairs(T):
    """Unordered species pairs in the order the model file stores their tables: row-major upper
    triangle (extract_mace_data.py:150-153)."""
    return [(a, b) for a in range(T) for b in range(a, T)]


def _receiver_of_edge(ea):
    return np.repeat(np.arange(ea["num_nodes"]), ea["num_neigh"])


def _elementary(rows, cols, r, c):
    E = np.zeros((rows, cols))
    E[r, c] = 1.0
    return E.ravel().tolist()


@pytest.fixture(scope="module", params=[0, 1, 2], ids=["Lmax0", "Lmax1", "Lmax2"])
def base(request):
    return H.tiny_model(K=K, L_max=request.param, n_pts=24, seed=5)


# ------------------------------------------------------------------------------------------------
# pair tables (mace.cpp:81-83, 107-109)
@pytest.mark.parametrize("T", [3, 4])
def test_pair_table_index_is_the_upper_triangle_position(T):
    """Each pair's table is the constant (1 + its position in the file's pair list), so R0 and R1
    of an edge must read that constant for the unordered pair of its end species.  Fails if
    pair_index enumerates the triangle differently (e.g. a*T+b, or the lower triangle) or is not
    symmetric in (receiver, sender)."""
    Z = [1, 6, 8, 7][:T]
    model = H.tiny_model(K=K, L_max=1, T=Z, n_pts=24, seed=5)
    pairs = _pairs(T)
    for which in (0, 1):
        v = np.asarray(model[f"radial_spline_values_{which}"])
        for p in range(len(pairs)):
            v[p] = 1.0 + p
        model[f"radial_spline_values_{which}"] = v.tolist()
        model[f"radial_spline_derivs_{which}"] = np.zeros_like(v).tolist()
    orc = OracleMACE(model)
    rng = np.random.default_rng(0)
    nt = np.array([a for a in range(T) for _ in range(T)], dtype=np.int32)      # receivers: every species T times
    nn = np.ones(T * T, dtype=np.int32)
    nty = np.array([b for _ in range(T) for b in range(T)], dtype=np.int32)      # one sender of every species each
    r = rng.uniform(0.5, model["r_cut"] - 0.2, size=T * T)
    geo = (T * T, nt, nn, nty, r)
    orc.compute_R0(*geo); orc.compute_R1(*geo)
    want = np.array([1.0 + pairs.index((min(a, b), max(a, b))) for a, b in zip(nt, nty)])
    R0 = orc.R0.reshape(T * T, -1); R1 = orc.R1.reshape(T * T, -1)
    assert R0.shape[1] == 4 * K and R1.shape[1] == len(model["Phi1_l"]) * K
    assert np.allclose(R0, want[:, None], rtol=0, atol=1e-13)
    assert np.allclose(R1, want[:, None], rtol=0, atol=1e-13)
    wrong = np.array([1.0 + (a * T + b) % len(pairs) for a, b in zip(nt, nty)])
    assert not np.allclose(R0[:, 0], wrong)


def test_radial_function_index_is_l_major_channel_minor(base):
    """R0[ij][l*K+k] is spline number l*K+k of the table (mace.cpp:167), R1[ij][path*K+k] likewise
    (mace.cpp:472): at the midpoint of a knot interval the Hermite cubic is
    (v0+v1)/2 + h (d0-d1)/8 of that function's own nodal values.  Fails if the oracle reads the
    table as [n_pts][functions] or [k][l]."""
    model = base
    orc = OracleMACE(model)
    h = model["radial_spline_h"]
    n = 7
    r = np.array([(n + 0.5) * h])
    nt = np.array([1], dtype=np.int32); nty = np.array([2], dtype=np.int32)
    p = _pairs(3).index((1, 2))
    for which, name in ((0, "R0"), (1, "R1")):
        getattr(orc, f"compute_{name}")(1, nt, np.array([1], dtype=np.int32), nty, r)
        v = np.asarray(model[f"radial_spline_values_{which}"])[p]   # [functions][n_pts]
        d = np.asarray(model[f"radial_spline_derivs_{which}"])[p]
        want = 0.5 * (v[:, n] + v[:, n + 1]) + h * (d[:, n] - d[:, n + 1]) / 8.0
        got = getattr(orc, name)
        assert np.allclose(got, want, rtol=1e-12, atol=1e-14)
        dwant = 1.5 * (v[:, n + 1] - v[:, n]) / h - 0.25 * (d[:, n] + d[:, n + 1])
        assert np.allclose(getattr(orc, name + "_deriv"), dwant, rtol=1e-11, atol=1e-13)


# ------------------------------------------------------------------------------------------------
# layer 0 (mace.cpp:150-201)
def test_H0_weights_belong_to_the_sender_species(base):
    """Constant radial tables (= 1) and H0[t][k] = (t+1)(k+1): the l = 0 row of Phi0 (Y_00 = 1) is
    then (k+1) * sum over the receiver's neighbours of (sender species + 1), mace.cpp:165.  With
    identity A0 weights A0 = Phi0.  Fails if H0 is indexed by the receiver's species."""
    model = copy.deepcopy(base)
    for which in (0, 1):
        v = np.ones_like(np.asarray(model[f"radial_spline_values_{which}"]))
        model[f"radial_spline_values_{which}"] = v.tolist()
        model[f"radial_spline_derivs_{which}"] = (0 * v).tolist()
    model["H0_weights"] = np.outer(np.arange(1, 4), np.arange(1, K + 1)).ravel().tolist()
    model["A0_weights"] = [[np.eye(K).ravel().tolist() for _ in range(4)] for _ in range(3)]
    orc = OracleMACE(model)
    nl, ea = _system(model)
    N = ea["num_nodes"]
    geo = (N, ea["node_types"], ea["num_neigh"], ea["neigh_types"])
    orc.compute_Y(ea["xyz"]); orc.compute_R0(*geo, ea["r"]); orc.compute_A0(*geo)
    A0 = orc.A0.reshape(N, 16, K)
    recv = _receiver_of_edge(ea)
    s = np.bincount(recv, weights=ea["neigh_types"] + 1.0, minlength=N)
    assert np.allclose(A0[:, 0, :], s[:, None] * np.arange(1, K + 1)[None, :], rtol=1e-13)
    s_wrong = (ea["node_types"] + 1.0) * ea["num_neigh"]
    assert not np.allclose(s, s_wrong)
    # the other rows carry Y_lm of the same edges: row lm of channel 0 is sum_j (t_j+1) Y_lm(ij)
    Y = orc.Y.reshape(-1, 16)
    for lm in (1, 2, 3, 6, 12):
        want = np.bincount(recv, weights=(ea["neigh_types"] + 1.0) * Y[:, lm], minlength=N)
        assert np.allclose(A0[:, lm, 0], want, rtol=1e-12, atol=1e-13)


def test_A0_weights_are_row_major_kp_k_of_the_receiver_species(base):
    """A0_weights[t][l] = elementary matrix with a one at row kp0, column k0 (flat kp0*K+k0), a
    different (kp0, k0) for every (t, l).  Row-major NoTrans x NoTrans (mace.cpp:184-198) gives
    A0[i, lm, k0] = Phi0[i, lm, kp0] for receivers of species t and lm in block l, zero in every
    other column.  Fails if the matrix is read as [k][kp], or taken from the sender's species."""
    model = copy.deepcopy(base)
    pick = {(t, l): ((t + l) % K, (t + 2 * l + 1) % K) for t in range(3) for l in range(4)}
    assert all(a != b for a, b in pick.values())
    ident = copy.deepcopy(model)
    ident["A0_weights"] = [[np.eye(K).ravel().tolist() for _ in range(4)] for _ in range(3)]
    model["A0_weights"] = [[_elementary(K, K, *pick[(t, l)]) for l in range(4)] for t in range(3)]
    nl, ea = _system(model)
    N = ea["num_nodes"]
    geo = (N, ea["node_types"], ea["num_neigh"], ea["neigh_types"])
    out = []
    for m in (ident, model):
        orc = OracleMACE(m)
        orc.compute_Y(ea["xyz"]); orc.compute_R0(*geo, ea["r"]); orc.compute_A0(*geo)
        out.append(orc.A0.reshape(N, 16, K))
    Phi0, A0 = out
    assert np.abs(Phi0).min() > 0
    for i in range(N):
        for l in range(4):
            kp0, k0 = pick[(int(ea["node_types"][i]), l)]
            blk = slice(l * l, (l + 1) ** 2)
            want = np.zeros((2 * l + 1, K)); want[:, k0] = Phi0[i, blk, kp0]
            assert np.array_equal(A0[i, blk], want)
            swapped = np.zeros((2 * l + 1, K)); swapped[:, kp0] = Phi0[i, blk, k0]
            assert not np.allclose(A0[i, blk], swapped)


# ------------------------------------------------------------------------------------------------
# symmetric contraction (mace.cpp:348-370, 759-777; loader 959-972, 1004-1015)
def test_M0_polynomial_of_species_LM_channel(base):
    """All M0 weights zero except species a*, output LM*, channel k*, where only monomial number
    n* has coefficient 1: M0[i, LM*, k*] = product of that monomial's A0[i, v, k*] on nodes of
    species a* and M0 is zero everywhere else; M0_grad[i, LM*, v, k*] is the product of the
    other factors (layout [LM][lm][k], mace.cpp:365).  Fails if the polynomial list is indexed
    [LM][a][k], [a][k][LM], by a neighbour's species, or if M0_grad is laid out [lm][LM][k]."""
    model = copy.deepcopy(base)
    nLM = (model["L_max"] + 1) ** 2
    a_s, LM_s, k_s = 1, nLM - 1, 3
    monos = model["M0_monomials"][LM_s]
    n_s = max(range(len(monos)), key=lambda n: (len(set(monos[n])), len(monos[n])))  # a mixed monomial
    for a in range(3):
        for LM in range(nLM):
            for k in range(K):
                w = [0.0] * len(model["M0_monomials"][LM])
                if (a, LM, k) == (a_s, LM_s, k_s):
                    w[n_s] = 1.0
                model["M0_weights"][a][LM][k] = w
    orc = OracleMACE(model)
    nl, ea = _system(model)
    N, nt = ea["num_nodes"], ea["node_types"]
    rng = np.random.default_rng(2)
    A0 = rng.normal(size=(N, 16, K))
    orc.A0 = A0; orc.compute_M0(N, nt)
    M0 = orc.M0.reshape(N, nLM, K); G = orc.M0_grad.reshape(N, nLM, 16, K)
    mono = monos[n_s]
    want = np.zeros((N, nLM, K)); wantG = np.zeros((N, nLM, 16, K))
    for i in range(N):
        if nt[i] != a_s:
            continue
        want[i, LM_s, k_s] = np.prod([A0[i, v, k_s] for v in mono])
        for pos, v in enumerate(mono):
            wantG[i, LM_s, v, k_s] += np.prod([A0[i, u, k_s] for q, u in enumerate(mono) if q != pos])
    assert (nt == a_s).any() and np.abs(want).max() > 0
    assert np.allclose(M0, want, rtol=1e-13, atol=0)
    assert np.allclose(G, wantG, rtol=1e-13, atol=0)


def test_M1_polynomial_of_species_channel(base):
    """Same for layer 1: P1[type_i*K + k] (mace.cpp:772), M1_grad laid out [lm][k] (mace.cpp:774)."""
    model = copy.deepcopy(base)
    a_s, k_s = 2, 1
    monos = model["M1_monomials"]
    n_s = max(range(len(monos)), key=lambda n: (len(set(monos[n])), len(monos[n])))
    for a in range(3):
        for k in range(K):
            w = [0.0] * len(monos)
            if (a, k) == (a_s, k_s):
                w[n_s] = 1.0
            model["M1_weights"][a][k] = w
    orc = OracleMACE(model)
    nl, ea = _system(model)
    N, nt = ea["num_nodes"], ea["node_types"]
    A1 = np.random.default_rng(3).normal(size=(N, 16, K))
    orc.A1 = A1; orc.compute_M1(N, nt)
    M1 = orc.M1.reshape(N, K); G = orc.M1_grad[: N * 16 * K].reshape(N, 16, K)
    mono = monos[n_s]
    want = np.zeros((N, K)); wantG = np.zeros((N, 16, K))
    for i in np.nonzero(nt == a_s)[0]:
        want[i, k_s] = np.prod([A1[i, v, k_s] for v in mono])
        for pos, v in enumerate(mono):
            wantG[i, v, k_s] += np.prod([A1[i, u, k_s] for q, u in enumerate(mono) if q != pos])
    assert np.abs(want).max() > 0
    assert np.allclose(M1, want, rtol=1e-13, atol=0)
    assert np.allclose(G, wantG, rtol=1e-13, atol=0)


# ------------------------------------------------------------------------------------------------
# H1 (mace.cpp:397-423)
def test_H1_weights_are_row_major_kp_k_per_l(base):
    """H1_weights block l = elementary (kp0_l, k0_l): H1[i, lm, k0_l] = M0[i, lm, kp0_l] for lm in
    block l, other columns zero.  Fails under a transposed read or a wrong block offset."""
    model = copy.deepcopy(base)
    L_max = model["L_max"]; nLM = (L_max + 1) ** 2
    pick = {l: ((2 * l + 1) % K, (2 * l + 2) % K) for l in range(L_max + 1)}
    assert all(a != b for a, b in pick.values())
    model["H1_weights"] = sum((_elementary(K, K, *pick[l]) for l in range(L_max + 1)), [])
    orc = OracleMACE(model)
    N = 4
    M0 = np.random.default_rng(4).normal(size=(N, nLM, K))
    orc.M0 = M0; orc.compute_H1(N)
    H1 = orc.H1.reshape(N, nLM, K)
    for l in range(L_max + 1):
        kp0, k0 = pick[l]
        blk = slice(l * l, (l + 1) ** 2)
        want = np.zeros((N, 2 * l + 1, K)); want[:, :, k0] = M0[:, blk, kp0]
        assert np.array_equal(H1[:, blk], want)


# ------------------------------------------------------------------------------------------------
# layer 1 aggregation (mace.cpp:453-502)
def test_Phi1_gathers_the_sender_row_and_enumerates_path_lm1_lm2(base):
    """Phi1r and Phi1 rebuilt in numpy from the oracle's R1, Y and a random H1 with the reference's
    running index (path outermost, then lm1 of Y, then lm2 of H1; mace.cpp:468-483) and the
    coupling triples of the file (mace.cpp:494-500).  H1 has more rows than receivers (ghost
    rows), and one extra receiver-less row is referenced by an edge, so a gather by receiver
    index cannot match.  Negative control: gathering H1[i] instead of H1[j] differs."""
    model = base
    orc = OracleMACE(model)
    nl, ea = _system(model)
    N = ea["num_nodes"]; nLM = (model["L_max"] + 1) ** 2
    P = len(model["Phi1_l"])
    geo = (N, ea["node_types"], ea["num_neigh"], ea["neigh_types"])
    orc.compute_Y(ea["xyz"]); orc.compute_R1(*geo, ea["r"])
    rng = np.random.default_rng(6)
    H1 = rng.normal(size=(N + 2, nLM, K))
    ni = ea["neigh_indices"].copy(); ni[0] = N + 1            # a ghost row as sender
    orc.H1 = H1; orc.compute_Phi1(N, ea["num_neigh"], ni)
    Y = orc.Y.reshape(-1, 16); R1 = orc.R1.reshape(-1, P, K)
    recv = _receiver_of_edge(ea)
    l1s, l2s = model["Phi1_l1"], model["Phi1_l2"]
    n_r = sum((2 * a + 1) * (2 * b + 1) for a, b in zip(l1s, l2s))
    n_e = sum(2 * l + 1 for l in model["Phi1_l"])

    def rebuild(sender_rows):
        Phi1r = np.zeros((N, n_r, K))
        for e in range(len(recv)):
            q = 0
            for p in range(P):
                for lm1 in range(l1s[p] ** 2, (l1s[p] + 1) ** 2):
                    for lm2 in range(l2s[p] ** 2, (l2s[p] + 1) ** 2):
                        Phi1r[recv[e], q] += R1[e, p] * Y[e, lm1] * H1[sender_rows[e], lm2]
                        q += 1
        Phi1 = np.zeros((N, n_e, K))
        for lme, c, q in zip(model["Phi1_lme"], model["Phi1_clebsch_gordan"], model["Phi1_lelm1lm2"]):
            Phi1[:, lme] += c * Phi1r[:, q]
        return Phi1r, Phi1
    Phi1r, Phi1 = rebuild(ni)
    assert np.allclose(orc.Phi1r.reshape(N, n_r, K), Phi1r, rtol=1e-12, atol=1e-14)
    assert np.allclose(orc.Phi1.reshape(N, n_e, K), Phi1, rtol=1e-12, atol=1e-14)
    assert not np.allclose(orc.Phi1.reshape(N, n_e, K), rebuild(recv)[1], rtol=1e-3)


def test_Phi1_of_a_single_unit_sender_feature(base):
    """H1 zero except one (row j*, component lm2*, channel k*) = 1.  Before the coupling sum,
    Phi1r[i, q, k*] = sum over edges i<-j* of R1[path(q), k*] Y[lm1(q)] for the q whose lm2 is
    lm2*, and zero elsewhere.  Fails if lm1 and lm2 swap roles in the running index."""
    model = base
    if model["L_max"] == 0:
        pytest.skip("needs a sender feature with more than one component")
    orc = OracleMACE(model)
    nl, ea = _system(model)
    N = ea["num_nodes"]; P = len(model["Phi1_l"])
    geo = (N, ea["node_types"], ea["num_neigh"], ea["neigh_types"])
    orc.compute_Y(ea["xyz"]); orc.compute_R1(*geo, ea["r"])
    j_s, lm2_s, k_s = int(ea["neigh_indices"][3]), 2, 1
    H1 = np.zeros((N, (model["L_max"] + 1) ** 2, K)); H1[j_s, lm2_s, k_s] = 1.0
    orc.H1 = H1; orc.compute_Phi1(N, ea["num_neigh"], ea["neigh_indices"])
    Y = orc.Y.reshape(-1, 16); R1 = orc.R1.reshape(-1, P, K)
    recv = _receiver_of_edge(ea)
    got = orc.Phi1r.reshape(N, -1, K)
    want = np.zeros_like(got)
    q = 0
    for p in range(P):
        l1, l2 = model["Phi1_l1"][p], model["Phi1_l2"][p]
        for m1 in range(2 * l1 + 1):
            for m2 in range(2 * l2 + 1):
                if l2 * l2 + m2 == lm2_s:
                    for e in np.nonzero(ea["neigh_indices"] == j_s)[0]:
                        want[recv[e], q, k_s] += R1[e, p, k_s] * Y[e, l1 * l1 + m1]
                q += 1
    assert np.abs(want).max() > 0
    assert np.allclose(got, want, rtol=1e-12, atol=1e-15)


# ------------------------------------------------------------------------------------------------
# A1 (mace.cpp:607-642)
def test_A1_weights_rows_are_e_major_kp_minor(base):
    """A1_weights[l] = elementary with a one at row e0*K+kp0, column k0.  The product takes
    Phi1[i] block l as a (2l+1) x (num_e K) row-major matrix (lda = num_e K, mace.cpp:629-632), so
    A1[i, l*l+m, k0] = Phi1[i, off_l + m*num_e*K + e0*K + kp0].  Fails if Phi1 is read as
    [l][e][m][k], the weight rows as kp*num_e+e, or the matrix transposed."""
    model = copy.deepcopy(base)
    Pl = model["Phi1_l"]
    num_e = [Pl.count(l) for l in range(4)]
    pick = {l: (num_e[l] - 1, (l + 1) % K, (2 * l + 3) % K) for l in range(4)}
    model["A1_weights"] = [_elementary(num_e[l] * K, K, pick[l][0] * K + pick[l][1], pick[l][2]) for l in range(4)]
    orc = OracleMACE(model)
    N = 3
    n_e = sum((2 * l + 1) * num_e[l] for l in range(4))
    Phi1 = np.random.default_rng(7).normal(size=(N, n_e * K))
    orc.Phi1 = Phi1; orc.compute_A1(N)
    A1 = orc.A1.reshape(N, 16, K)
    off = 0
    for l in range(4):
        e0, kp0, k0 = pick[l]
        for m in range(2 * l + 1):
            want = np.zeros((N, K))
            want[:, k0] = Phi1[:, off + m * num_e[l] * K + e0 * K + kp0]
            assert np.array_equal(A1[:, l * l + m], want)
        off += (2 * l + 1) * num_e[l] * K


# ------------------------------------------------------------------------------------------------
# H2 and readouts (mace.cpp:796-832, 876-903; multilayer_perceptron.cpp:88-147)
def test_H2_weights_are_consumed_transposed_and_by_receiver_species(base):
    """dgemv RowMajor Trans (mace.cpp:804-830): H2[i,k] = sum_kp W[kp*K+k] x[kp].  With
    H2_weights_for_H1[t] = elementary (kp_t, k_t) and H2_weights_for_M1 = elementary (kp_m, k_m):
    H2[i, k_t] = H1[i, 0, kp_t] (species t of node i), H2[i, k_m] = M1[i, kp_m], zero elsewhere.
    Fails if either matrix is read [k][kp], or the l = 0 block of H1 is not the first K entries."""
    model = copy.deepcopy(base)
    nLM = (model["L_max"] + 1) ** 2
    pick = {0: (0, 2), 1: (1, 3), 2: (4, 0)}
    kp_m, k_m = 2, 4
    model["H2_weights_for_H1"] = [_elementary(K, K, *pick[t]) for t in range(3)]
    model["H2_weights_for_M1"] = _elementary(K, K, kp_m, k_m)
    orc = OracleMACE(model)
    nt = np.array([0, 1, 2, 1, 0], dtype=np.int32); N = len(nt)
    rng = np.random.default_rng(8)
    H1 = rng.normal(size=(N, nLM, K)); M1 = rng.normal(size=(N, K))
    orc.H1 = H1; orc.M1 = M1; orc.compute_H2(N, nt)
    H2 = orc.H2.reshape(N, K)
    want = np.zeros((N, K))
    for i in range(N):
        kp, k = pick[int(nt[i])]
        want[i, k] += H1[i, 0, kp]
        want[i, k_m] += M1[i, kp_m]
    assert np.array_equal(H2, want)


def test_readout_weight_layouts(base):
    """readout_2_weights_1 is [16][K] row-major (dgemv NoTrans, m = 16, n = K, lda = K): a single
    one at flat index j0*K + k0 makes hidden unit j0 equal H2[i, k0] and leaves the others at 0, so
    E_i = E0[t_i] + w1 . H1[i, 0, :] + w2[j0] c x s(x), x = H2[i, k0], and
    H2_adj[i, k] = w2[j0] c (s + x s (1 - s)) at k = k0 only; H1_adj = w1 in the l = 0 block, zero
    in the others (mace.cpp:885-893).  K = 5 != 16, so a [K][16] read lands on another unit and
    channel.  Fails also if the first readout takes another block of H1."""
    model = copy.deepcopy(base)
    nLM = (model["L_max"] + 1) ** 2
    j0, k0 = 9, 3
    w1 = np.zeros(16 * K); w1[j0 * K + k0] = 1.0
    model["readout_2_weights_1"] = w1.tolist()
    orc = OracleMACE(model)
    nt = np.array([2, 0, 1, 1], dtype=np.int32); N = len(nt)
    rng = np.random.default_rng(9)
    H1 = rng.normal(size=(N, nLM, K)); H2 = rng.normal(size=(N, K))
    orc.H1 = H1; orc.H2 = H2; orc.node_energies = np.zeros(N)
    orc.compute_readouts(N, nt)
    c = model["readout_2_scale_factor"]; w2 = np.asarray(model["readout_2_weights_2"])
    x = H2[:, k0]; s = 1.0 / (1.0 + np.exp(-x))
    ro1 = np.asarray(model["readout_1_weights"])
    E = np.asarray(model["atomic_energies"])[nt] + H1[:, 0, :] @ ro1 + w2[j0] * c * x * s
    assert np.allclose(orc.node_energies, E, rtol=1e-13, atol=1e-15)
    g = np.zeros((N, K)); g[:, k0] = w2[j0] * c * (s + x * s * (1 - s))
    assert np.allclose(orc.H2_adj.reshape(N, K), g, rtol=1e-13, atol=0)
    seed = np.zeros((N, nLM, K)); seed[:, 0, :] = ro1
    assert np.array_equal(orc.H1_adj.reshape(N, nLM, K), seed)


# ------------------------------------------------------------------------------------------------
# the whole forward path once more, as one chain of numpy contractions
def test_forward_chain_in_numpy(base):
    """Every forward stage from (Y, R0, R1) to the node energies rebuilt with numpy contractions
    written from the reference's loops, on a model with random, asymmetric, species-dependent
    weights and distinct pair tables; polynomials by brute-force monomial sums.  A consistent
    transposition anywhere in the oracle changes these numbers by O(1)."""
    model = base
    orc = OracleMACE(model)
    nl, ea = _system(model, n=8, seed=21)
    orc.compute_node_energies_forces(*H.call_args(ea))
    N = ea["num_nodes"]; nt = ea["node_types"]; nty = ea["neigh_types"]; ni = ea["neigh_indices"]
    L_max = model["L_max"]; nLM = (L_max + 1) ** 2; P = len(model["Phi1_l"])
    recv = _receiver_of_edge(ea)
    Y = orc.Y.reshape(-1, 16); R0 = orc.R0.reshape(-1, 4, K); R1 = orc.R1.reshape(-1, P, K)
    l_of = np.array([l for l in range(4) for _ in range(2 * l + 1)])
    H0 = np.asarray(model["H0_weights"]).reshape(3, K)
    W0 = np.asarray(model["A0_weights"]).reshape(3, 4, K, K)                 # [t][l][kp][k]
    Phi0 = np.zeros((N, 16, K))
    np.add.at(Phi0, recv, R0[:, l_of, :] * Y[:, :, None] * H0[nty][:, None, :])
    A0 = np.einsum("imp,impk->imk", Phi0, W0[nt][:, l_of])
    assert np.allclose(orc.A0.reshape(N, 16, K), A0, rtol=1e-11, atol=1e-14)

    def poly(monos, w, x):                                                   # x: [16]
        return sum(c * np.prod([x[v] for v in mono]) for c, mono in zip(w, monos))
    M0 = np.zeros((N, nLM, K))
    for i in range(N):
        for LM in range(nLM):
            for k in range(K):
                M0[i, LM, k] = poly(model["M0_monomials"][LM], model["M0_weights"][int(nt[i])][LM][k], A0[i, :, k])
    assert np.allclose(orc.M0.reshape(N, nLM, K), M0, rtol=1e-10, atol=1e-13)
    LM_l = np.array([l for l in range(L_max + 1) for _ in range(2 * l + 1)])
    WH1 = np.asarray(model["H1_weights"]).reshape(L_max + 1, K, K)
    H1 = np.einsum("imp,mpk->imk", M0, WH1[LM_l])
    assert np.allclose(orc.H1.reshape(N, nLM, K), H1, rtol=1e-10, atol=1e-13)
    # layer 1
    l1s, l2s, ls = model["Phi1_l1"], model["Phi1_l2"], model["Phi1_l"]
    rows = []
    for p in range(P):
        for lm1 in range(l1s[p] ** 2, (l1s[p] + 1) ** 2):
            for lm2 in range(l2s[p] ** 2, (l2s[p] + 1) ** 2):
                rows.append((p, lm1, lm2))
    rp, r1, r2 = (np.array(c) for c in zip(*rows))
    Phi1r = np.zeros((N, len(rows), K))
    np.add.at(Phi1r, recv, R1[:, rp, :] * Y[:, r1, None] * H1[ni][:, r2, :])
    n_e = sum(2 * l + 1 for l in ls)
    Phi1 = np.zeros((N, n_e, K))
    for lme, c, q in zip(model["Phi1_lme"], model["Phi1_clebsch_gordan"], model["Phi1_lelm1lm2"]):
        Phi1[:, lme] += c * Phi1r[:, q]
    assert np.allclose(orc.Phi1.reshape(N, n_e, K), Phi1, rtol=1e-10, atol=1e-13)
    num_e = [ls.count(l) for l in range(4)]
    A1 = np.zeros((N, 16, K)); off = 0
    for l in range(4):
        W = np.asarray(model["A1_weights"][l]).reshape(num_e[l] * K, K)
        blk = Phi1[:, off:off + (2 * l + 1) * num_e[l]].reshape(N, 2 * l + 1, num_e[l] * K)
        A1[:, l * l:(l + 1) ** 2] = blk @ W
        off += (2 * l + 1) * num_e[l]
    assert np.allclose(orc.A1.reshape(N, 16, K), A1, rtol=1e-10, atol=1e-13)
    M1 = np.array([[poly(model["M1_monomials"], model["M1_weights"][int(nt[i])][k], A1[i, :, k]) for k in range(K)]
                   for i in range(N)])
    assert np.allclose(orc.M1.reshape(N, K), M1, rtol=1e-9, atol=1e-13)
    WH = np.asarray(model["H2_weights_for_H1"]).reshape(3, K, K); WM = np.asarray(model["H2_weights_for_M1"]).reshape(K, K)
    H2 = np.einsum("ip,ipk->ik", H1[:, 0], WH[nt]) + M1 @ WM
    assert np.allclose(orc.H2.reshape(N, K), H2, rtol=1e-9, atol=1e-13)
    c = model["readout_2_scale_factor"]
    hid = H2 @ np.asarray(model["readout_2_weights_1"]).reshape(16, K).T
    act = c * hid / (1.0 + np.exp(-hid))
    E = (np.asarray(model["atomic_energies"])[nt] + H1[:, 0] @ np.asarray(model["readout_1_weights"])
         + act @ np.asarray(model["readout_2_weights_2"]))
    assert np.allclose(orc.node_energies, E, rtol=1e-9, atol=1e-12)
