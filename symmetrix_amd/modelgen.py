"""Random-init generator for symmetrix JSON model files.

Counterpart of the reference's checkpoint extractor
(symmetrix/source/symmetrix/extract_mace_data.py:19-519): it emits every key
`MACE::load_from_json` reads (libsymmetrix/source/mace.cpp:905-1030) with the
same shapes, index orders and rough magnitudes, but from seeded Gaussian
weights instead of a trained torch model (no checkpoint can be fetched here).

Both the CPU oracle and the GPU engine consume the same file, so the
generator's normalisation choices do not enter any parity statement; what it
must get right is the *structure*: spline grids, path lists, Clebsch-Gordan
index conventions and an equivariant symmetric-contraction polynomial, so
that the energy is rotation invariant and the work per atom is realistic.
"""
from __future__ import annotations

import json
from math import pi, sqrt

import numpy as np
from scipy.interpolate import CubicSpline

from . import cg

ATOMIC_NUMBERS = {"H": 1, "C": 6, "N": 7, "O": 8}


def _bessel_cutoff(r, r_cut, n_bessel, p):
    """sqrt(2/rc) sin(n pi r/rc)/r times the polynomial envelope of order p."""
    n = np.arange(1, n_bessel + 1, dtype=np.float64)
    bes = sqrt(2.0 / r_cut) * np.sin(np.outer(r, n) * pi / r_cut) / r[:, None]
    x = r / r_cut
    env = (1.0 - (p + 1.0) * (p + 2.0) / 2.0 * x**p
           + p * (p + 2.0) * x**(p + 1) - p * (p + 1.0) / 2.0 * x**(p + 2))
    env = np.where(x < 1.0, env, 0.0)
    return bes * env[:, None]


def _silu(x):
    return 1.679177 * x / (1.0 + np.exp(-x))


def _radial_tables(rng, r, n_bessel, mlp, n_out, r_cut, p):
    """Tabulated radial MLP output and its spline derivatives at the knots.

    Same recipe as extract_mace_data.py:145-172: MLP(bessel*cutoff) sampled on
    linspace(1e-12, r_cut, n) and splined column by column with scipy's
    not-a-knot / clamped cubic spline; stored as knot values + derivatives.
    """
    feats = _bessel_cutoff(r, r_cut, n_bessel, p)
    widths = [n_bessel] + list(mlp) + [n_out]
    h = feats
    for li in range(len(widths) - 1):
        W = rng.normal(size=(widths[li], widths[li + 1])) / sqrt(widths[li])
        h = h @ W
        if li < len(widths) - 2:
            h = _silu(h)
    spl = CubicSpline(r, h, axis=0, bc_type=("not-a-knot", "clamped"))
    vals = spl(r)
    ders = spl.derivative()(r)
    return vals.T.copy(), ders.T.copy()  # [n_out][n_pts]


def _density_splines(rng, r, h, T, n_bessel, r_cut, p, name):
    """tanh(density_fn(bessels)^2) per unordered pair, splined like the radial tables (extract_mace_data.py:204-226)."""
    feats = _bessel_cutoff(r, r_cut, n_bessel, p)
    vals, ders = [], []
    for a in range(T):
        for b in range(a, T):
            w = rng.normal(size=n_bessel) / sqrt(n_bessel)
            spl = CubicSpline(r, np.tanh((feats @ w) ** 2), bc_type=("not-a-knot", "clamped"))
            vals.append(spl(r).tolist())
            ders.append(spl.derivative()(r).tolist())
    return {f"{name}_spline_h": float(h), f"{name}_spline_values": vals, f"{name}_spline_derivs": ders}


def generate_model(
    atomic_numbers,
    num_channels,
    L_max,
    r_cut,
    n_bessel=8,
    cutoff_p=5,
    mlp=(64, 64, 64),
    correlation=3,
    num_spline_points=256,
    avg_num_neighbors=30.0,
    seed=0,
    pair_dependent_radial=True,
    zbl=False,
    density_normalisation=False,
):
    """Return the model as a dict ready for json.dump.

    zbl adds the pair-repulsion keys (extract_mace_data.py:130-138); density_normalisation makes both
    interaction layers "density" layers: one normalisation spline per unordered species pair
    (extract_mace_data.py:201-226, 386-411).
    """
    rng = np.random.default_rng(seed)
    Z = sorted(int(z) for z in atomic_numbers)
    T = len(Z)
    K = int(num_channels)
    l_max = 3
    n_lm = (l_max + 1) ** 2
    n_LM = (L_max + 1) ** 2

    out = {
        "num_elements": T,
        "num_channels": K,
        "r_cut": float(r_cut),
        "l_max": l_max,
        "L_max": int(L_max),
        "atomic_numbers": Z,
        "atomic_energies": rng.normal(size=T).tolist(),
        "has_zbl": bool(zbl),
    }
    if zbl:
        # constants of mace's ZBLBasis; covalent radii indexed by atomic number (synthetic beyond H, C, N, O)
        radii = [0.2] + [0.5 + 0.004 * z for z in range(1, max(Z) + 1)]
        for z, rad in ((1, 0.31), (6, 0.76), (7, 0.71), (8, 0.66)):
            if z < len(radii):
                radii[z] = rad
        out["zbl_a_exp"] = 0.3
        out["zbl_a_prefactor"] = 0.4543
        out["zbl_c"] = [0.1818 * 0.8, 0.5099 * 0.8, 0.2802 * 0.8, 0.02817 * 0.8]
        out["zbl_covalent_radii"] = radii
        out["zbl_p"] = 6

    # ----- radial splines: one table per unordered pair (a<=b), row-major upper triangle
    r, h = np.linspace(1e-12, r_cut, num_spline_points, retstep=True)
    paths = cg.tensor_product_paths(l_max, L_max)
    P = len(paths)
    v0, d0, v1, d1 = [], [], [], []
    shared = None
    for a in range(T):
        for b in range(a, T):
            if pair_dependent_radial or shared is None:
                t0 = _radial_tables(rng, r, n_bessel, mlp, (l_max + 1) * K, r_cut, cutoff_p)
                t1 = _radial_tables(rng, r, n_bessel, mlp, P * K, r_cut, cutoff_p)
                shared = (t0, t1)
            (a0, b0), (a1, b1) = shared
            v0.append(a0.tolist()); d0.append(b0.tolist())
            v1.append(a1.tolist()); d1.append(b1.tolist())
    out["radial_spline_h"] = float(h)
    out["radial_spline_values_0"] = v0
    out["radial_spline_derivs_0"] = d0
    out["radial_spline_values_1"] = v1
    out["radial_spline_derivs_1"] = d1

    # ----- layer 0
    out["H0_weights"] = rng.normal(size=T * K).tolist()
    out["A0_scaled"] = bool(density_normalisation)
    if density_normalisation:
        out.update(_density_splines(rng, r, h, T, n_bessel, r_cut, cutoff_p, "A0"))
    # (the extractor drops the 1/avg_num_neighbors factor for density layers; a random model keeps a comparable
    # magnitude by dividing by the typical divisor instead)
    norm0 = avg_num_neighbors / 3.0 if density_normalisation else avg_num_neighbors
    out["A0_weights"] = [
        [(rng.normal(size=(K, K)) / (sqrt(K) * norm0) * 4.0).ravel().tolist()
         for _ in range(l_max + 1)]
        for _ in range(T)
    ]

    # ----- symmetric contraction, layer 0: outputs LM = 0..n_LM-1
    def contraction(L, scale):
        terms = cg.symmetric_contraction_terms(L, l_max, correlation)
        per_M = []
        for M in range(2 * L + 1):
            keys = []
            for t in terms:
                for k_ in t[M]:
                    if k_ not in keys:
                        keys.append(k_)
            U = np.zeros((len(terms), len(keys)))
            for e, t in enumerate(terms):
                for k_, v in t[M].items():
                    U[e, keys.index(k_)] = v
            per_M.append((keys, U))
        # weights W[a, eta, k], shared by all M of this L (equivariance)
        W = rng.normal(size=(T, len(terms), K)) * scale
        return per_M, W

    M0_w = {a: {} for a in range(T)}
    M0_m = {}
    for L in range(L_max + 1):
        per_M, W = contraction(L, 0.3)
        for M in range(2 * L + 1):
            keys, U = per_M[M]
            LM = L * L + M
            M0_m[LM] = [list(k_) for k_ in keys]
            for a in range(T):
                coef = np.einsum("ek,em->km", W[a], U)  # [K][n_mono]
                M0_w[a][LM] = {k: coef[k].tolist() for k in range(K)}
    out["M0_weights"] = M0_w
    out["M0_monomials"] = M0_m

    out["H1_weights"] = (rng.normal(size=(L_max + 1, K, K)) / sqrt(K)).ravel().tolist()

    # ----- layer 1 tensor product
    Phi1_l = [p_[0] for p_ in paths]
    Phi1_l1 = [p_[1] for p_ in paths]
    Phi1_l2 = [p_[2] for p_ in paths]
    num_e = [Phi1_l.count(l) for l in range(l_max + 1)]
    lme_off = np.concatenate([[0], np.cumsum([(2 * l + 1) * num_e[l] for l in range(l_max + 1)])])
    q_off = np.concatenate([[0], np.cumsum([(2 * a + 1) * (2 * b + 1) for (_, a, b) in paths])])
    cg_lme, cg_val, cg_q = [], [], []
    # same enumeration order as extract_mace_data.py:351-375: lm1 outer, lm2, then path, then m
    for l1 in range(l_max + 1):
        for m1 in range(-l1, l1 + 1):
            for l2 in range(L_max + 1):
                for m2 in range(-l2, l2 + 1):
                    for le, (l, pl1, pl2) in enumerate(paths):
                        if pl1 != l1 or pl2 != l2:
                            continue
                        C = cg.real_cg(l1, l2, l) * sqrt(2 * l + 1)
                        e = le - sum(1 for x in Phi1_l if x < l)
                        for m in range(-l, l + 1):
                            c = C[l1 + m1, l2 + m2, l + m]
                            if abs(c) > 1e-12:
                                cg_lme.append(int(lme_off[l] + (l + m) * num_e[l] + e))
                                cg_val.append(float(c))
                                cg_q.append(int(q_off[le] + (l1 + m1) * (2 * l2 + 1) + (l2 + m2)))
    out["Phi1_l"] = Phi1_l
    out["Phi1_l1"] = Phi1_l1
    out["Phi1_l2"] = Phi1_l2
    out["Phi1_lme"] = cg_lme
    out["Phi1_clebsch_gordan"] = cg_val
    out["Phi1_lelm1lm2"] = cg_q

    out["A1_scaled"] = bool(density_normalisation)
    if density_normalisation:
        out.update(_density_splines(rng, r, h, T, n_bessel, r_cut, cutoff_p, "A1"))
    norm1 = avg_num_neighbors / 3.0 if density_normalisation else avg_num_neighbors
    out["A1_weights"] = [
        (rng.normal(size=(num_e[l], K, K)) / (sqrt(num_e[l] * K) * norm1) * 4.0).ravel().tolist()
        for l in range(l_max + 1)
    ]

    per_M, W = contraction(0, 0.3)
    keys, U = per_M[0]
    out["M1_monomials"] = [list(k_) for k_ in keys]
    out["M1_weights"] = {
        a: {k: (W[a, :, k] @ U).tolist() for k in range(K)} for a in range(T)
    }

    out["H2_weights_for_H1"] = [(rng.normal(size=(K, K)) / sqrt(K)).ravel().tolist() for _ in range(T)]
    out["H2_weights_for_M1"] = (rng.normal(size=(K, K)) / sqrt(K)).ravel().tolist()
    out["readout_1_weights"] = (rng.normal(size=K) / sqrt(K)).tolist()
    out["readout_2_weights_1"] = (rng.normal(size=(16, K)) / sqrt(K)).ravel().tolist()
    out["readout_2_weights_2"] = (rng.normal(size=16) / 4.0).tolist()
    out["readout_2_scale_factor"] = 1.679177
    return out


def write_model(path, **kwargs):
    model = generate_model(**kwargs)
    with open(path, "w") as f:
        json.dump(model, f)
    return model


# The synthetic model configurations named by the benchmark description.
CONFIGS = {
    "tiny": dict(atomic_numbers=[1, 6, 8], num_channels=32, L_max=0, r_cut=5.0, n_bessel=8),
    "off_small": dict(atomic_numbers=[1, 6, 7, 8], num_channels=96, L_max=0, r_cut=4.5, n_bessel=8),
    "off_medium": dict(atomic_numbers=[1, 6, 7, 8], num_channels=128, L_max=1, r_cut=5.0, n_bessel=8),
    # hidden features up to l = 2 (128x0e+128x1o+128x2e), otherwise the model above
    "off_medium_l2": dict(atomic_numbers=[1, 6, 7, 8], num_channels=128, L_max=2, r_cut=5.0, n_bessel=8),
    "mp_medium": dict(atomic_numbers=[13, 22, 26, 28, 29], num_channels=128, L_max=1, r_cut=6.0,
                      n_bessel=10, avg_num_neighbors=80.0),
}
