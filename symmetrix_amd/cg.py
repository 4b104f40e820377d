"""Real spherical harmonics and real Clebsch-Gordan coefficients (numpy).

Used by the random-init model generator (`modelgen.py`), which plays the role
the reference's extractor plays for real checkpoints
(symmetrix/source/symmetrix/extract_mace_data.py:323-381 for the layer-1
tensor-product paths, :242-304 and :425-474 for the symmetric-contraction
monomials).  Nothing here runs at inference time.

Convention.  `real_sph_harm` returns the 16 harmonics l<=3 in the basis the
engine uses (libsymmetrix/source/mace.cpp:118-148): standard orthonormal real
harmonics (m<0 ~ sin|m|phi, m>0 ~ cos m phi, no Condon-Shortley sign in the
real form) evaluated at the cyclically permuted vector (z, x, y) and scaled by
2*sqrt(pi) ("component" normalisation, sum_m Y_lm^2 = 2l+1).  The cyclic
permutation is a proper rotation, so Clebsch-Gordan coefficients of the
standard real basis couple these functions unchanged.
"""
from __future__ import annotations

from fractions import Fraction
from functools import lru_cache
from math import factorial, sqrt, pi

import numpy as np


def real_sph_harm_std(u: np.ndarray) -> np.ndarray:
    """Orthonormal real harmonics l<=3 of unit vectors u[...,3] -> [...,16]."""
    x, y, z = u[..., 0], u[..., 1], u[..., 2]
    Y = np.empty(u.shape[:-1] + (16,), dtype=np.float64)
    Y[..., 0] = 0.5 * sqrt(1.0 / pi)
    c1 = sqrt(3.0 / (4.0 * pi))
    Y[..., 1] = c1 * y
    Y[..., 2] = c1 * z
    Y[..., 3] = c1 * x
    Y[..., 4] = 0.5 * sqrt(15.0 / pi) * x * y
    Y[..., 5] = 0.5 * sqrt(15.0 / pi) * y * z
    Y[..., 6] = 0.25 * sqrt(5.0 / pi) * (2.0 * z * z - x * x - y * y)
    Y[..., 7] = 0.5 * sqrt(15.0 / pi) * x * z
    Y[..., 8] = 0.25 * sqrt(15.0 / pi) * (x * x - y * y)
    Y[..., 9] = 0.25 * sqrt(35.0 / (2.0 * pi)) * y * (3.0 * x * x - y * y)
    Y[..., 10] = 0.5 * sqrt(105.0 / pi) * x * y * z
    Y[..., 11] = 0.25 * sqrt(21.0 / (2.0 * pi)) * y * (4.0 * z * z - x * x - y * y)
    Y[..., 12] = 0.25 * sqrt(7.0 / pi) * z * (2.0 * z * z - 3.0 * x * x - 3.0 * y * y)
    Y[..., 13] = 0.25 * sqrt(21.0 / (2.0 * pi)) * x * (4.0 * z * z - x * x - y * y)
    Y[..., 14] = 0.25 * sqrt(105.0 / pi) * (x * x - y * y) * z
    Y[..., 15] = 0.25 * sqrt(35.0 / (2.0 * pi)) * x * (x * x - 3.0 * y * y)
    return Y


def real_sph_harm(xyz: np.ndarray) -> np.ndarray:
    """Engine-convention harmonics of (not necessarily unit) vectors [...,3]."""
    xyz = np.asarray(xyz, dtype=np.float64)
    u = xyz / np.linalg.norm(xyz, axis=-1, keepdims=True)
    shuffled = np.stack([u[..., 2], u[..., 0], u[..., 1]], axis=-1)
    return 2.0 * sqrt(pi) * real_sph_harm_std(shuffled)


@lru_cache(maxsize=None)
def _cg_complex(j1: int, m1: int, j2: int, m2: int, j: int, m: int) -> float:
    """<j1 m1 j2 m2 | j m>, Condon-Shortley phases (Racah's closed form)."""
    if m1 + m2 != m or j < abs(j1 - j2) or j > j1 + j2:
        return 0.0
    if abs(m1) > j1 or abs(m2) > j2 or abs(m) > j:
        return 0.0
    f = factorial
    pref = Fraction((2 * j + 1) * f(j + j1 - j2) * f(j - j1 + j2) * f(j1 + j2 - j),
                    f(j1 + j2 + j + 1))
    pref *= f(j + m) * f(j - m) * f(j1 - m1) * f(j1 + m1) * f(j2 - m2) * f(j2 + m2)
    s = Fraction(0)
    for k in range(0, j1 + j2 - j + 1):
        d = [k, j1 + j2 - j - k, j1 - m1 - k, j2 + m2 - k, j - j2 + m1 + k, j - j1 - m2 + k]
        if min(d) < 0:
            continue
        den = 1
        for q in d:
            den *= f(q)
        s += Fraction((-1) ** k, den)
    return float(s) * sqrt(float(pref))


@lru_cache(maxsize=None)
def _real_to_complex(l: int) -> np.ndarray:
    """T[m_real, m_complex] with Y^real_{l,a} = sum_b T[a,b] Y^complex_{l,b}."""
    T = np.zeros((2 * l + 1, 2 * l + 1), dtype=np.complex128)
    T[l, l] = 1.0
    for m in range(1, l + 1):
        # m > 0: (1/sqrt2) ((-1)^m Y_l^m + Y_l^-m)
        T[l + m, l + m] = (-1) ** m / sqrt(2.0)
        T[l + m, l - m] = 1.0 / sqrt(2.0)
        # m < 0: (i/sqrt2) (Y_l^-|m| - (-1)^m Y_l^|m|)
        T[l - m, l - m] = 1j / sqrt(2.0)
        T[l - m, l + m] = -1j * (-1) ** m / sqrt(2.0)
    return T


@lru_cache(maxsize=None)
def real_cg(l1: int, l2: int, l: int) -> np.ndarray:
    """Real intertwiner C[m1, m2, m] for Y_l1 (x) Y_l2 -> Y_l in the real basis.

    For l1+l2+l even the transformed complex coefficients are real; for an odd
    sum they are purely imaginary and the imaginary part is the (equally valid,
    antisymmetric, cross-product-like) real intertwiner.  Normalised so that
    sum_{m1 m2} C[m1,m2,m]^2 = 1 for every m.
    """
    Cc = np.zeros((2 * l1 + 1, 2 * l2 + 1, 2 * l + 1))
    for m1 in range(-l1, l1 + 1):
        for m2 in range(-l2, l2 + 1):
            m = m1 + m2
            if abs(m) <= l:
                Cc[l1 + m1, l2 + m2, l + m] = _cg_complex(l1, m1, l2, m2, l, m)
    T1, T2, T3 = _real_to_complex(l1), _real_to_complex(l2), _real_to_complex(l)
    Cr = np.einsum("ab,cd,ef,bdf->ace", T1, T2, np.conj(T3), Cc.astype(np.complex128))
    part = Cr.real if (l1 + l2 + l) % 2 == 0 else Cr.imag
    other = Cr.imag if (l1 + l2 + l) % 2 == 0 else Cr.real
    assert np.abs(other).max() < 1e-12
    return np.ascontiguousarray(part)


def tensor_product_paths(l_max: int, L_max: int):
    """Layer-1 paths (l_out, l_Y, l_H) sorted by l_out.

    Mirrors what the extractor reads off `interactions[1].conv_tp`
    (extract_mace_data.py:323-325): every (l1 = order of Y, l2 = order of H1)
    coupling to l <= l_max with the parity rule l1+l2+l even (irreps are
    0e,1o,2e,3o), instructions sorted by output order.
    """
    paths = []
    for l in range(l_max + 1):
        for l2 in range(L_max + 1):
            for l1 in range(l_max + 1):
                if abs(l1 - l2) <= l <= l1 + l2 and (l1 + l2 + l) % 2 == 0:
                    paths.append((l, l1, l2))
    paths.sort(key=lambda p: p[0])
    return paths


def symmetric_contraction_terms(L: int, l_max: int, correlation: int):
    """Coupling tensors of the product basis for output order L.

    Returns a list over `eta` of dicts {M_index: {sorted lm-tuple: coeff}},
    one per coupling scheme, for body orders 1..correlation.  The same
    accumulation on sorted tuples with a 1e-12 magnitude threshold as the
    extractor (extract_mace_data.py:247-272).  Output parity is (-1)^L.
    """
    terms = []

    def lm(l, m):
        return l * l + l + m

    # nu = 1
    if L <= l_max:
        terms.append({M: {(lm(L, M - L),): 1.0} for M in range(2 * L + 1)})
    # nu = 2
    if correlation >= 2:
        for l1 in range(l_max + 1):
            for l2 in range(l1, l_max + 1):
                if not (abs(l1 - l2) <= L <= l1 + l2) or (l1 + l2 + L) % 2:
                    continue
                C = real_cg(l1, l2, L)
                t = {}
                for M in range(2 * L + 1):
                    d = {}
                    for a in range(2 * l1 + 1):
                        for b in range(2 * l2 + 1):
                            c = C[a, b, M]
                            if abs(c) > 1e-12:
                                key = tuple(sorted((lm(l1, a - l1), lm(l2, b - l2))))
                                d[key] = d.get(key, 0.0) + c
                    t[M] = {k: v for k, v in d.items() if abs(v) > 1e-12}
                if any(t[M] for M in t):
                    terms.append(t)
    # nu = 3
    if correlation >= 3:
        for l1 in range(l_max + 1):
            for l2 in range(l1, l_max + 1):
                for l3 in range(l2, l_max + 1):
                    if (l1 + l2 + l3 + L) % 2:
                        continue
                    for l12 in range(abs(l1 - l2), l1 + l2 + 1):
                        if not (abs(l12 - l3) <= L <= l12 + l3):
                            continue
                        C12 = real_cg(l1, l2, l12)
                        C3 = real_cg(l12, l3, L)
                        U = np.einsum("abi,icM->abcM", C12, C3)
                        t = {}
                        for M in range(2 * L + 1):
                            d = {}
                            nz = np.argwhere(np.abs(U[..., M]) > 1e-12)
                            for a, b, c in nz:
                                key = tuple(sorted((lm(l1, int(a) - l1), lm(l2, int(b) - l2), lm(l3, int(c) - l3))))
                                d[key] = d.get(key, 0.0) + float(U[a, b, c, M])
                            t[M] = {k: v for k, v in d.items() if abs(v) > 1e-12}
                        if any(t[M] for M in t):
                            terms.append(t)
    return terms
