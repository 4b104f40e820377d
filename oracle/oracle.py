"""Python face of the CPU oracle (test infrastructure, not the product).

Loads a symmetrix JSON model with the standard-library json module, rebuilds
the polynomial product graphs the way the reference constructor does
(libsymmetrix/source/multivariate_polynomial.cpp:10-101, with
`_two_part_partitions` from libsymmetrix/source/tools.cpp:69-109) and drives
the C restatement in mace_oracle.c through ctypes.  Method and attribute names
follow the reference's pybind class (symmetrix/source/cpp/mace.cpp:12-243) so
that tests read like the reference's own.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this module.
"""
from __future__ import annotations

import ctypes as C
import json
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference tree exists)."""
    so = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(os.path.join(_HERE, "mace_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        L = C.CDLL(so)
        L.orc_model_create.restype = C.c_void_p
        L.orc_get.restype = C.POINTER(C.c_double)
        L.orc_poly_evaluate_gradient.restype = C.c_double
        L.orc_mlp_evaluate_gradient.restype = C.c_double
        _LIB = L
    return _LIB


def ref_lib():
    """The reference leaf objects (oracle/_ref/libsmxref.so) or None."""
    so = os.path.join(_HERE, "_ref", "libsmxref.so")
    if not os.path.exists(so):
        return None
    L = C.CDLL(so)
    for n in ("ref_spline_set_create", "ref_spline_create", "ref_zbl_create"):
        getattr(L, n).restype = C.c_void_p
    for n in ("ref_zbl_compute", "ref_zbl_compute_gradient", "ref_zbl_envelope"):
        getattr(L, n).restype = C.c_double
    return L


def _d(a):
    return np.ascontiguousarray(a, dtype=np.float64)


def _i(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _pd(a):
    return a.ctypes.data_as(C.POINTER(C.c_double))


def _pi(a):
    return a.ctypes.data_as(C.POINTER(C.c_int))


# ---------------------------------------------------------------------------
def two_part_partitions(v):
    """tools.cpp:69-109: all splits of the sequence v into two non-empty
    subsequences, in the order the reference generates them."""
    v = list(v)
    if not v:
        return []
    partitions = [[[v[0]]]]
    for x in v[1:]:
        prev = partitions
        partitions = []
        for pp in prev:
            if len(pp) == 1:
                partitions.append([list(s) for s in pp] + [[x]])
            if len(pp) <= 2:
                for j in range(len(pp)):
                    q = [list(s) for s in pp]
                    q[j].append(x)
                    partitions.append(q)
    partitions = [p for p in partitions if len(p) != 1]
    partitions.sort(key=len)  # stable; every survivor has two parts
    return partitions


def build_product_graph(num_variables, coefficients, monomials):
    """multivariate_polynomial.cpp:10-101.

    Returns (nodes, edges, node_coefficients, num_auxiliary_nodes): nodes in
    "shorter first, then lexicographic" order; edges[e] = indices of the two
    parents of node num_variables+e; coefficients placed on their nodes.
    """
    key = lambda t: (len(t), t)
    table = {}
    for c, mono in zip(coefficients, monomials):
        table.setdefault(tuple(mono), c)  # std::map::insert keeps the first
    monos = sorted(table, key=key)
    coefs = [table[t] for t in monos]

    node_set = {(i,) for i in range(num_variables)} | set(monos)

    def find_parents(node):
        for part in two_part_partitions(node):
            if tuple(part[0]) in node_set and tuple(part[1]) in node_set:
                return tuple(part[0]), tuple(part[1])
        return None

    num_aux = 0
    for node in sorted(node_set, key=key):  # inserted nodes are shorter, hence never revisited
        if len(node) == 1:
            continue
        cur = node
        factors = find_parents(cur)
        while factors is None:
            cur = cur[:-1]
            node_set.add(cur)
            num_aux += 1
            factors = find_parents(cur)
    nodes = sorted(node_set, key=key)
    index = {n: i for i, n in enumerate(nodes)}
    edges = []
    for node in nodes:
        if len(node) == 1:
            continue
        f0, f1 = find_parents(node)
        edges.append((index[f0], index[f1]))
    node_coefficients = np.zeros(len(nodes))
    for t, c in zip(monos, coefs):
        node_coefficients[index[t]] = c
    return nodes, edges, node_coefficients, num_aux


# ---------------------------------------------------------------------------
class OracleMACE:
    """CPU oracle with the reference's Python-binding surface."""

    _ARRAYS = ["node_forces", "node_energies", "R0", "R0_deriv", "R1", "R1_deriv", "Y", "Y_grad",
               "A0", "A0_adj", "M0", "M0_grad", "M0_adj", "H1", "H1_adj", "Phi1", "Phi1_adj",
               "Phi1r", "dPhi1r", "A1", "A1_adj", "M1", "M1_grad", "M1_adj", "H2", "H2_adj"]

    def __init__(self, model):
        if isinstance(model, (str, os.PathLike)):
            with open(model) as f:
                model = json.load(f)
        else:
            model = json.loads(json.dumps(model))  # integer dict keys become strings, as in a file
        self.file = model
        L = lib()
        object.__setattr__(self, "_h", None)
        self._L = L
        self._h = C.c_void_p(L.orc_model_create())
        T = int(model["num_elements"]); K = int(model["num_channels"])
        self.num_elements, self.num_channels = T, K
        self.r_cut = float(model["r_cut"])
        self.l_max = int(model["l_max"]); self.L_max = int(model["L_max"])
        self.num_lm = (self.l_max + 1) ** 2; self.num_LM = (self.L_max + 1) ** 2
        self.atomic_numbers = [int(z) for z in model["atomic_numbers"]]
        an = _i(self.atomic_numbers); ae = _d(model["atomic_energies"])
        L.orc_model_set_basic(self._h, T, K, self.l_max, self.L_max, C.c_double(self.r_cut), _pi(an), _pd(ae))
        h = float(model["radial_spline_h"])
        for which in (0, 1):
            v = _d(model[f"radial_spline_values_{which}"]); d = _d(model[f"radial_spline_derivs_{which}"])
            L.orc_model_set_radial(self._h, which, C.c_double(h), v.shape[0], v.shape[1], v.shape[2], _pd(v), _pd(d))
        for which, name in ((0, "A0"), (1, "A1")):
            if model[f"{name}_scaled"]:
                v = _d(model[f"{name}_spline_values"]); d = _d(model[f"{name}_spline_derivs"])
                L.orc_model_set_scaling(self._h, which, C.c_double(float(model[f"{name}_spline_h"])),
                                        v.shape[0], v.shape[1], _pd(v), _pd(d))
        if model["has_zbl"]:
            c = _d(model["zbl_c"]); rad = _d(model["zbl_covalent_radii"])
            L.orc_model_set_zbl(self._h, C.c_double(model["zbl_a_exp"]), C.c_double(model["zbl_a_prefactor"]),
                                _pd(c), _pd(rad), len(rad), int(model["zbl_p"]))
        self.H0_weights = _d(model["H0_weights"])
        A0w = _d(model["A0_weights"]); H1w = _d(model["H1_weights"])
        H2H1 = _d(model["H2_weights_for_H1"]); H2M1 = _d(model["H2_weights_for_M1"])
        ro1 = _d(model["readout_1_weights"]); w1 = _d(model["readout_2_weights_1"]); w2 = _d(model["readout_2_weights_2"])
        L.orc_model_set_weights(self._h, _pd(self.H0_weights), _pd(A0w), _pd(H1w), _pd(H2H1), _pd(H2M1),
                                _pd(ro1), _pd(w1), _pd(w2), C.c_double(float(model["readout_2_scale_factor"])))
        # polynomials: one graph per LM (identical for every species and channel)
        self.graphs0 = []
        for LM in range(self.num_LM):
            monos = model["M0_monomials"][str(LM)]
            w = model["M0_weights"]
            nodes, edges, _, _ = build_product_graph(self.num_lm, [0.0] * len(monos), monos)
            self.graphs0.append((nodes, edges))
            coef = np.zeros((T, K, len(nodes)))
            for a in range(T):
                for k in range(K):
                    coef[a, k] = self._place(nodes, monos, w[str(a)][str(LM)][str(k)])
            e = _i(edges).reshape(-1)
            L.orc_model_set_poly(self._h, 0, LM, self.num_lm, len(nodes), _pi(e), _pd(_d(coef)))
        monos = model["M1_monomials"]
        nodes, edges, _, _ = build_product_graph(self.num_lm, [0.0] * len(monos), monos)
        self.graph1 = (nodes, edges)
        coef = np.zeros((T, K, len(nodes)))
        for a in range(T):
            for k in range(K):
                coef[a, k] = self._place(nodes, monos, model["M1_weights"][str(a)][str(k)])
        e = _i(edges).reshape(-1)
        L.orc_model_set_poly(self._h, 1, 0, self.num_lm, len(nodes), _pi(e), _pd(_d(coef)))
        l = _i(model["Phi1_l"]); l1 = _i(model["Phi1_l1"]); l2 = _i(model["Phi1_l2"])
        lme = _i(model["Phi1_lme"]); cgv = _d(model["Phi1_clebsch_gordan"]); q = _i(model["Phi1_lelm1lm2"])
        L.orc_model_set_phi1(self._h, len(l), _pi(l), _pi(l1), _pi(l2), len(lme), _pi(lme), _pd(cgv), _pi(q))
        for li, w in enumerate(model["A1_weights"]):
            w = _d(w)
            L.orc_model_set_A1_weights(self._h, li, _pd(w), len(w))

    @staticmethod
    def _place(nodes, monos, coefs):
        """Coefficients on their graph nodes (first occurrence wins, as std::map::insert)."""
        index = {n: i for i, n in enumerate(nodes)}
        out = np.zeros(len(nodes))
        seen = set()
        for c, mono in zip(coefs, monos):
            t = tuple(mono)
            if t in seen:
                continue
            seen.add(t)
            out[index[t]] = c
        return out

    def __del__(self):
        if getattr(self, "_h", None):
            self._L.orc_model_free(self._h)
            self._h = None

    # read/write access to intermediates, as the pybind def_readwrite members
    def __getattr__(self, name):
        if name in OracleMACE._ARRAYS:
            n = C.c_long()
            p = self._L.orc_get(self._h, name.encode(), C.byref(n))
            if n.value <= 0:
                return np.zeros(0)
            return np.ctypeslib.as_array(p, shape=(n.value,)).copy()
        raise AttributeError(name)

    def __setattr__(self, name, value):
        if name in OracleMACE._ARRAYS:
            a = _d(value).reshape(-1)
            self._L.orc_set(self._h, name.encode(), _pd(a), len(a))
        else:
            object.__setattr__(self, name, value)

    # --- stages -----------------------------------------------------------
    def compute_node_energies_forces(self, num_nodes, node_types, num_neigh, neigh_indices, neigh_types, xyz, r):
        nt, nn, ni, nty = _i(node_types), _i(num_neigh), _i(neigh_indices), _i(neigh_types)
        x, rr = _d(xyz).reshape(-1), _d(r)
        rc = self._L.orc_compute_node_energies_forces(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(ni), _pi(nty),
                                                      _pd(x), _pd(rr), C.c_long(len(rr)))
        if rc:
            raise ValueError("Out of bounds in CubicSpline::evaluate.")

    def compute_Y(self, xyz):
        x = _d(xyz).reshape(-1)
        self._L.orc_compute_Y(self._h, _pd(x), C.c_long(len(x)))

    def compute_R0(self, num_nodes, node_types, num_neigh, neigh_types, r):
        nt, nn, nty, rr = _i(node_types), _i(num_neigh), _i(neigh_types), _d(r)
        self._L.orc_compute_R0(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(rr), C.c_long(len(rr)))

    def compute_R1(self, num_nodes, node_types, num_neigh, neigh_types, r):
        nt, nn, nty, rr = _i(node_types), _i(num_neigh), _i(neigh_types), _d(r)
        self._L.orc_compute_R1(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(rr), C.c_long(len(rr)))

    def compute_A0(self, num_nodes, node_types, num_neigh, neigh_types):
        nt, nn, nty = _i(node_types), _i(num_neigh), _i(neigh_types)
        self._L.orc_compute_A0(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty))

    def reverse_A0(self, num_nodes, node_types, num_neigh, neigh_types, xyz, r):
        nt, nn, nty = _i(node_types), _i(num_neigh), _i(neigh_types)
        x, rr = _d(xyz).reshape(-1), _d(r)
        self._L.orc_reverse_A0(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(x), _pd(rr))

    def compute_A0_scaled(self, num_nodes, node_types, num_neigh, neigh_types, r):
        nt, nn, nty, rr = _i(node_types), _i(num_neigh), _i(neigh_types), _d(r)
        if self._L.orc_compute_A0_scaled(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(rr)):
            raise ValueError("Out of bounds in CubicSpline::evaluate.")

    def reverse_A0_scaled(self, num_nodes, node_types, num_neigh, neigh_types, xyz, r):
        nt, nn, nty = _i(node_types), _i(num_neigh), _i(neigh_types)
        x, rr = _d(xyz).reshape(-1), _d(r)
        if self._L.orc_reverse_A0_scaled(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(x), _pd(rr)):
            raise ValueError("Out of bounds in CubicSpline::evaluate.")

    def compute_A1_scaled(self, num_nodes, node_types, num_neigh, neigh_types, r):
        nt, nn, nty, rr = _i(node_types), _i(num_neigh), _i(neigh_types), _d(r)
        if self._L.orc_compute_A1_scaled(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(rr)):
            raise ValueError("Out of bounds in CubicSpline::evaluate.")

    def reverse_A1_scaled(self, num_nodes, node_types, num_neigh, neigh_types, xyz, r, zero_dxyz=True):
        nt, nn, nty = _i(node_types), _i(num_neigh), _i(neigh_types)
        x, rr = _d(xyz).reshape(-1), _d(r)
        if self._L.orc_reverse_A1_scaled(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(x), _pd(rr),
                                         C.c_long(len(x)), int(zero_dxyz)):
            raise ValueError("Out of bounds in CubicSpline::evaluate.")

    def compute_M0(self, num_nodes, node_types):
        nt = _i(node_types)
        self._L.orc_compute_M0(self._h, int(num_nodes), _pi(nt))

    def reverse_M0(self, num_nodes, node_types=None):
        self._L.orc_reverse_M0(self._h, int(num_nodes))

    def compute_H1(self, num_nodes):
        self._L.orc_compute_H1(self._h, int(num_nodes))

    def reverse_H1(self, num_nodes):
        self._L.orc_reverse_H1(self._h, int(num_nodes))

    def compute_Phi1(self, num_nodes, num_neigh, neigh_indices):
        nn, ni = _i(num_neigh), _i(neigh_indices)
        self._L.orc_compute_Phi1(self._h, int(num_nodes), _pi(nn), _pi(ni))

    def reverse_Phi1(self, num_nodes, num_neigh, neigh_indices, xyz, r, zero_dxyz=True, zero_H1_adj=True):
        nn, ni = _i(num_neigh), _i(neigh_indices)
        x, rr = _d(xyz).reshape(-1), _d(r)
        self._L.orc_reverse_Phi1(self._h, int(num_nodes), _pi(nn), _pi(ni), _pd(x), _pd(rr), C.c_long(len(x)),
                                 int(zero_dxyz), int(zero_H1_adj))

    def compute_A1(self, num_nodes):
        self._L.orc_compute_A1(self._h, int(num_nodes))

    def reverse_A1(self, num_nodes):
        self._L.orc_reverse_A1(self._h, int(num_nodes))

    def compute_M1(self, num_nodes, node_types):
        nt = _i(node_types)
        self._L.orc_compute_M1(self._h, int(num_nodes), _pi(nt))

    def reverse_M1(self, num_nodes, node_types=None):
        self._L.orc_reverse_M1(self._h, int(num_nodes))

    def compute_H2(self, num_nodes, node_types):
        nt = _i(node_types)
        self._L.orc_compute_H2(self._h, int(num_nodes), _pi(nt))

    def reverse_H2(self, num_nodes, node_types, zero_H1_adj=True):
        nt = _i(node_types)
        self._L.orc_reverse_H2(self._h, int(num_nodes), _pi(nt), int(zero_H1_adj))

    def compute_readouts(self, num_nodes, node_types):
        nt = _i(node_types)
        self._L.orc_compute_readouts(self._h, int(num_nodes), _pi(nt))
