"""Python face of the engine: class MACE with the names of the reference's
pybind class (symmetrix/source/cpp/mace.cpp:12-243), implemented over the C ABI.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib

_ARRAYS = ["node_forces", "node_energies", "H0_weights", "R0", "R1", "Y", "Y_grad", "A0", "A0_adj", "M0",
           "M0_grad", "M0_adj", "H1", "H1_adj", "Phi1", "Phi1_adj", "A1", "A1_adj", "M1", "M1_grad", "M1_adj",
           "H2", "H2_adj", "Phi0"]


def _i(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _d(a):
    return np.ascontiguousarray(a, dtype=np.float64)


def _pi(a):
    return a.ctypes.data_as(C.POINTER(C.c_int))


def _pd(a):
    return a.ctypes.data_as(C.POINTER(C.c_double))


class MACE:
    """Two-layer MACE evaluator on one MI355X.

    MACE(filename, dtype="float64"): dtype "float32" selects the fp32-feature
    mode (the reference's MACEKokkosFloat split of precisions).
    """

    def __init__(self, filename, dtype="float64"):
        object.__setattr__(self, "_h", None)
        if dtype not in ("float64", "float32"):
            raise ValueError(f"Unsupported dtype '{dtype}'. Supported dtypes are 'float64' and 'float32'.")
        L = _lib.lib()
        self._L = L
        h = C.c_void_p()
        flags = _lib.SMX_FP64 if dtype == "float64" else _lib.SMX_FP32_FEATURES
        _lib.check(L.smx_model_load(str(filename).encode(), flags, C.byref(h)))
        self._h = h
        self.dtype = dtype
        n = C.c_int()
        T = self._int("num_elements")
        buf = (C.c_int * T)()
        _lib.check(L.smx_model_get_atomic_numbers(self._h, buf, T, C.byref(n)))
        self.atomic_numbers = list(buf)
        ebuf = (C.c_double * T)()
        _lib.check(L.smx_model_get_atomic_energies(self._h, ebuf, T, C.byref(n)))
        self.atomic_energies = list(ebuf)
        v = C.c_double()
        _lib.check(L.smx_model_get_double(self._h, b"r_cut", C.byref(v)))
        self.r_cut = v.value
        for key in ("num_elements", "num_channels", "l_max", "num_lm", "L_max", "num_LM", "num_lme", "num_lelm1lm2"):
            object.__setattr__(self, key, self._int(key))
        self.has_zbl = bool(self._int("has_zbl"))

    def _int(self, key):
        v = C.c_int()
        _lib.check(self._L.smx_model_get_int(self._h, key.encode(), C.byref(v)))
        return v.value

    def __del__(self):
        if getattr(self, "_h", None):
            self._L.smx_model_free(self._h)
            self._h = None

    # --- read/write members ------------------------------------------------
    def __getattr__(self, name):
        if name in _ARRAYS:
            n = C.c_long()
            _lib.check(self._L.smx_get_array(self._h, name.encode(), None, 0, C.byref(n)))
            out = np.zeros(n.value)
            if n.value:
                _lib.check(self._L.smx_get_array(self._h, name.encode(), _pd(out), n.value, C.byref(n)))
            return out
        raise AttributeError(name)

    def __setattr__(self, name, value):
        if name in _ARRAYS:
            a = _d(value).reshape(-1)
            _lib.check(self._L.smx_set_array(self._h, name.encode(), _pd(a), C.c_long(len(a))))
        else:
            object.__setattr__(self, name, value)

    # --- whole pipeline ----------------------------------------------------
    def compute_node_energies_forces(self, num_nodes, node_types, num_neigh, neigh_indices, neigh_types, xyz, r):
        nt, nn, ni, nty = _i(node_types), _i(num_neigh), _i(neigh_indices), _i(neigh_types)
        x, rr = _d(xyz).reshape(-1), _d(r)
        if len(x) != 3 * len(rr) or len(ni) != len(rr) or len(nty) != len(rr):
            raise ValueError("edge arrays differ in length")
        if len(nt) < num_nodes or len(nn) < num_nodes:
            raise ValueError("node arrays shorter than num_nodes")
        _lib.check(self._L.smx_compute_node_energies_forces(
            self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(ni), _pi(nty), _pd(x), _pd(rr), C.c_long(len(rr))))

    def compute_ghosted(self, num_local_nodes, num_ghost_nodes, node_types, num_neigh, neigh_indices, neigh_types, xyz, r):
        """Ghost atoms as extra nodes that go through layer 0 only: the no_mpi_message_passing mode of the pair
        style (pair_symmetrix/pair_symmetrix_mace.cpp:557-748).  Local nodes and their edges come first."""
        nt, nn, ni, nty = _i(node_types), _i(num_neigh), _i(neigh_indices), _i(neigh_types)
        x, rr = _d(xyz).reshape(-1), _d(r)
        n = int(num_local_nodes) + int(num_ghost_nodes)
        if len(nt) < n or len(nn) < n or len(ni) != len(rr) or len(nty) != len(rr) or len(x) != 3 * len(rr):
            raise ValueError("array lengths do not match the node and edge counts")
        _lib.check(self._L.smx_compute_ghosted(
            self._h, int(num_local_nodes), int(num_ghost_nodes), _pi(nt), _pi(nn), _pi(ni), _pi(nty), _pd(x), _pd(rr),
            C.c_long(len(rr))))

    def compute_device(self, num_nodes, node_types, num_neigh, neigh_indices, neigh_types, xyz, r, num_edges,
                       node_energies=0, node_forces=0, stream=0):
        """Device-resident variant: every argument is a device address (int)."""
        _lib.check(self._L.smx_compute_device(
            self._h, int(num_nodes), C.c_void_p(node_types), C.c_void_p(num_neigh), C.c_void_p(neigh_indices),
            C.c_void_p(neigh_types), C.c_void_p(xyz), C.c_void_p(r), C.c_long(num_edges),
            C.c_void_p(node_energies), C.c_void_p(node_forces), C.c_void_p(stream)))

    def compute_ghosted_device(self, num_local_nodes, num_ghost_nodes, node_types, num_neigh, neigh_indices, neigh_types,
                               xyz, r, num_edges, num_local_edges, node_energies=0, node_forces=0, stream=0):
        """compute_ghosted with every array a device address (int); does not synchronise."""
        _lib.check(self._L.smx_compute_ghosted_device(
            self._h, int(num_local_nodes), int(num_ghost_nodes), C.c_void_p(node_types), C.c_void_p(num_neigh),
            C.c_void_p(neigh_indices), C.c_void_p(neigh_types), C.c_void_p(xyz), C.c_void_p(r), C.c_long(num_edges),
            C.c_long(num_local_edges), C.c_void_p(node_energies), C.c_void_p(node_forces), C.c_void_p(stream)))

    def synchronize(self):
        _lib.check(self._L.smx_synchronize(self._h))

    def set_staging_limit(self, nbytes):
        """Bound for the buffer of per-edge adjoint messages; longer edge lists are taken in receiver chunks."""
        _lib.check(self._L.smx_set_staging_limit(self._h, C.c_long(int(nbytes))))

    def set_profiling(self, enabled):
        _lib.check(self._L.smx_set_profiling(self._h, int(bool(enabled))))

    def stage_times(self):
        names = self._L.smx_stage_names().decode().split(";")
        buf = (C.c_float * len(names))()
        n = C.c_int()
        _lib.check(self._L.smx_get_stage_times(self._h, buf, len(names), C.byref(n)))
        return dict(zip(names, list(buf)))

    def reduce_forces(self, num_atoms, sender_atom, receiver_atom=None, virial=False):
        sa = _i(sender_atom)
        ra = _i(receiver_atom) if receiver_atom is not None else None
        F = np.zeros((num_atoms, 3))
        V = np.zeros(6)
        _lib.check(self._L.smx_reduce_forces(self._h, int(num_atoms), _pi(sa), _pi(ra) if ra is not None else None,
                                             _pd(F), _pd(V) if virial else None))
        return (F, V) if virial else F

    def reduce_forces_device(self, num_atoms, sender_atom_ptr, virial=False):
        """reduce_forces with the per-edge sender atoms in a device array (receiver i = atom i)."""
        F = np.zeros((num_atoms, 3))
        V = np.zeros(6)
        _lib.check(self._L.smx_reduce_forces_device(self._h, int(num_atoms), C.c_void_p(sender_atom_ptr), _pd(F),
                                                    _pd(V) if virial else None))
        return (F, V) if virial else F

    # --- stages --------------------------------------------------------------
    @property
    def zbl(self):
        """The `zbl` member of the reference class (libsymmetrix/source/mace.hpp:39): `mace.zbl.compute_ZBL(...)`."""
        return _ZBL(self)

    def compute_ZBL(self, num_nodes, node_types, num_neigh, neigh_types, r, xyz):
        """Pair repulsion added to this model's node_energies / node_forces (zbl.cpp:96-125), the call the pair
        style makes before the stage sequence (pair_symmetrix_mace.cpp:449-452).  No-op without ZBL."""
        nt, nn, nty = _i(node_types), _i(num_neigh), _i(neigh_types)
        x, rr = _d(xyz).reshape(-1), _d(r)
        if len(x) != 3 * len(rr) or len(nty) != len(rr):
            raise ValueError("edge arrays differ in length")
        _lib.check(self._L.smx_compute_ZBL(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(rr), _pd(x),
                                           C.c_long(len(rr))))

    def fill(self, name, n, value=0.0):
        """`name` sized to n entries equal to value, on the device (no host copy)."""
        _lib.check(self._L.smx_fill_array(self._h, name.encode(), C.c_long(int(n)), C.c_double(float(value))))

    def compute_Y(self, xyz):
        x = _d(xyz).reshape(-1)
        _lib.check(self._L.smx_compute_Y(self._h, _pd(x), C.c_long(len(x))))

    def compute_R0(self, num_nodes, node_types, num_neigh, neigh_types, r):
        nt, nn, nty, rr = _i(node_types), _i(num_neigh), _i(neigh_types), _d(r)
        _lib.check(self._L.smx_compute_R0(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(rr), C.c_long(len(rr))))

    def compute_R1(self, num_nodes, node_types, num_neigh, neigh_types, r):
        nt, nn, nty, rr = _i(node_types), _i(num_neigh), _i(neigh_types), _d(r)
        _lib.check(self._L.smx_compute_R1(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(rr), C.c_long(len(rr))))

    def compute_A0(self, num_nodes, node_types, num_neigh, neigh_types):
        nt, nn, nty = _i(node_types), _i(num_neigh), _i(neigh_types)
        _lib.check(self._L.smx_compute_A0(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), C.c_long(len(nty))))

    def reverse_A0(self, num_nodes, node_types, num_neigh, neigh_types, xyz, r):
        nt, nn, nty = _i(node_types), _i(num_neigh), _i(neigh_types)
        x, rr = _d(xyz).reshape(-1), _d(r)
        _lib.check(self._L.smx_reverse_A0(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(x), _pd(rr), C.c_long(len(rr))))

    def compute_A0_scaled(self, num_nodes, node_types, num_neigh, neigh_types, r):
        nt, nn, nty, rr = _i(node_types), _i(num_neigh), _i(neigh_types), _d(r)
        _lib.check(self._L.smx_compute_A0_scaled(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(rr), C.c_long(len(rr))))

    def reverse_A0_scaled(self, num_nodes, node_types, num_neigh, neigh_types, xyz, r):
        nt, nn, nty = _i(node_types), _i(num_neigh), _i(neigh_types)
        x, rr = _d(xyz).reshape(-1), _d(r)
        _lib.check(self._L.smx_reverse_A0_scaled(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(x), _pd(rr),
                                                 C.c_long(len(rr))))

    def compute_A1_scaled(self, num_nodes, node_types, num_neigh, neigh_types, r):
        nt, nn, nty, rr = _i(node_types), _i(num_neigh), _i(neigh_types), _d(r)
        _lib.check(self._L.smx_compute_A1_scaled(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(rr), C.c_long(len(rr))))

    def reverse_A1_scaled(self, num_nodes, node_types, num_neigh, neigh_types, xyz, r, zero_dxyz=True):
        nt, nn, nty = _i(node_types), _i(num_neigh), _i(neigh_types)
        x, rr = _d(xyz).reshape(-1), _d(r)
        _lib.check(self._L.smx_reverse_A1_scaled(self._h, int(num_nodes), _pi(nt), _pi(nn), _pi(nty), _pd(x), _pd(rr),
                                                 C.c_long(len(rr)), int(bool(zero_dxyz))))

    def compute_M0(self, num_nodes, node_types):
        nt = _i(node_types)
        _lib.check(self._L.smx_compute_M0(self._h, int(num_nodes), _pi(nt)))

    def reverse_M0(self, num_nodes, node_types):
        nt = _i(node_types)
        _lib.check(self._L.smx_reverse_M0(self._h, int(num_nodes), _pi(nt)))

    def compute_H1(self, num_nodes):
        _lib.check(self._L.smx_compute_H1(self._h, int(num_nodes)))

    def reverse_H1(self, num_nodes):
        _lib.check(self._L.smx_reverse_H1(self._h, int(num_nodes)))

    def compute_Phi1(self, num_nodes, num_neigh, neigh_indices):
        nn, ni = _i(num_neigh), _i(neigh_indices)
        _lib.check(self._L.smx_compute_Phi1(self._h, int(num_nodes), _pi(nn), _pi(ni), C.c_long(len(ni))))

    def reverse_Phi1(self, num_nodes, num_neigh, neigh_indices, xyz, r, zero_dxyz=True, zero_H1_adj=True):
        nn, ni = _i(num_neigh), _i(neigh_indices)
        x, rr = _d(xyz).reshape(-1), _d(r)
        _lib.check(self._L.smx_reverse_Phi1(self._h, int(num_nodes), _pi(nn), _pi(ni), _pd(x), _pd(rr),
                                            C.c_long(len(rr)), int(zero_dxyz), int(zero_H1_adj)))

    def compute_A1(self, num_nodes):
        _lib.check(self._L.smx_compute_A1(self._h, int(num_nodes)))

    def reverse_A1(self, num_nodes):
        _lib.check(self._L.smx_reverse_A1(self._h, int(num_nodes)))

    def compute_M1(self, num_nodes, node_types):
        nt = _i(node_types)
        _lib.check(self._L.smx_compute_M1(self._h, int(num_nodes), _pi(nt)))

    def reverse_M1(self, num_nodes, node_types):
        nt = _i(node_types)
        _lib.check(self._L.smx_reverse_M1(self._h, int(num_nodes), _pi(nt)))

    def compute_H2(self, num_nodes, node_types):
        nt = _i(node_types)
        _lib.check(self._L.smx_compute_H2(self._h, int(num_nodes), _pi(nt)))

    def reverse_H2(self, num_nodes, node_types, zero_H1_adj=True):
        nt = _i(node_types)
        _lib.check(self._L.smx_reverse_H2(self._h, int(num_nodes), _pi(nt), int(zero_H1_adj)))

    def compute_readouts(self, num_nodes, node_types):
        nt = _i(node_types)
        _lib.check(self._L.smx_compute_readouts(self._h, int(num_nodes), _pi(nt)))


class _ZBL:
    """`compute_ZBL` with the argument list of libsymmetrix/source/zbl.hpp:26-34.  The pair repulsion is added on the
    device to the owning model's node_energies / node_forces; the two output arguments are written as well when they
    are numpy arrays."""

    def __init__(self, owner):
        self._o = owner

    def compute_ZBL(self, num_nodes, node_types, num_neigh, neigh_types, atomic_numbers, r, xyz, node_energies=None,
                    node_forces=None):
        o = self._o
        if list(atomic_numbers) != list(o.atomic_numbers):
            raise ValueError("compute_ZBL: atomic_numbers must be the model's own species table")
        if node_energies is not None:
            o.node_energies = node_energies
        if node_forces is not None:
            o.node_forces = node_forces
        o.compute_ZBL(num_nodes, node_types, num_neigh, neigh_types, r, xyz)
        if isinstance(node_energies, np.ndarray):
            node_energies[...] = o.node_energies[:node_energies.size].reshape(node_energies.shape)
        if isinstance(node_forces, np.ndarray):
            node_forces[...] = o.node_forces[:node_forces.size].reshape(node_forces.shape)
