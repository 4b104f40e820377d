"""Canonical full neighbour list for periodic cells (host, numpy).

The reference engine never sorts or filters edges: its callers hand it flat
per-receiver arrays (libsymmetrix/source/mace.cpp:17-24).  The LAMMPS caller
keeps pairs with r^2 < r_cut^2 computed from ghost-image coordinates
(pair_symmetrix/pair_symmetrix_mace.cpp:287-315); the ASE caller passes
neighbor_list('ijdD') through (symmetrix/source/symmetrix/symmetrix_calc.py:77-83).
Edge order there is whatever LAMMPS bins or matscipy produce, so this build
defines one canonical order that every builder here must reproduce exactly:

    receivers ascending; within a receiver senders ascending; several
    periodic images of the same sender ordered by cell shift (sx, sy, sz)
    lexicographically.

Image coordinates are formed first (x_j + S.cell, as LAMMPS ghosts are) and
then differenced with x_i, so xyz and r are bit-identical across builders.
"""
from __future__ import annotations

import numpy as np


def wrap_positions(positions, cell, pbc=(True, True, True), offsets=None):
    """Positions folded into the cell along the periodic axes, and the integer lattice offsets taken off:
    returns (wrapped [N,3], offsets int [N,3]) with positions = wrapped + offsets . cell.

    The builders below enumerate ceil(r_cut / height) image shells, which finds every pair only when all atoms
    lie within one cell span; molecular dynamics does not keep them there (the reference's caller hands
    unwrapped positions straight to neighbor_list('ijdD'), symmetrix_calc.py:77).  Atoms already inside the
    cell come back bit for bit (offset 0).  `offsets` ([N,3] integers) are taken off instead of the floor of
    the fractional coordinates: the frame of an earlier call, in which atoms that moved since may lie a
    little outside the cell."""
    pos = np.ascontiguousarray(positions, dtype=np.float64).reshape(-1, 3)
    cell = np.asarray(cell, dtype=np.float64)
    if cell.shape == (3,):
        cell = np.diag(cell)
    if len(pos) == 0:
        return pos, np.zeros((0, 3), dtype=np.int64)
    pbc = np.asarray(pbc, dtype=bool)
    frac = pos @ np.linalg.inv(cell)
    if not np.all(np.isfinite(frac)):
        raise ValueError("positions are not finite")
    if offsets is not None:
        off = np.asarray(offsets, dtype=np.int64).reshape(-1, 3)
        if off.shape != pos.shape:
            raise ValueError("offsets must hold three integers per atom")
    else:
        off = np.where(pbc[None, :], np.floor(frac), 0.0).astype(np.int64)
    if not off.any():
        return pos, off
    return pos - off.astype(np.float64) @ cell, off


def neighbor_list(positions, cell, r_cut, pbc=(True, True, True), offsets=None):
    """Full neighbour list of an orthorhombic or triclinic periodic cell.

    Returns dict with i, j (int32), S (int32 [E,3] cell shifts), xyz ([E,3] =
    x_j + S.cell - x_i), r ([E]), first_neigh ([N+1]) in canonical order.  Atoms may lie outside the cell:
    they are folded in first and the lattice offsets go into S, so that S still refers to the positions given.
    With `offsets` the list is formed in that frame instead (see wrap_positions).
    """
    pos_in = np.ascontiguousarray(positions, dtype=np.float64)
    cell = np.asarray(cell, dtype=np.float64)
    if cell.shape == (3,):
        cell = np.diag(cell)
    N = len(pos_in)
    if N == 0:
        return dict(i=np.zeros(0, np.int32), j=np.zeros(0, np.int32), S=np.zeros((0, 3), np.int32),
                    xyz=np.zeros((0, 3)), r=np.zeros(0), first_neigh=np.zeros(1, np.int64))
    pbc = np.asarray(pbc, dtype=bool)
    pos, wrap = wrap_positions(pos_in, cell, pbc, offsets)
    # number of image shells needed along each lattice vector
    vol = abs(np.linalg.det(cell))
    heights = np.array([vol / np.linalg.norm(np.cross(cell[(a + 1) % 3], cell[(a + 2) % 3])) for a in range(3)])
    inv = np.linalg.inv(cell)
    frac = pos @ inv
    lo_f = frac.min(axis=0) if N else np.zeros(3)
    hi_f = frac.max(axis=0) if N else np.zeros(3)
    # a pair (i, j + S) within r_cut has |f_j + S - f_i| <= r_cut / height along every axis: |S| <= r_cut / height +
    # (spread of the fractional coordinates), which is below ceil(r_cut / height) + 1 for atoms inside the cell
    nshell = np.maximum(np.ceil(r_cut / heights), np.floor(r_cut / heights + (hi_f - lo_f))).astype(int)
    nshell = np.where(pbc, nshell, 0)
    margin = r_cut / heights
    img_j, img_S, img_pos = [], [], []
    for sx in range(-nshell[0], nshell[0] + 1):
        for sy in range(-nshell[1], nshell[1] + 1):
            for sz in range(-nshell[2], nshell[2] + 1):
                S = np.array([sx, sy, sz])
                f = frac + S
                keep = np.all((f >= lo_f - margin - 1e-9) & (f <= hi_f + margin + 1e-9), axis=1)
                idx = np.nonzero(keep)[0]
                if len(idx) == 0:
                    continue
                img_j.append(idx)
                img_S.append(np.broadcast_to(S, (len(idx), 3)))
                shift = S.astype(np.float64) @ cell
                img_pos.append(pos[idx] + shift)
    img_j = np.concatenate(img_j); img_S = np.concatenate(img_S); img_pos = np.concatenate(img_pos)
    # bin images on a Cartesian grid of cell size >= r_cut
    lo = img_pos.min(axis=0) - 1e-6
    ext = img_pos.max(axis=0) + 1e-6 - lo
    nb = np.maximum(1, np.floor(ext / r_cut).astype(int))
    nb = np.minimum(nb, 256)
    bs = ext / nb
    def bins(p):
        b = np.floor((p - lo) / bs).astype(np.int64)
        return np.clip(b, 0, nb - 1)
    ib = bins(img_pos)
    flat = (ib[:, 0] * nb[1] + ib[:, 1]) * nb[2] + ib[:, 2]
    order = np.argsort(flat, kind="stable")
    flat_sorted = flat[order]
    nbin = int(nb.prod())
    starts = np.searchsorted(flat_sorted, np.arange(nbin + 1))
    lb = bins(pos)
    out_i, out_img = [], []
    r2cut = r_cut * r_cut
    for dx in (-1, 0, 1):
        for dy in (-1, 0, 1):
            for dz in (-1, 0, 1):
                nbx = lb + np.array([dx, dy, dz])
                ok = np.all((nbx >= 0) & (nbx < nb), axis=1)
                # skip duplicate visits when a dimension has fewer than 3 bins
                if (nb[0] == 1 and dx != 0) or (nb[1] == 1 and dy != 0) or (nb[2] == 1 and dz != 0):
                    continue
                ii = np.nonzero(ok)[0]
                if len(ii) == 0:
                    continue
                f = (nbx[ii, 0] * nb[1] + nbx[ii, 1]) * nb[2] + nbx[ii, 2]
                s, e = starts[f], starts[f + 1]
                cnt = e - s
                tot = int(cnt.sum())
                if tot == 0:
                    continue
                rep_i = np.repeat(ii, cnt)
                offs = np.arange(tot) - np.repeat(np.cumsum(cnt) - cnt, cnt)
                img = order[np.repeat(s, cnt) + offs]
                d = img_pos[img] - pos[rep_i]
                r2 = d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1] + d[:, 2] * d[:, 2]
                keep = r2 < r2cut
                keep &= ~((img_j[img] == rep_i) & np.all(img_S[img] == 0, axis=1))
                out_i.append(rep_i[keep]); out_img.append(img[keep])
    if out_i:
        ei = np.concatenate(out_i); eimg = np.concatenate(out_img)
    else:
        ei = np.zeros(0, dtype=np.int64); eimg = np.zeros(0, dtype=np.int64)
    ej = img_j[eimg]; eS = img_S[eimg]
    perm = np.lexsort((eS[:, 2], eS[:, 1], eS[:, 0], ej, ei))
    ei, ej, eS, eimg = ei[perm], ej[perm], eS[perm], eimg[perm]
    d = img_pos[eimg] - pos[ei]
    r = np.sqrt(d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1] + d[:, 2] * d[:, 2])
    first = np.zeros(N + 1, dtype=np.int64)
    np.add.at(first, ei + 1, 1)
    first = np.cumsum(first)
    # x_j + S.cell - x_i for the positions as given: the shift found for the folded atoms, corrected by their offsets
    eS = eS + wrap[ei] - wrap[ej]
    return dict(i=ei.astype(np.int32), j=ej.astype(np.int32), S=eS.astype(np.int32),
                xyz=np.ascontiguousarray(d), r=r, first_neigh=first)


def brute_force_neighbor_list(positions, cell, r_cut, pbc=(True, True, True)):
    """O(N^2 * images) reference for small cells (tests only)."""
    pos = np.asarray(positions, dtype=np.float64)
    cell = np.asarray(cell, dtype=np.float64)
    if cell.shape == (3,):
        cell = np.diag(cell)
    N = len(pos)
    vol = abs(np.linalg.det(cell))
    heights = np.array([vol / np.linalg.norm(np.cross(cell[(a + 1) % 3], cell[(a + 2) % 3])) for a in range(3)])
    nshell = np.where(np.asarray(pbc, bool), np.ceil(r_cut / heights).astype(int), 0)
    # edge vectors are defined on the folded positions (as in neighbor_list); shifts refer to the positions given
    pos, wrap = wrap_positions(pos, cell, pbc)
    rows = []
    for i in range(N):
        for j in range(N):
            for sx in range(-nshell[0], nshell[0] + 1):
                for sy in range(-nshell[1], nshell[1] + 1):
                    for sz in range(-nshell[2], nshell[2] + 1):
                        if i == j and sx == 0 and sy == 0 and sz == 0:
                            continue
                        pj = pos[j] + np.array([sx, sy, sz], dtype=np.float64) @ cell
                        d = pj - pos[i]
                        r2 = d[0] * d[0] + d[1] * d[1] + d[2] * d[2]
                        if r2 < r_cut * r_cut:
                            S = np.array([sx, sy, sz]) + wrap[i] - wrap[j]
                            rows.append((i, j, S[0], S[1], S[2], d[0], d[1], d[2], np.sqrt(r2)))
    rows.sort(key=lambda t: t[:5])
    a = np.array(rows, dtype=np.float64).reshape(-1, 9)
    return dict(i=a[:, 0].astype(np.int32), j=a[:, 1].astype(np.int32), S=a[:, 2:5].astype(np.int32),
                xyz=np.ascontiguousarray(a[:, 5:8]), r=a[:, 8].copy())


def edge_arrays(nl, species_index, num_nodes=None):
    """Flat arrays in the layout MACE::compute_node_energies_forces takes
    (libsymmetrix/source/mace.cpp:17-24)."""
    i, j = nl["i"], nl["j"]
    N = len(species_index) if num_nodes is None else num_nodes
    species_index = np.asarray(species_index, dtype=np.int32)
    return dict(
        num_nodes=N,
        node_types=species_index[:N].copy(),
        num_neigh=np.bincount(i, minlength=N).astype(np.int32),
        neigh_indices=j.astype(np.int32),
        neigh_types=species_index[j].astype(np.int32),
        xyz=np.ascontiguousarray(nl["xyz"], dtype=np.float64).reshape(-1),
        r=np.ascontiguousarray(nl["r"], dtype=np.float64),
    )


def ghost_edge_arrays(nl, species_index):
    """The same periodic system with ghost atoms as explicit nodes, as the pair style lays it out in its
    no_mpi_message_passing mode (pair_symmetrix/pair_symmetrix_mace.cpp:557-658).

    Local nodes 0..N-1 come first; every periodic image (j, S != 0) that neighbours a local atom becomes a ghost
    node, ordered by (j, S).  Edges of local receivers point at local or ghost nodes; a ghost node carries the
    edge list of its owner atom (only species, xyz and r of those edges are used).  sender_atom[edge] and
    receiver_atom[node] name the owners for the force scatter f[i] -= f_ij, f[j] += f_ij (:700-716).
    """
    i, j, S = nl["i"], nl["j"], np.asarray(nl["S"]).reshape(-1, 3)
    species_index = np.asarray(species_index, dtype=np.int32)
    N = len(species_index)
    first = np.asarray(nl["first_neigh"])
    xyz = np.asarray(nl["xyz"], dtype=np.float64).reshape(-1, 3)
    r = np.asarray(nl["r"], dtype=np.float64)
    is_img = np.any(S != 0, axis=1)
    keys = np.concatenate([j[is_img, None].astype(np.int64), S[is_img].astype(np.int64)], axis=1)
    ghosts, inverse = (np.unique(keys, axis=0, return_inverse=True) if len(keys) else (np.zeros((0, 4), np.int64), np.zeros(0, np.int64)))
    G = len(ghosts)
    neigh_local = j.astype(np.int32).copy()
    neigh_local[is_img] = N + np.asarray(inverse).reshape(-1).astype(np.int32)
    owner = ghosts[:, 0].astype(np.int64)
    counts = (first[1:] - first[:-1]).astype(np.int64)
    g_edges = np.concatenate([np.arange(first[o], first[o + 1]) for o in owner]) if G else np.zeros(0, np.int64)
    return dict(
        num_local_nodes=N, num_ghost_nodes=G,
        node_types=np.concatenate([species_index, species_index[owner]]).astype(np.int32),
        num_neigh=np.concatenate([counts, counts[owner]]).astype(np.int32),
        neigh_indices=np.concatenate([neigh_local, np.zeros(len(g_edges), np.int32)]).astype(np.int32),
        neigh_types=np.concatenate([species_index[j], species_index[j[g_edges]]]).astype(np.int32),
        xyz=np.ascontiguousarray(np.concatenate([xyz, xyz[g_edges]])).reshape(-1),
        r=np.ascontiguousarray(np.concatenate([r, r[g_edges]])),
        sender_atom=np.concatenate([j, j[g_edges]]).astype(np.int32),
        receiver_atom=np.concatenate([np.arange(N), owner]).astype(np.int32),
        ghost_owner=owner.astype(np.int32),
    )


def image_shifts(cell, r_cut, pbc=(True, True, True)):
    """Integer cell shifts (lexicographic order) and their Cartesian vectors, as neighbor_list forms them."""
    cell = np.asarray(cell, dtype=np.float64)
    if cell.shape == (3,):
        cell = np.diag(cell)
    pbc = np.asarray(pbc, dtype=bool)
    vol = abs(np.linalg.det(cell))
    heights = np.array([vol / np.linalg.norm(np.cross(cell[(a + 1) % 3], cell[(a + 2) % 3])) for a in range(3)])
    nshell = np.where(pbc, np.ceil(r_cut / heights).astype(int), 0)
    ints, vecs = [], []
    for sx in range(-nshell[0], nshell[0] + 1):
        for sy in range(-nshell[1], nshell[1] + 1):
            for sz in range(-nshell[2], nshell[2] + 1):
                S = np.array([sx, sy, sz])
                ints.append(S)
                vecs.append(S.astype(np.float64) @ cell)
    return np.ascontiguousarray(ints, dtype=np.int32), np.ascontiguousarray(vecs, dtype=np.float64)


class DeviceNeighborList:
    """The same list built on the GPU from device-resident positions (smx_nlist_* of the C ABI).

    build() takes the address of a device array of positions ([N][3] float64) and, optionally, of species
    indices ([N] int32); the edge arrays stay on the device (addresses in .ptr) for MACE.compute_device, and
    to_host() returns them as the dict neighbor_list() / edge_arrays() would give.
    """

    def __init__(self):
        import ctypes as C
        from . import _lib
        self._C, self._lib = C, _lib
        self._L = _lib.lib()
        self._h = self._L.smx_nlist_create()
        if not self._h:
            raise RuntimeError("smx_nlist_create failed: " + self._L.smx_last_error().decode())
        self.num_atoms = 0
        self.num_edges = 0
        self.ptr = {}
        self._wrap = None      # lattice offsets taken off the positions of the last build_host
        self._cell = None

    @property
    def offsets(self):
        """Integer lattice offsets [N,3] that build_host took off the positions (None after build())."""
        return self._wrap

    def __del__(self):
        try:
            if self._h:
                self._L.smx_nlist_free(self._h)
        except Exception:
            pass

    _names = ("num_neigh", "first_neigh", "neigh_indices", "neigh_types", "neigh_shift", "xyz", "r")

    def _refresh(self, E):
        C = self._C
        self.num_edges = int(E)
        out = [C.c_void_p(0) for _ in self._names]
        self._lib.check(self._L.smx_nlist_arrays(C.c_void_p(self._h), *[C.byref(o) for o in out]))
        self.ptr = {n: (o.value or 0) for n, o in zip(self._names, out)}
        dp, dt = C.c_void_p(0), C.c_void_p(0)
        self._lib.check(self._L.smx_nlist_inputs(C.c_void_p(self._h), C.byref(dp), C.byref(dt)))
        self.ptr["positions"], self.ptr["node_types"] = dp.value or 0, dt.value or 0
        return self.num_edges

    def build(self, num_atoms, positions_ptr, types_ptr, cell, r_cut, pbc=(True, True, True), skin=0.0, stream=0):
        """New search: pairs within r_cut + skin are remembered, edges are the pairs within r_cut.

        The device positions are used as they are and must lie inside the cell along periodic axes (fold them with
        wrap_positions first, or use build_host): the shift table covers one cell span."""
        C = self._C
        self._wrap = None
        r_list = float(r_cut) + float(skin)
        ints, vecs = image_shifts(cell, r_list, pbc)
        E = C.c_long(0)
        self._lib.check(self._L.smx_nlist_build(
            C.c_void_p(self._h), int(num_atoms), C.c_void_p(positions_ptr), C.c_void_p(types_ptr or 0), len(ints),
            ints.ctypes.data_as(C.POINTER(C.c_int)), vecs.ctypes.data_as(C.POINTER(C.c_double)), C.c_double(r_list),
            C.c_double(r_cut), C.c_void_p(stream), C.byref(E)))
        self.num_atoms = int(num_atoms)
        return self._refresh(E.value)

    def build_host(self, positions, types, cell, r_cut, pbc=(True, True, True), skin=0.0):
        """build() from numpy positions [N][3] and species indices [N]; device copies are kept in the list object
        (addresses in .ptr["positions"], .ptr["node_types"])."""
        C = self._C
        # folded into the cell: the image shifts below cover one cell span (an update keeps these offsets, so
        # that the remembered pairs stay the same pairs)
        pos, self._wrap = wrap_positions(positions, cell, pbc)
        cellm = np.asarray(cell, dtype=np.float64)
        self._cell = np.diag(cellm) if cellm.shape == (3,) else cellm
        ty = np.ascontiguousarray(types, dtype=np.int32)
        if len(ty) != len(pos):
            raise ValueError("positions and types differ in length")
        r_list = float(r_cut) + float(skin)
        ints, vecs = image_shifts(cell, r_list, pbc)
        E = C.c_long(0)
        self._lib.check(self._L.smx_nlist_build_host(
            C.c_void_p(self._h), len(pos), pos.ctypes.data_as(C.POINTER(C.c_double)), ty.ctypes.data_as(C.POINTER(C.c_int)),
            len(ints), ints.ctypes.data_as(C.POINTER(C.c_int)), vecs.ctypes.data_as(C.POINTER(C.c_double)),
            C.c_double(r_list), C.c_double(r_cut), C.byref(E)))
        self.num_atoms = len(pos)
        return self._refresh(E.value)

    def update_host(self, positions, r_cut):
        """update() from numpy positions, with the species of the last build_host."""
        C = self._C
        pos = np.ascontiguousarray(positions, dtype=np.float64).reshape(-1, 3)
        if len(pos) != self.num_atoms:
            raise ValueError("the number of atoms differs from the last build")
        if self._wrap is not None and self._wrap.any():
            pos = pos - self._wrap.astype(np.float64) @ self._cell
        E = C.c_long(0)
        self._lib.check(self._L.smx_nlist_update_host(C.c_void_p(self._h), pos.ctypes.data_as(C.POINTER(C.c_double)),
                                                      C.c_double(r_cut), C.byref(E)))
        return self._refresh(E.value)

    def update(self, positions_ptr, types_ptr, r_cut, stream=0):
        """Edges within r_cut at new positions, from the pairs remembered by the last build (no new search)."""
        C = self._C
        E = C.c_long(0)
        self._lib.check(self._L.smx_nlist_update(C.c_void_p(self._h), C.c_void_p(positions_ptr), C.c_void_p(types_ptr or 0),
                                                 C.c_double(r_cut), C.c_void_p(stream), C.byref(E)))
        return self._refresh(E.value)

    def to_host(self):
        C = self._C
        N, E = self.num_atoms, self.num_edges
        nn = np.zeros(N, dtype=np.int32); ni = np.zeros(E, dtype=np.int32); nty = np.zeros(E, dtype=np.int32)
        S = np.zeros((E, 3), dtype=np.int32); xyz = np.zeros((E, 3)); r = np.zeros(E)
        p = lambda a, t: a.ctypes.data_as(C.POINTER(t))
        self._lib.check(self._L.smx_nlist_copy_to_host(C.c_void_p(self._h), p(nn, C.c_int), p(ni, C.c_int), p(nty, C.c_int),
                                                       p(S, C.c_int), p(xyz, C.c_double), p(r, C.c_double)))
        first = np.concatenate([[0], np.cumsum(nn)]).astype(np.int64)
        i = np.repeat(np.arange(N, dtype=np.int32), nn)
        if self._wrap is not None and self._wrap.any():
            S = (S + self._wrap[i] - self._wrap[ni]).astype(np.int32)
        return dict(i=i, j=ni, S=S, xyz=xyz, r=r, first_neigh=first,
                    num_neigh=nn, neigh_types=nty)
