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


def neighbor_list(positions, cell, r_cut, pbc=(True, True, True)):
    """Full neighbour list of an orthorhombic or triclinic periodic cell.

    Returns dict with i, j (int32), S (int32 [E,3] cell shifts), xyz ([E,3] =
    x_j + S.cell - x_i), r ([E]), first_neigh ([N+1]) in canonical order.
    """
    pos = np.ascontiguousarray(positions, dtype=np.float64)
    cell = np.asarray(cell, dtype=np.float64)
    if cell.shape == (3,):
        cell = np.diag(cell)
    N = len(pos)
    pbc = np.asarray(pbc, dtype=bool)
    # number of image shells needed along each lattice vector
    vol = abs(np.linalg.det(cell))
    heights = np.array([vol / np.linalg.norm(np.cross(cell[(a + 1) % 3], cell[(a + 2) % 3])) for a in range(3)])
    nshell = np.where(pbc, np.ceil(r_cut / heights).astype(int), 0)
    inv = np.linalg.inv(cell)
    frac = pos @ inv
    lo_f = frac.min(axis=0) if N else np.zeros(3)
    hi_f = frac.max(axis=0) if N else np.zeros(3)
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
                            rows.append((i, j, sx, sy, sz, d[0], d[1], d[2], np.sqrt(r2)))
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
