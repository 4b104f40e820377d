"""Seeded synthetic atomic systems for the benchmark/parity configurations.

Each builder returns (positions[N,3], cell[3], species_index[N]) where
species_index refers to the sorted species list of the matching model
configuration in `modelgen.CONFIGS`.  Everything is numpy `default_rng(seed)`.
"""
from __future__ import annotations

import numpy as np


def random_box(n_atoms, density, probs, min_dist=0.9, seed=0):
    """Cubic periodic box, uniform positions with sequential rejection at a
    minimum-image pair distance `min_dist`, species drawn with `probs`."""
    rng = np.random.default_rng(seed)
    L = (n_atoms / density) ** (1.0 / 3.0)
    nb = max(1, int(L / min_dist))
    bs = L / nb
    grid = {}
    pos = np.zeros((n_atoms, 3))
    n = 0
    md2 = min_dist * min_dist
    while n < n_atoms:
        cand = rng.uniform(0.0, L, size=(max(64, n_atoms - n), 3))
        for p in cand:
            b = tuple(np.minimum((p / bs).astype(int), nb - 1))
            ok = True
            for dx in (-1, 0, 1):
                for dy in (-1, 0, 1):
                    for dz in (-1, 0, 1):
                        key = ((b[0] + dx) % nb, (b[1] + dy) % nb, (b[2] + dz) % nb)
                        for q in grid.get(key, ()):
                            d = pos[q] - p
                            d -= L * np.round(d / L)
                            if d @ d < md2:
                                ok = False
                                break
                        if not ok:
                            break
                    if not ok:
                        break
                if not ok:
                    break
            if ok:
                pos[n] = p
                grid.setdefault(b, []).append(n)
                n += 1
                if n == n_atoms:
                    break
    species = rng.choice(len(probs), size=n_atoms, p=np.asarray(probs, dtype=np.float64))
    return pos, np.array([L, L, L]), species.astype(np.int32)


def water_box(n_molecules, density=0.033, oh=0.96, jitter=0.05, seed=0, species_O=3, species_H=0):
    """Water-like box: O uniform at `density` molecules/A^3, two H at `oh` from
    their O in random directions, Gaussian jitter on everything."""
    rng = np.random.default_rng(seed)
    L = (n_molecules / density) ** (1.0 / 3.0)
    O = rng.uniform(0.0, L, size=(n_molecules, 3))
    def rand_dirs(n):
        v = rng.normal(size=(n, 3))
        return v / np.linalg.norm(v, axis=1, keepdims=True)
    H1 = O + oh * rand_dirs(n_molecules)
    H2 = O + oh * rand_dirs(n_molecules)
    pos = np.concatenate([O, H1, H2]) + rng.normal(scale=jitter, size=(3 * n_molecules, 3))
    pos %= L
    species = np.concatenate([np.full(n_molecules, species_O), np.full(2 * n_molecules, species_H)])
    return pos, np.array([L, L, L]), species.astype(np.int32)


def fcc_alloy(reps, a=3.6, n_species=5, sigma=0.1, seed=0):
    """Perturbed fcc lattice, species uniform over n_species."""
    rng = np.random.default_rng(seed)
    basis = np.array([[0, 0, 0], [0.5, 0.5, 0], [0.5, 0, 0.5], [0, 0.5, 0.5]]) * a
    gx, gy, gz = np.meshgrid(np.arange(reps[0]), np.arange(reps[1]), np.arange(reps[2]), indexing="ij")
    origins = np.stack([gx, gy, gz], axis=-1).reshape(-1, 3) * a
    pos = (origins[:, None, :] + basis[None, :, :]).reshape(-1, 3)
    pos = pos + rng.normal(scale=sigma, size=pos.shape)
    cell = np.array(reps, dtype=np.float64) * a
    pos %= cell
    species = rng.integers(0, n_species, size=len(pos))
    return pos, cell, species.astype(np.int32)


def config_system(name, seed=0, scale=1.0):
    """Systems named by the benchmark description; `scale` shrinks atom counts
    for tests (same density and recipe)."""
    if name == "tiny":            # 192 atoms, H/C/O uniform
        return random_box(max(8, int(192 * scale)), 0.10, [1 / 3, 1 / 3, 1 / 3], seed=seed)
    if name == "off_small":       # 3000 atoms, H/C/N/O 0.5/0.3/0.1/0.1
        return random_box(max(8, int(3000 * scale)), 0.10, [0.5, 0.3, 0.1, 0.1], seed=seed)
    if name in ("off_medium", "off_medium_l2"):      # 25 002 atoms water-like (8334 molecules)
        return water_box(max(4, int(8334 * scale)), seed=seed)
    if name == "mp_medium":       # 25 x 25 x 20 fcc cells = 50 000 atoms
        s = scale ** (1.0 / 3.0)
        reps = (max(2, round(25 * s)), max(2, round(25 * s)), max(2, round(20 * s)))
        return fcc_alloy(reps, seed=seed)
    raise KeyError(name)
