"""Shared builders for the test-suite: tiny seeded models and systems."""
import json
import os

import numpy as np

from symmetrix_amd import modelgen, neighbors, systems


def tiny_model(K=4, L_max=1, T=(1, 6, 8), r_cut=4.0, n_pts=48, seed=3, pair=True, zbl=False, density=False):
    return modelgen.generate_model(list(T), K, L_max, r_cut, num_spline_points=n_pts, seed=seed,
                                   pair_dependent_radial=pair, zbl=zbl, density_normalisation=density)


def add_foreign_monomials(model, layers=(0, 1), seed=0):
    """One monomial from outside the standard product basis in every polynomial of the given layers (a term linear in
    a harmonic that cannot couple to the output: Y_1,-1 for scalar outputs, Y_00 for the others), with random
    coefficients.  Such a file is still a valid symmetrix model; its contraction takes the general kernel."""
    rng = np.random.default_rng(seed)
    if 0 in layers:
        for LM, monos in model["M0_monomials"].items():
            extra = [1] if int(LM) == 0 else [0]
            assert extra not in monos
            monos.append(extra)
            for a in model["M0_weights"]:
                for k in model["M0_weights"][a][LM]:
                    model["M0_weights"][a][LM][k].append(float(rng.normal() * 0.1))
    if 1 in layers:
        assert [1] not in model["M1_monomials"]
        model["M1_monomials"].append([1])
        for a in model["M1_weights"]:
            for k in model["M1_weights"][a]:
                model["M1_weights"][a][k].append(float(rng.normal() * 0.1))
    return model


def write_model(model, path):
    with open(path, "w") as f:
        json.dump(model, f)
    return str(path)


def small_system(n_atoms=12, density=0.08, probs=(0.4, 0.3, 0.3), seed=1):
    return systems.random_box(n_atoms, density, list(probs), seed=seed)


def edges_of(pos, cell, species, r_cut):
    nl = neighbors.neighbor_list(pos, cell, r_cut)
    return nl, neighbors.edge_arrays(nl, species)


def call_args(ea):
    return (ea["num_nodes"], ea["node_types"], ea["num_neigh"], ea["neigh_indices"], ea["neigh_types"],
            ea["xyz"], ea["r"])


def atom_forces(nl, f, n_atoms):
    """Per-edge -dE/dxyz -> per-atom forces, symmetrix_calc.py:93-97."""
    f = np.asarray(f).reshape(-1, 3)
    F = np.zeros((n_atoms, 3))
    np.add.at(F, nl["j"], f)
    np.add.at(F, nl["i"], -f)
    return F
