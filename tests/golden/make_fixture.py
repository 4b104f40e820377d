"""Writes tests/golden/tiny_model.json and tests/golden/tiny_case.npz.

A tiny seeded model (2 species, 4 channels, L_max = 1, 16 spline knots) and a
6-atom periodic cell, with every intermediate of the CPU oracle for that
input.  The vectors are produced by this repository's own oracle
(oracle/mace_oracle.c), not by the reference: they freeze the oracle's answers
so that later edits to it, to the generator or to the GPU engine are caught.
Run from the repository root:  python tests/golden/make_fixture.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle.oracle import OracleMACE  # noqa: E402
from symmetrix_amd import modelgen, neighbors  # noqa: E402

NAMES = ["Y", "Y_grad", "R0", "R1", "A0", "M0", "H1", "Phi1", "A1", "M1", "H2", "H2_adj", "M1_adj", "A1_adj",
         "Phi1_adj", "H1_adj", "M0_adj", "A0_adj", "node_energies", "node_forces"]


def main():
    model = modelgen.generate_model([1, 8], 4, 1, 3.5, num_spline_points=16, seed=11)
    # round-trip through text so that the committed file is exactly what is loaded
    text = json.dumps(model)
    with open(os.path.join(HERE, "tiny_model.json"), "w") as f:
        f.write(text)
    rng = np.random.default_rng(5)
    cell = np.array([4.2, 4.6, 5.0])
    pos = rng.uniform(0, 1, size=(6, 3)) * cell
    species = np.array([0, 1, 0, 0, 1, 0], dtype=np.int32)
    nl = neighbors.neighbor_list(pos, cell, model["r_cut"])
    ea = neighbors.edge_arrays(nl, species)
    orc = OracleMACE(json.loads(text))
    orc.compute_node_energies_forces(ea["num_nodes"], ea["node_types"], ea["num_neigh"], ea["neigh_indices"],
                                     ea["neigh_types"], ea["xyz"], ea["r"])
    out = {n: getattr(orc, n) for n in NAMES}
    np.savez_compressed(os.path.join(HERE, "tiny_case.npz"), positions=pos, cell=cell, species=species,
                        i=nl["i"], j=nl["j"], S=nl["S"], node_types=ea["node_types"], num_neigh=ea["num_neigh"],
                        neigh_indices=ea["neigh_indices"], neigh_types=ea["neigh_types"], xyz=ea["xyz"], r=ea["r"],
                        **out)
    print("edges", len(ea["r"]), "E", out["node_energies"].sum())


if __name__ == "__main__":
    main()
