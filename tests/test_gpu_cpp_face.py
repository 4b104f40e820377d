"""The C++ face of the engine driven by a compiled C++20 caller (GPU).

tests/cpp/pair_modes_driver is built by g++ against include/symmetrix_amd/mace.hpp,
pair_symmetrix_amd/mace_evaluation.cpp and libsymmetrix_amd.so (`make -C tests/cpp`, part of
__graft_entry__.build()).  It runs what the reference pair style does between its "begin mace evaluation"
and "end mace evaluation" marks in its three modes (pair_symmetrix/pair_symmetrix_mace.cpp:319-320,
444-495, 660-698) plus the force scatter, on one rank, where periodic images play the ghosts
(the reference's own way of testing the modes, pair_symmetrix/test/test_pair_symmetrix_mace.py:28-39).
"""
import os
import subprocess

import numpy as np
import pytest

from oracle.oracle import OracleMACE
from symmetrix_amd import neighbors
from tests import helpers as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "tests", "cpp", "pair_modes_driver")


def _case(f, mode, Nl, Ng, rows, nt, nn, node_i, ni, nty, nj, halo_ghost, halo_owner, xyz, r):
    E = len(r)
    np.array([mode, Nl, Ng, E, rows, len(halo_ghost)], dtype=np.int64).tofile(f)
    for a in (nt, nn, node_i, ni, nty, nj, halo_ghost, halo_owner):
        np.ascontiguousarray(a, dtype=np.int32).tofile(f)
    np.ascontiguousarray(xyz, dtype=np.float64).tofile(f)
    np.ascontiguousarray(r, dtype=np.float64).tofile(f)


@pytest.mark.gpu
@pytest.mark.parametrize("L_max,dtype,one_table,density", [(0, "float64", False, False), (1, "float64", False, True),
                                                            (1, "float32", False, True), (0, "float64", True, False),
                                                            (0, "float32", True, True)])
def test_cpp_caller_runs_the_three_pair_style_modes(tmp_path, L_max, dtype, one_table, density):
    """`one_table`: one radial table for all species pairs, so that the channel-slice kernels run (the layer-1
    partial forces wait for the layer-0 adjoint there, beside the ZBL and density-normalisation forces)."""
    if not os.path.exists(DRIVER):
        pytest.fail("tests/cpp/pair_modes_driver is not built: python -c 'import __graft_entry__ as g; g.build()'")
    model = H.tiny_model(K=16, L_max=L_max, n_pts=48, seed=12, pair=not one_table, zbl=True, density=density)
    path = H.write_model(model, tmp_path / "m.json")
    pos, cell, sp = H.small_system(36, seed=21)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    N = len(sp)
    ga = neighbors.ghost_edge_arrays(nl, sp)
    Nl, Ng = ga["num_local_nodes"], ga["num_ghost_nodes"]
    El = int(ga["num_neigh"][:Nl].sum())
    ghost_rows = np.arange(Nl, Nl + Ng)
    none = np.zeros(0, np.int32)
    case = tmp_path / "case.bin"
    with open(case, "wb") as f:
        np.array([4], dtype=np.int64).tofile(f)
        # 1: owners as senders
        _case(f, 1, N, 0, N, ea["node_types"], ea["num_neigh"], np.arange(N), ea["neigh_indices"], ea["neigh_types"],
              ea["neigh_indices"], none, none, ea["xyz"], ea["r"])
        # 2: local nodes; senders are atom rows (local + ghost), ghost rows filled by the forward exchange
        _case(f, 2, Nl, 0, Nl + Ng, ga["node_types"][:Nl], ga["num_neigh"][:Nl], np.arange(Nl), ga["neigh_indices"][:El],
              ga["neigh_types"][:El], ga["neigh_indices"][:El], ghost_rows, ga["ghost_owner"], ga["xyz"][:3 * El], ga["r"][:El])
        # 3 and 4: ghost nodes after the local ones; forces land on the owners
        for mode in (3, 4):
            _case(f, mode, Nl, Ng, N, ga["node_types"], ga["num_neigh"], ga["receiver_atom"], ga["neigh_indices"],
                  ga["neigh_types"], ga["sender_atom"], none, none, ga["xyz"], ga["r"])
    out = tmp_path / "out.bin"
    print(f"driver: {Nl} local + {Ng} ghost nodes, L_max {L_max}, {dtype}", flush=True)
    res = subprocess.run([DRIVER, path, "0" if dtype == "float64" else "1", str(case), str(out)], capture_output=True,
                         text=True, timeout=100)
    print(res.stdout, res.stderr, flush=True)
    assert res.returncode == 0, res.stderr
    raw = np.fromfile(out, dtype=np.float64)
    results, o = [], 0
    for rows in (N, Nl + Ng, N, N):
        etot = raw[o]; en = raw[o + 1:o + 1 + Nl]; o += 1 + Nl
        F = raw[o:o + 3 * rows].reshape(rows, 3).copy(); o += 3 * rows
        vir = raw[o:o + 6]; o += 6
        if rows > N:                      # ghost rows' forces go to their owners (LAMMPS reverse communication)
            np.add.at(F, ga["ghost_owner"], F[N:])
            F = F[:N]
        results.append((etot, en, F, vir))
    assert o == len(raw)
    orc = OracleMACE(model)
    orc.compute_node_energies_forces(*H.call_args(ea))
    e_ref = orc.node_energies
    f_ref = H.atom_forces(nl, orc.node_forces, N)
    fe = orc.node_forces.reshape(-1, 3); d = ea["xyz"].reshape(-1, 3)
    v_ref = np.array([(d[:, 0] * fe[:, 0]).sum(), (d[:, 1] * fe[:, 1]).sum(), (d[:, 2] * fe[:, 2]).sum(),
                      0.5 * (d[:, 0] * fe[:, 1] + d[:, 1] * fe[:, 0]).sum(), 0.5 * (d[:, 0] * fe[:, 2] + d[:, 2] * fe[:, 0]).sum(),
                      0.5 * (d[:, 1] * fe[:, 2] + d[:, 2] * fe[:, 1]).sum()])
    etol, ftol, vtol = (1e-10, 1e-8, 1e-9) if dtype == "float64" else (1e-5, 1e-4, 1e-4)   # the bar of the parity tests
    vscale = max(1.0, np.abs(v_ref).max())
    for name, (etot, en, F, vir) in zip(("no_domain_decomposition", "mpi_message_passing", "no_mpi_message_passing",
                                         "no_mpi_message_passing (stage calls)"), results):
        assert abs(etot - e_ref.sum()) <= etol * abs(e_ref.sum()), name
        assert np.abs(en - e_ref).max() <= etol * np.abs(e_ref).max(), name
        assert np.abs(F - f_ref).max() <= ftol, name
        # a ghost node's edges are copies of its owner's edge vectors, so the sum over all copies is the same virial
        assert np.abs(vir - v_ref).max() <= vtol * vscale, name
