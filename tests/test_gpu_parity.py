"""GPU parity tests proper (run on an MI355X with -m gpu).

Every check goes through the C ABI (symmetrix_amd.mace.MACE is a ctypes face of
include/symmetrix_amd.h) and compares the HIP engine with the CPU oracle on the
same seeded inputs.  Tolerances are the ones the task states:
  fp64 mode           energy rel <= 1e-10, forces max-abs <= 1e-8 eV/A
  fp32-feature mode   energy rel <= 1e-5,  forces max-abs <= 1e-4 eV/A
"""
import json
import os

import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
TOL = {"float64": dict(E=1e-10, F=1e-8, inter=1e-11), "float32": dict(E=1e-5, F=1e-4, inter=2e-5)}
INTERMEDIATES = ["Y", "Y_grad", "R0", "R1", "A0", "M0", "H1", "Phi1", "A1", "M1", "H2", "H2_adj", "M1_adj",
                 "A1_adj", "Phi1_adj", "H1_adj", "M0_adj", "A0_adj", "M1_grad", "M0_grad"]
# (M0_grad last: with several polynomials per channel an evaluation keeps no layer-0 gradients, the adjoint forms
# them again from A0; asking for the array evaluates them from the A0 the evaluation left)


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    from symmetrix_amd.mace import MACE
    return MACE


def _oracle():
    from oracle.oracle import OracleMACE
    return OracleMACE


def _compare(orc, eng, dtype, names=INTERMEDIATES):
    tol = TOL[dtype]
    for name in names:
        a = getattr(orc, name); b = getattr(eng, name)
        assert a.shape == b.shape, name
        scale = max(1.0, np.abs(a).max()) if len(a) else 1.0
        assert np.abs(a - b).max(initial=0.0) <= tol["inter"] * scale * 10, name
    Eo, Eg = orc.node_energies.sum(), eng.node_energies.sum()
    assert abs(Eo - Eg) <= tol["E"] * abs(Eo)
    assert np.abs(orc.node_energies - eng.node_energies).max() <= tol["E"] * max(1.0, np.abs(orc.node_energies).max()) * 10
    assert np.abs(orc.node_forces - eng.node_forces).max(initial=0.0) <= tol["F"]


CASES = [
    # K, L_max, atoms, pair-dependent radial
    (32, 0, 40, True), (32, 1, 40, True), (96, 0, 48, False), (128, 1, 36, True), (48, 1, 24, True),
    (20, 0, 17, True), (64, 1, 30, False), (128, 0, 30, True),
    # wider than one block of channels: several channel groups, column tiles and slices
    (256, 0, 20, False), (192, 1, 16, False),
    # hidden features up to l = 2 (128x0e+128x1o+128x2e and the like): 17 paths, 9 polynomials
    (16, 2, 30, True), (128, 2, 20, False), (40, 2, 26, True),
]


@pytest.mark.parametrize("dtype", ["float64", "float32"])
@pytest.mark.parametrize("K,L_max,natoms,pair", CASES)
def test_pipeline_matches_oracle(gpu, tmp_models, K, L_max, natoms, pair, dtype):
    model = H.tiny_model(K=K, L_max=L_max, n_pts=64, seed=K + L_max, pair=pair)
    path = H.write_model(model, tmp_models / f"m_{K}_{L_max}_{int(pair)}.json")
    orc = _oracle()(model)
    eng = gpu(path, dtype)
    pos, cell, sp = H.small_system(natoms, seed=natoms)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    print(f"case K={K} L_max={L_max} atoms={natoms} edges={len(ea['r'])} {dtype}", flush=True)
    orc.compute_node_energies_forces(*H.call_args(ea))
    eng.compute_node_energies_forces(*H.call_args(ea))
    _compare(orc, eng, dtype)
    # bit-reproducible: no atomics on floats anywhere
    f1, e1 = eng.node_forces, eng.node_energies
    eng.compute_node_energies_forces(*H.call_args(ea))
    assert np.array_equal(f1, eng.node_forces) and np.array_equal(e1, eng.node_energies)
    # caller-side reduction, symmetrix_calc.py:93-102 / pair_symmetrix_mace.cpp:334-368
    F, V = eng.reduce_forces(len(pos), nl["j"], virial=True)
    assert np.allclose(F, H.atom_forces(nl, orc.node_forces, len(pos)), atol=TOL[dtype]["F"] * 10)
    f = orc.node_forces.reshape(-1, 3); x = ea["xyz"].reshape(-1, 3)
    W = x.T @ f
    Vref = np.array([W[0, 0], W[1, 1], W[2, 2], 0.5 * (W[0, 1] + W[1, 0]), 0.5 * (W[0, 2] + W[2, 0]), 0.5 * (W[1, 2] + W[2, 1])])
    assert np.allclose(V, Vref, atol=TOL[dtype]["F"] * 100)


@pytest.mark.parametrize("dtype", ["float64", "float32"])
@pytest.mark.parametrize("K,L_max,natoms,layers", [(32, 0, 40, (0, 1)), (33, 1, 25, (0, 1)), (96, 0, 48, (1,)),
                                                   (20, 1, 30, (0,)), (16, 2, 22, (0, 1)), (128, 1, 20, (0, 1))])
def test_monomials_outside_the_standard_basis_take_the_general_kernel(gpu, tmp_models, K, L_max, natoms, layers, dtype):
    """The symmetric contraction has a kernel compiled for the monomial lists of the standard product basis (every
    other model in this file runs it) and a general one that walks whatever lists the file holds.  Files with one
    more monomial in the polynomials of layer 0, of layer 1 or of both: the loader must send exactly those layers to
    the general kernel, and all intermediates, energies and forces must still match the oracle."""
    model = H.add_foreign_monomials(H.tiny_model(K=K, L_max=L_max, n_pts=64, seed=K + L_max, pair=False), layers, seed=K)
    path = H.write_model(model, tmp_models / f"foreign_{K}_{L_max}_{len(layers)}_{layers[0]}.json")
    orc = _oracle()(model)
    eng = gpu(path, dtype)
    assert eng._int("contraction_tables") == 3 - sum(1 << l for l in layers)
    pos, cell, sp = H.small_system(natoms, seed=natoms)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    print(f"case K={K} L_max={L_max} atoms={natoms} edges={len(ea['r'])} foreign monomials in layers {layers} {dtype}", flush=True)
    orc.compute_node_energies_forces(*H.call_args(ea))
    eng.compute_node_energies_forces(*H.call_args(ea))
    _compare(orc, eng, dtype)


@pytest.mark.parametrize("dtype", ["float64", "float32"])
@pytest.mark.parametrize("K,natoms", [(20, 70), (96, 200), (33, 9)])
def test_two_species_three_radial_tables(gpu, tmp_models, K, natoms, dtype):
    """Scalar hidden features with a few distinct pair tables: the general edge kernels
    (the channel-slice kernels hold one table)."""
    model = H.tiny_model(K=K, L_max=0, T=(1, 8), n_pts=50, seed=K, pair=True)
    path = H.write_model(model, tmp_models / f"two_{K}.json")
    orc = _oracle()(model)
    eng = gpu(path, dtype)
    pos, cell, sp = H.small_system(natoms, probs=(0.6, 0.4), seed=natoms)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    print(f"case K={K} atoms={natoms} edges={len(ea['r'])} {dtype}", flush=True)
    orc.compute_node_energies_forces(*H.call_args(ea))
    eng.compute_node_energies_forces(*H.call_args(ea))
    _compare(orc, eng, dtype)


@pytest.mark.parametrize("dtype", ["float64", "float32"])
@pytest.mark.parametrize("K,natoms", [(24, 60), (7, 33)])
def test_long_spline_tables_take_the_narrow_slice_kernels(gpu, tmp_models, K, natoms, dtype):
    """One radial table with 400 nodes: a slice of 32 bytes of channels no longer fits the LDS, so the slices
    are half as wide and the four-lanes-per-edge kernels of both directions run instead of the 32-byte ones."""
    model = H.tiny_model(K=K, L_max=0, n_pts=400, seed=K, pair=False)
    path = H.write_model(model, tmp_models / f"long_{K}.json")
    orc = _oracle()(model)
    eng = gpu(path, dtype)
    pos, cell, sp = H.small_system(natoms, seed=natoms)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    print(f"case K={K} atoms={natoms} edges={len(ea['r'])} {dtype} 400 spline nodes", flush=True)
    orc.compute_node_energies_forces(*H.call_args(ea))
    eng.compute_node_energies_forces(*H.call_args(ea))
    _compare(orc, eng, dtype)
    f1, e1 = eng.node_forces, eng.node_energies
    eng.compute_node_energies_forces(*H.call_args(ea))
    assert np.array_equal(f1, eng.node_forces) and np.array_equal(e1, eng.node_energies)


@pytest.mark.parametrize("dtype", ["float64", "float32"])
@pytest.mark.parametrize("K,natoms", [(6, 41), (7, 33), (20, 52)])
def test_channel_counts_that_leave_the_last_slice_incomplete(gpu, tmp_models, K, natoms, dtype):
    """One radial table that fits the LDS in 32-byte slices (4 doubles or 8 floats of channels), scalar hidden
    features, and a channel count that is no multiple of the slice: the last slice of the 32-byte kernels of both
    directions has channels missing (K = 20 only in single precision), which they handle by element-wise loads and
    stores compiled apart from the whole-slice code."""
    model = H.tiny_model(K=K, L_max=0, n_pts=64, seed=100 + K, pair=False)
    path = H.write_model(model, tmp_models / f"partial_{K}.json")
    orc = _oracle()(model)
    eng = gpu(path, dtype)
    pos, cell, sp = H.small_system(natoms, seed=natoms)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    print(f"case K={K} atoms={natoms} edges={len(ea['r'])} {dtype} incomplete last slice", flush=True)
    orc.compute_node_energies_forces(*H.call_args(ea))
    eng.compute_node_energies_forces(*H.call_args(ea))
    _compare(orc, eng, dtype)
    f1, e1 = eng.node_forces, eng.node_energies
    eng.compute_node_energies_forces(*H.call_args(ea))
    assert np.array_equal(f1, eng.node_forces) and np.array_equal(e1, eng.node_energies)


@pytest.mark.parametrize("dtype", ["float64", "float32"])
def test_golden_fixture(gpu, dtype):
    z = np.load(os.path.join(GOLD, "tiny_case.npz"))
    eng = gpu(os.path.join(GOLD, "tiny_model.json"), dtype)
    eng.compute_node_energies_forces(len(z["node_types"]), z["node_types"], z["num_neigh"], z["neigh_indices"],
                                     z["neigh_types"], z["xyz"], z["r"])
    tol = TOL[dtype]
    E = z["node_energies"].sum()
    assert abs(eng.node_energies.sum() - E) <= tol["E"] * abs(E)
    assert np.abs(eng.node_forces - z["node_forces"]).max() <= tol["F"]
    for name in ("A0", "M0", "H1", "Phi1", "A1", "M1", "H2", "H1_adj", "A0_adj"):
        assert np.abs(getattr(eng, name) - z[name]).max() <= tol["inter"] * 10 * max(1.0, np.abs(z[name]).max()), name


@pytest.mark.parametrize("dtype", ["float64", "float32"])
@pytest.mark.parametrize("K,L_max,natoms,zbl,density", [(32, 0, 40, True, False), (96, 0, 48, True, True),
                                                        (48, 1, 30, True, True), (128, 1, 24, False, True),
                                                        (32, 2, 22, True, True)])
def test_pair_terms_match_oracle(gpu, tmp_models, K, L_max, natoms, zbl, density, dtype):
    """Models with ZBL repulsion and / or density-normalised layers (mace.cpp:27-35, 273-346, 681-757)."""
    model = H.tiny_model(K=K, L_max=L_max, n_pts=64, seed=K + L_max, pair=(K != 96), zbl=zbl, density=density)
    path = H.write_model(model, tmp_models / f"p_{K}_{L_max}_{int(zbl)}{int(density)}.json")
    orc = _oracle()(model)
    eng = gpu(path, dtype)
    pos, cell, sp = H.small_system(natoms, seed=natoms + 1)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    print(f"case K={K} L_max={L_max} atoms={natoms} zbl={zbl} density={density} {dtype}", flush=True)
    orc.compute_node_energies_forces(*H.call_args(ea))
    eng.compute_node_energies_forces(*H.call_args(ea))
    _compare(orc, eng, dtype)
    f1, e1 = eng.node_forces, eng.node_energies
    eng.compute_node_energies_forces(*H.call_args(ea))
    assert np.array_equal(f1, eng.node_forces) and np.array_equal(e1, eng.node_energies)


def test_density_normalisation_stage_calls(gpu, tmp_models):
    """compute_A0_scaled / reverse_A0_scaled and their layer-1 twins called stage by stage, as test_mace.py does."""
    model = H.tiny_model(K=8, L_max=1, n_pts=40, seed=9, density=True)
    path = H.write_model(model, tmp_models / "stage_scaled.json")
    orc = _oracle()(model)
    eng = gpu(path)
    pos, cell, sp = H.small_system(10, seed=3)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    N, nt, nn, ni, nty, xyz, r = H.call_args(ea)
    rng = np.random.default_rng(1)
    for m in (orc, eng):
        m.compute_Y(xyz); m.compute_R0(N, nt, nn, nty, r); m.compute_A0(N, nt, nn, nty)
        m.compute_A0_scaled(N, nt, nn, nty, r)
    assert np.allclose(orc.A0, eng.A0, atol=1e-12)
    adj = rng.normal(size=len(orc.A0))
    for m in (orc, eng):
        m.A0_adj = adj
        m.node_forces = np.zeros(len(xyz))
        m.reverse_A0_scaled(N, nt, nn, nty, xyz, r)
    assert np.allclose(orc.A0_adj, eng.A0_adj, atol=1e-12)
    assert np.allclose(orc.node_forces, eng.node_forces, atol=1e-11)
    A1 = rng.normal(size=N * 16 * 8)
    for m in (orc, eng):
        m.A1 = A1
        m.compute_A1_scaled(N, nt, nn, nty, r)
        m.A1_adj = adj[:len(A1)]
        m.reverse_A1_scaled(N, nt, nn, nty, xyz, r, True)
    assert np.allclose(orc.A1, eng.A1, atol=1e-12) and np.allclose(orc.A1_adj, eng.A1_adj, atol=1e-12)
    assert np.allclose(orc.node_forces, eng.node_forces, atol=1e-11)


def test_stage_level_calls_follow_the_reference_test_method(gpu, tmp_models):
    """symmetrix/test/test_mace.py drives the evaluator stage by stage and overwrites
    intermediates between calls (e.g. :246-249).  Same here, against the oracle."""
    model = H.tiny_model(K=8, L_max=1, n_pts=40, seed=9)
    path = H.write_model(model, tmp_models / "stage.json")
    orc = _oracle()(model)
    eng = gpu(path)
    pos, cell, sp = H.small_system(10, seed=3)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    N, nt, nn, ni, nty, xyz, r = H.call_args(ea)
    rng = np.random.default_rng(0)
    for m in (orc, eng):
        m.compute_Y(xyz)
        m.compute_R0(N, nt, nn, nty, r)
        m.compute_A0(N, nt, nn, nty)
    assert np.allclose(orc.A0, eng.A0, atol=1e-12)
    assert np.allclose(orc.R0, eng.R0, atol=1e-12) and np.allclose(orc.Y, eng.Y, atol=1e-13)
    A0 = rng.normal(size=len(orc.A0))
    for m in (orc, eng):
        m.A0 = A0
        m.compute_M0(N, nt)
        m.M0_adj = np.ones(len(m.M0))
        m.reverse_M0(N, nt)
    assert np.allclose(orc.M0, eng.M0, atol=1e-11) and np.allclose(orc.A0_adj, eng.A0_adj, atol=1e-10)
    for m in (orc, eng):
        m.compute_H1(N)
        m.H1_adj = np.ones(len(m.H1))
        m.reverse_H1(N)
    assert np.allclose(orc.H1, eng.H1, atol=1e-11) and np.allclose(orc.M0_adj, eng.M0_adj, atol=1e-11)
    for m in (orc, eng):
        m.compute_R1(N, nt, nn, nty, r)
        m.compute_Phi1(N, nn, ni)
        m.Phi1_adj = np.ones(len(m.Phi1))
        m.reverse_Phi1(N, nn, ni, xyz, r, True, True)
    assert np.allclose(orc.Phi1, eng.Phi1, atol=1e-11)
    assert np.allclose(orc.node_forces, eng.node_forces, atol=1e-10)
    assert np.allclose(orc.H1_adj, eng.H1_adj, atol=1e-10)
    for m in (orc, eng):
        m.compute_A1(N)
        m.A1_adj = np.ones(len(m.A1))
        m.reverse_A1(N)
    assert np.allclose(orc.A1, eng.A1, atol=1e-12) and np.allclose(orc.Phi1_adj, eng.Phi1_adj, atol=1e-12)
    for m in (orc, eng):
        m.compute_M1(N, nt)
        m.M1_adj = np.ones(len(m.M1))
        m.reverse_M1(N, nt)
    assert np.allclose(orc.M1, eng.M1, atol=1e-12) and np.allclose(orc.A1_adj, eng.A1_adj, atol=1e-11)
    for m in (orc, eng):
        m.compute_H2(N, nt)
        m.H2_adj = np.ones(len(m.H2))
        m.reverse_H2(N, nt, True)
    assert np.allclose(orc.H2, eng.H2, atol=1e-12)
    assert np.allclose(orc.M1_adj, eng.M1_adj, atol=1e-12) and np.allclose(orc.H1_adj, eng.H1_adj, atol=1e-12)
    for m in (orc, eng):
        m.node_energies = np.zeros(N)
        m.compute_readouts(N, nt)
    assert np.allclose(orc.node_energies, eng.node_energies, atol=1e-12)
    assert np.allclose(orc.H2_adj, eng.H2_adj, atol=1e-12) and np.allclose(orc.H1_adj, eng.H1_adj, atol=1e-13)
    # reverse_A0 accumulates into node_forces (mace.cpp:237)
    for m in (orc, eng):
        m.A0_adj = np.ones(len(m.A0))
        m.node_forces = np.zeros(len(xyz))
        m.reverse_A0(N, nt, nn, nty, xyz, r)
    assert np.allclose(orc.node_forces, eng.node_forces, atol=1e-10)


def test_edge_cases(gpu, tmp_models):
    model = H.tiny_model(K=8, L_max=0, n_pts=32, seed=2)
    path = H.write_model(model, tmp_models / "edge.json")
    orc = _oracle()(model)
    eng = gpu(path)
    # no nodes at all
    eng.compute_node_energies_forces(0, [], [], [], [], [], [])
    assert len(eng.node_energies) == 0 and len(eng.node_forces) == 0
    # isolated atoms only: E_i = E0[type]
    eng.compute_node_energies_forces(3, [0, 2, 1], [0, 0, 0], [], [], [], [])
    assert np.allclose(eng.node_energies, np.array(model["atomic_energies"])[[0, 2, 1]], atol=1e-14)
    # ragged degrees, including zero-degree receivers in the middle
    rng = np.random.default_rng(4)
    nn = np.array([3, 0, 5, 1, 0, 2], dtype=np.int32)
    E = int(nn.sum())
    nt = rng.integers(0, 3, size=6).astype(np.int32)
    ni = rng.integers(0, 6, size=E).astype(np.int32)
    nty = nt[ni]
    xyz = rng.normal(size=(E, 3)); xyz *= (rng.uniform(0.8, 3.9, size=(E, 1)) / np.linalg.norm(xyz, axis=1, keepdims=True))
    r = np.linalg.norm(xyz, axis=1)
    args = (6, nt, nn, ni, nty, xyz.reshape(-1), r)
    orc.compute_node_energies_forces(*args); eng.compute_node_energies_forces(*args)
    _compare(orc, eng, "float64")
    # a receiver with more edges than one LDS chunk, several times over
    nn = np.array([70, 1], dtype=np.int32); E = 71
    ni = rng.integers(0, 2, size=E).astype(np.int32); nt = np.array([0, 1], dtype=np.int32); nty = nt[ni]
    xyz = rng.normal(size=(E, 3)); xyz *= (rng.uniform(0.8, 3.9, size=(E, 1)) / np.linalg.norm(xyz, axis=1, keepdims=True))
    args = (2, nt, nn, ni, nty, xyz.reshape(-1), np.linalg.norm(xyz, axis=1))
    orc.compute_node_energies_forces(*args); eng.compute_node_energies_forces(*args)
    _compare(orc, eng, "float64")


def test_invalid_inputs_raise(gpu, tmp_models):
    model = H.tiny_model(K=8, L_max=0, n_pts=32, seed=2)
    eng = gpu(H.write_model(model, tmp_models / "inv.json"))
    xyz = np.array([[1.0, 0, 0], [-1.0, 0, 0]]).reshape(-1)
    ok = (2, [0, 1], [1, 1], [1, 0], [1, 0], xyz, [1.0, 1.0])
    eng.compute_node_energies_forces(*ok)
    with pytest.raises(ValueError):      # beyond the spline table (cubic_spline_set.cpp:54 would read past it)
        eng.compute_node_energies_forces(2, [0, 1], [1, 1], [1, 0], [1, 0], xyz * 5, [5.0, 5.0])
    with pytest.raises(ValueError):      # species index outside the model
        eng.compute_node_energies_forces(2, [0, 7], [1, 1], [1, 0], [1, 0], xyz, [1.0, 1.0])
    with pytest.raises(ValueError):      # sender outside the node range
        eng.compute_node_energies_forces(2, [0, 1], [1, 1], [5, 0], [1, 0], xyz, [1.0, 1.0])
    with pytest.raises(ValueError):      # counts do not add up
        eng.compute_node_energies_forces(2, [0, 1], [2, 1], [1, 0], [1, 0], xyz, [1.0, 1.0])
    eng.compute_node_energies_forces(*ok)   # still usable afterwards


@pytest.mark.parametrize("workload", ["off_small", "mp_medium"])
def test_full_size_properties(gpu, tmp_models, workload):
    """At the benchmark's full size: properties that do not need the oracle."""
    from symmetrix_amd import modelgen, neighbors, systems
    cfg = dict(modelgen.CONFIGS[workload]); cfg["pair_dependent_radial"] = False
    path = str(tmp_models / f"{workload}.json")
    modelgen.write_model(path, **cfg)
    pos, cell, sp = systems.config_system(workload)
    nl = neighbors.neighbor_list(pos, cell, cfg["r_cut"]); ea = neighbors.edge_arrays(nl, sp)
    e64 = gpu(path, "float64")
    e64.compute_node_energies_forces(*H.call_args(ea))
    E64, f64 = e64.node_energies.sum(), e64.node_forces
    F = e64.reduce_forces(len(pos), nl["j"])
    assert np.abs(F.sum(0)).max() < 1e-9                       # Newton's third law
    assert np.allclose(F, H.atom_forces(nl, f64, len(pos)), atol=1e-10)
    # relabelling the atoms permutes the answers
    perm = np.random.default_rng(0).permutation(len(pos))
    nl2 = neighbors.neighbor_list(pos[perm], cell, cfg["r_cut"]); ea2 = neighbors.edge_arrays(nl2, sp[perm])
    e64.compute_node_energies_forces(*H.call_args(ea2))
    assert abs(e64.node_energies.sum() - E64) <= 1e-10 * abs(E64)
    assert np.allclose(e64.reduce_forces(len(pos), nl2["j"]), F[perm], atol=1e-9)
    # fp32-feature mode against fp64 mode
    e32 = gpu(path, "float32")
    e32.compute_node_energies_forces(*H.call_args(ea))
    assert abs(e32.node_energies.sum() - E64) <= 1e-5 * abs(E64)
    assert np.abs(e32.node_forces - f64).max() <= 1e-4


def test_calculator_energy_forces_stress(gpu, tmp_models):
    """The calculator face (symmetrix_calc.py:72-102): forces are -dE/dx and the
    stress is dE/d(strain)/V, both checked by central differences of the engine's own energy."""
    from symmetrix_amd.calc import SymmetrixCalculator
    model = H.tiny_model(K=16, L_max=1, n_pts=64, seed=21)
    path = H.write_model(model, tmp_models / "calc.json")
    calc = SymmetrixCalculator(path, species=["H", "C", "O"], num_spline_points=64)   # conversion keywords are accepted
    # a file that is no symmetrix JSON: RuntimeError, as the reference's loader raises before it converts
    # (symmetrix_calc.py:54-56); the message names the conversion to run
    bad = tmp_models / "checkpoint.model"
    bad.write_bytes(b"PK\x03\x04 not json")
    with pytest.raises(RuntimeError, match="symmetrix_extract_mace"):
        SymmetrixCalculator(str(bad))
    pos, cell, sp = H.small_system(14, density=0.09, seed=8)
    Z = np.array(model["atomic_numbers"])[sp]
    res = calc.compute(pos, cell, Z)
    orc = _oracle()(model)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    orc.compute_node_energies_forces(*H.call_args(ea))
    assert res["energy"] == pytest.approx(orc.node_energies.sum(), rel=1e-10)
    assert np.allclose(res["forces"], H.atom_forces(nl, orc.node_forces, len(pos)), atol=1e-8)
    # the list built on the device (default) and the numpy builder give the same bits
    res_h = SymmetrixCalculator(path, neighbor_list="host").compute(pos, cell, Z)
    assert res_h["energy"] == res["energy"] and np.array_equal(res_h["energies"], res["energies"])
    assert np.array_equal(res_h["forces"], res["forces"]) and np.array_equal(res_h["stress"], res["stress"])
    F, e0 = res["forces"].copy(), res["energy"]
    h = 1e-5
    for a, c in ((0, 0), (3, 1), (7, 2)):
        p = pos.copy(); p[a, c] += h; ep = calc.compute(p, cell, Z)["energy"]
        p[a, c] -= 2 * h; em = calc.compute(p, cell, Z)["energy"]
        assert -(ep - em) / (2 * h) == pytest.approx(F[a, c], abs=1e-6)
    stress = calc.compute(pos, cell, Z)["stress"]
    V = float(np.prod(cell))
    voigt = [(0, 0), (1, 1), (2, 2), (1, 2), (0, 2), (0, 1)]
    for q, (a, b) in enumerate(voigt):
        def strained(eps):
            S = np.eye(3); S[a, b] += eps / 2; S[b, a] += eps / 2
            return calc.compute(pos @ S.T, np.diag(cell) @ S.T, Z)["energy"]
        d = (strained(h) - strained(-h)) / (2 * h) / V
        assert d == pytest.approx(stress[q], abs=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["ortho", "triclinic", "small_cell", "open", "empty"])
def test_device_neighbor_list_is_bit_identical_to_the_host_builder(case):
    """Edge order, integer arrays, xyz and r of the device builder against symmetrix_amd.neighbors.neighbor_list."""
    import torch
    from symmetrix_amd import neighbors
    rng = np.random.default_rng(11)
    pbc = (True, True, True)
    if case == "ortho":
        cell = np.array([13.0, 11.0, 12.5]); pos = rng.uniform(0, 1, size=(300, 3)) * cell; rc = 4.5
    elif case == "triclinic":
        cell = np.array([[9.0, 0.0, 0.0], [2.5, 8.0, 0.0], [-1.5, 2.0, 10.0]])
        pos = rng.uniform(0, 1, size=(150, 3)) @ cell; rc = 5.0
    elif case == "small_cell":
        cell = np.array([3.1, 3.3, 2.9]); pos = rng.uniform(0, 1, size=(5, 3)) * cell; rc = 5.0   # several images per pair
    elif case == "open":
        cell = np.array([30.0, 30.0, 30.0]); pos = rng.uniform(5, 12, size=(60, 3)); rc = 4.0; pbc = (False, True, False)
    else:
        cell = np.array([10.0, 10.0, 10.0]); pos = np.zeros((0, 3)); rc = 4.0
    types = rng.integers(0, 3, size=len(pos)).astype(np.int32)
    ref = neighbors.neighbor_list(pos, cell, rc, pbc)
    dpos = torch.from_numpy(np.ascontiguousarray(pos)).cuda()
    dty = torch.from_numpy(types).cuda()
    dnl = neighbors.DeviceNeighborList()
    print(f"case {case} atoms={len(pos)} edges={len(ref['r'])}", flush=True)
    E = dnl.build(len(pos), dpos.data_ptr(), dty.data_ptr(), cell, rc, pbc)
    got = dnl.to_host()
    assert E == len(ref["r"])
    assert np.array_equal(got["i"], ref["i"]) and np.array_equal(got["j"], ref["j"])
    assert np.array_equal(got["S"], ref["S"].reshape(-1, 3))
    assert np.array_equal(got["xyz"], ref["xyz"].reshape(-1, 3)) and np.array_equal(got["r"], ref["r"])
    assert np.array_equal(got["first_neigh"], ref["first_neigh"])
    assert np.array_equal(got["neigh_types"], types[ref["j"]])


@pytest.mark.gpu
def test_device_neighbor_list_update_equals_fresh_build():
    """Skin list + per-step cutoff filter at moved positions against a fresh host build at the moved positions."""
    import torch
    from symmetrix_amd import neighbors
    rng = np.random.default_rng(3)
    cell = np.array([[12.0, 0.0, 0.0], [1.0, 11.0, 0.0], [0.5, -1.0, 12.5]])
    pos = rng.uniform(0, 1, size=(400, 3)) @ cell
    types = rng.integers(0, 4, size=len(pos)).astype(np.int32)
    rc, skin = 4.5, 1.0
    dnl = neighbors.DeviceNeighborList()
    dty = torch.from_numpy(types).cuda()
    dpos = torch.from_numpy(pos).cuda()
    dnl.build(len(pos), dpos.data_ptr(), dty.data_ptr(), cell, rc, skin=skin)
    for step in range(3):
        pos = pos + rng.uniform(-0.15, 0.15, size=pos.shape)      # total drift stays below skin / 2
        dpos = torch.from_numpy(pos).cuda()
        print(f"update step {step}", flush=True)
        E = dnl.update(dpos.data_ptr(), dty.data_ptr(), rc)
        # the list keeps the frame of its build: atoms that drifted out of the cell are not folded back in
        got, ref = dnl.to_host(), neighbors.neighbor_list(pos, cell, rc, offsets=np.zeros((len(pos), 3), dtype=int))
        assert E == len(ref["r"])
        for k in ("i", "j", "S", "xyz", "r", "first_neigh"):
            assert np.array_equal(got[k], ref[k].reshape(got[k].shape)), k
    with pytest.raises(ValueError):
        dnl.update(dpos.data_ptr(), dty.data_ptr(), rc + 2 * skin)
    # the same through host arrays
    hnl = neighbors.DeviceNeighborList()
    hnl.build_host(pos, types, cell, rc, skin=skin)
    pos2 = pos + rng.uniform(-0.1, 0.1, size=pos.shape)
    E = hnl.update_host(pos2, rc)
    got, ref = hnl.to_host(), neighbors.neighbor_list(pos2, cell, rc, offsets=hnl.offsets)
    assert hnl.offsets.any()                   # some atoms had left the cell before this build
    assert E == len(ref["r"]) and np.array_equal(got["j"], ref["j"]) and np.array_equal(got["r"], ref["r"])
    assert np.array_equal(got["S"], ref["S"]) and np.array_equal(got["xyz"], ref["xyz"])
    far = pos2 + rng.integers(-2, 3, size=pos2.shape) @ cell      # whole lattice vectors away: same edges
    E2 = hnl.build_host(far, types, cell, rc)
    got2, ref2 = hnl.to_host(), neighbors.neighbor_list(far, cell, rc)
    assert E2 == len(ref2["r"]) == len(neighbors.neighbor_list(pos2, cell, rc)["r"])
    for k in ("i", "j", "S", "xyz", "r"):
        assert np.array_equal(got2[k], ref2[k].reshape(got2[k].shape)), k
    assert np.array_equal(got["neigh_types"], types[ref["j"]])


@pytest.mark.gpu
def test_device_resident_loop_positions_to_forces(gpu, tmp_models):
    """positions on the device -> device neighbour list -> compute_device -> per-atom forces, against the host path."""
    import torch
    from symmetrix_amd import neighbors
    model = H.tiny_model(K=16, L_max=1, n_pts=48, seed=5)
    path = H.write_model(model, tmp_models / "loop.json")
    eng = gpu(path)
    pos, cell, sp = H.small_system(40, seed=8)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    eng.compute_node_energies_forces(*H.call_args(ea))
    e_ref, f_ref = eng.node_energies.copy(), eng.node_forces.copy()
    dpos = torch.from_numpy(np.ascontiguousarray(pos)).cuda()
    dty = torch.from_numpy(np.asarray(sp, dtype=np.int32)).cuda()
    dnl = neighbors.DeviceNeighborList()
    E = dnl.build(len(pos), dpos.data_ptr(), dty.data_ptr(), cell, model["r_cut"])
    oE = torch.zeros(len(pos), dtype=torch.float64, device="cuda"); oF = torch.zeros(3 * E, dtype=torch.float64, device="cuda")
    p = dnl.ptr
    eng.compute_device(len(pos), dty.data_ptr(), p["num_neigh"], p["neigh_indices"], p["neigh_types"], p["xyz"], p["r"], E,
                       oE.data_ptr(), oF.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert np.array_equal(oE.cpu().numpy(), e_ref) and np.array_equal(oF.cpu().numpy(), f_ref)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float64", "float32"])
def test_receiver_chunks_of_the_layer1_adjoint_change_nothing(gpu, tmp_models, dtype):
    """A staging limit far below the message volume (many chunks, down to a few receivers each) gives the same bits."""
    model = H.tiny_model(K=16, L_max=1, n_pts=48, seed=9)
    path = H.write_model(model, tmp_models / "chunks.json")
    pos, cell, sp = H.small_system(60, seed=4)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    eng = gpu(path, dtype)
    eng.compute_node_energies_forces(*H.call_args(ea))
    e_ref, f_ref, h_ref = eng.node_energies.copy(), eng.node_forces.copy(), np.array(eng.H1_adj)
    row_bytes = 4 * 16 * (8 if dtype == "float64" else 4)
    for limit in (len(ea["r"]) * row_bytes // 3, 200 * row_bytes, int(ea["num_neigh"].max()) * row_bytes):
        eng.set_staging_limit(limit)
        print(f"staging limit {limit} bytes", flush=True)
        eng.compute_node_energies_forces(*H.call_args(ea))
        assert np.array_equal(eng.node_energies, e_ref)
        assert np.array_equal(eng.node_forces, f_ref)
        assert np.array_equal(np.array(eng.H1_adj), h_ref)
    eng.set_staging_limit(row_bytes)          # below one receiver's messages
    with pytest.raises(RuntimeError):
        eng.compute_node_energies_forces(*H.call_args(ea))


# (L_max, dtype, one radial table for all pairs, ZBL, density normalisation).  One table and scalar hidden features
# take the channel-slice kernels, whose layer-1 partial forces wait in the staging array for the layer-0 adjoint
# (K = 16 is a whole number of 32-byte slices in both precisions): with ghost nodes, ZBL or the density
# normalisation the force array has other contributions before, between and beside those two.
MODE_CASES = [(0, "float64", False, False, False), (1, "float64", False, True, True), (0, "float32", False, True, False),
              (1, "float32", False, True, True), (2, "float64", False, True, True)]
MODE_CASES += [(0, dt, True, zbl, dens) for dt in ("float64", "float32")
               for zbl, dens in ((False, False), (True, False), (False, True), (True, True))]


@pytest.mark.gpu
@pytest.mark.parametrize("L_max,dtype,one_table,zbl,density", MODE_CASES)
def test_pair_style_modes_agree(gpu, tmp_models, L_max, dtype, one_table, zbl, density):
    """The three ways the pair style feeds the engine on one rank give one answer (the reference's
    tests/test_pair_symmetrix_mace.py:28-39): owners as senders (no_domain_decomposition), ghost nodes that go
    through layer 0 (no_mpi_message_passing, one call), and ghost rows of H1 filled by a forward copy with the
    adjoint summed back (mpi_message_passing, stage calls as pair_symmetrix_mace.cpp:372-550 issues them).  The
    first is compared with the oracle, the others with the first."""
    from symmetrix_amd import neighbors
    model = H.tiny_model(K=16, L_max=L_max, n_pts=48, seed=12, pair=not one_table, zbl=zbl, density=density)
    path = H.write_model(model, tmp_models / f"modes{L_max}{dtype}{int(one_table)}{int(zbl)}{int(density)}.json")
    pos, cell, sp = H.small_system(36, seed=21)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    N = len(sp)
    eng = gpu(path, dtype)
    assert eng._int("num_radial_tables_0") == (1 if one_table else 6)
    eng.compute_node_energies_forces(*H.call_args(ea))
    orc = _oracle()(model)
    orc.compute_node_energies_forces(*H.call_args(ea))
    _compare(orc, eng, dtype, names=[])
    e_ref = eng.node_energies.copy()
    f_ref = eng.reduce_forces(N, ea["neigh_indices"])
    ga = neighbors.ghost_edge_arrays(nl, sp)
    Nl, Ng = ga["num_local_nodes"], ga["num_ghost_nodes"]
    assert Ng > 0
    print(f"ghost mode: {Nl} local + {Ng} ghost nodes, {len(ga['r'])} edges", flush=True)
    eng.compute_ghosted(Nl, Ng, ga["node_types"], ga["num_neigh"], ga["neigh_indices"], ga["neigh_types"], ga["xyz"], ga["r"])
    e_g = eng.node_energies.copy()
    f_g = eng.reduce_forces(N, ga["sender_atom"], ga["receiver_atom"])
    assert e_g.shape == (Nl,)
    ftol = 1e-11 if dtype == "float64" else 2e-5
    assert np.array_equal(e_g, e_ref)      # same edges in the same order for every local receiver
    assert np.abs(f_g - f_ref).max() <= ftol * max(1.0, np.abs(f_ref).max())
    assert np.abs(f_g - H.atom_forces(nl, orc.node_forces, N)).max() <= TOL[dtype]["F"]
    # the same call again, and after an evaluation of the owner layout in between: bit for bit
    eng.compute_node_energies_forces(*H.call_args(ea))
    eng.compute_ghosted(Nl, Ng, ga["node_types"], ga["num_neigh"], ga["neigh_indices"], ga["neigh_types"], ga["xyz"], ga["r"])
    assert np.array_equal(eng.node_energies, e_g)
    assert np.array_equal(eng.reduce_forces(N, ga["sender_atom"], ga["receiver_atom"]), f_g)

    # message-passing mode: local nodes only; H1 of the ghosts copied from their owners, H1_adj summed back
    El = int(ga["num_neigh"][:Nl].sum())
    nt, nn = ga["node_types"][:Nl], ga["num_neigh"][:Nl]
    ni, nty, x, r = ga["neigh_indices"][:El], ga["neigh_types"][:El], ga["xyz"][:3 * El], ga["r"][:El]
    eng2 = gpu(path, dtype)
    eng2.fill("node_energies", Nl); eng2.fill("node_forces", 3 * El)
    if eng2.has_zbl:
        eng2.zbl.compute_ZBL(Nl, nt, nn, nty, eng2.atomic_numbers, r, x)         # pair_symmetrix_mace.cpp:449-452
    eng2.compute_Y(x)
    eng2.compute_R0(Nl, nt, nn, nty, r); eng2.compute_A0(Nl, nt, nn, nty); eng2.compute_A0_scaled(Nl, nt, nn, nty, r)
    eng2.compute_M0(Nl, nt); eng2.compute_H1(Nl)
    nlm_k = eng2.H1.size // Nl
    H1 = np.array(eng2.H1).reshape(Nl, nlm_k)
    eng2.H1 = np.concatenate([H1, H1[ga["ghost_owner"]]]).reshape(-1)          # forward_comm
    eng2.compute_R1(Nl, nt, nn, nty, r); eng2.compute_Phi1(Nl, nn, ni); eng2.compute_A1(Nl)
    eng2.compute_A1_scaled(Nl, nt, nn, nty, r); eng2.compute_M1(Nl, nt); eng2.compute_H2(Nl, nt)
    eng2.compute_readouts(Nl, nt)
    eng2.reverse_H2(Nl, nt, False); eng2.reverse_M1(Nl, nt)
    eng2.reverse_A1_scaled(Nl, nt, nn, nty, x, r, False); eng2.reverse_A1(Nl)
    eng2.reverse_Phi1(Nl, nn, ni, x, r, False, False)
    Hadj = np.array(eng2.H1_adj).reshape(Nl + Ng, nlm_k)
    np.add.at(Hadj, ga["ghost_owner"], Hadj[Nl:])                                # reverse_comm
    eng2.H1_adj = Hadj[:Nl].reshape(-1).copy()
    eng2.reverse_H1(Nl); eng2.reverse_M0(Nl, nt); eng2.reverse_A0_scaled(Nl, nt, nn, nty, x, r)
    eng2.reverse_A0(Nl, nt, nn, nty, x, r)
    etol = 1e-12 if dtype == "float64" else 1e-6
    assert np.abs(eng2.node_energies - e_ref).max() <= etol * max(1.0, np.abs(e_ref).max())
    f_m = eng2.reduce_forces(N, ga["sender_atom"][:El])
    assert np.abs(f_m - f_ref).max() <= ftol * 10 * max(1.0, np.abs(f_ref).max())


@pytest.mark.gpu
def test_rotation_and_replication_through_the_calculator(tmp_models):
    """A rigid rotation of positions and cell leaves the energy alone and rotates the forces; a cell repeated along
    an axis repeats energies and forces.  Both go through the device neighbour list with general triclinic cells."""
    from symmetrix_amd.calc import SymmetrixCalculator
    model = H.tiny_model(K=16, L_max=1, n_pts=64, seed=31, zbl=True, density=True)
    path = H.write_model(model, tmp_models / "rot.json")
    calc = SymmetrixCalculator(path)
    pos, cell, sp = H.small_system(24, density=0.08, seed=13)
    Z = np.array(model["atomic_numbers"])[sp]
    cell = np.diag(cell)
    res = calc.compute(pos, cell, Z)
    e0, f0, en0 = res["energy"], res["forces"].copy(), res["energies"].copy()
    rng = np.random.default_rng(5)
    Q, _ = np.linalg.qr(rng.normal(size=(3, 3)))
    if np.linalg.det(Q) < 0:
        Q[:, 0] = -Q[:, 0]
    rot = calc.compute(pos @ Q.T, cell @ Q.T, Z)
    assert abs(rot["energy"] - e0) <= 1e-10 * abs(e0)
    assert np.abs(rot["forces"] - f0 @ Q.T).max() <= 1e-8 * max(1.0, np.abs(f0).max())
    pos2 = np.concatenate([pos, pos + cell[0]])
    cell2 = cell.copy(); cell2[0] *= 2
    rep = calc.compute(pos2, cell2, np.concatenate([Z, Z]))
    assert np.abs(rep["energies"][:len(pos)] - en0).max() <= 1e-10 * max(1.0, np.abs(en0).max())
    assert np.abs(rep["energies"][len(pos):] - en0).max() <= 1e-10 * max(1.0, np.abs(en0).max())
    assert np.abs(rep["forces"][:len(pos)] - f0).max() <= 1e-8 * max(1.0, np.abs(f0).max())
    assert np.abs(rep["stress"] - res["stress"]).max() <= 1e-9 * max(1.0, np.abs(res["stress"]).max())


@pytest.mark.gpu
@pytest.mark.parametrize("L_max", [0, 1])
def test_a_step_captured_in_a_hip_graph_replays_bitwise(gpu, tmp_models, L_max):
    """Callers that cannot launch from the host each step capture the device-resident call once (after a call at the
    same sizes, which allocates) and replay it.  Replays are interleaved with eager calls on other inputs and each
    one is compared with the eager result."""
    import torch
    model = H.tiny_model(K=32, L_max=L_max, n_pts=48, seed=17, zbl=True, density=(L_max == 1))
    path = H.write_model(model, tmp_models / f"graph{L_max}.json")
    eng = gpu(path, "float64")
    pos, cell, sp = H.small_system(50, seed=2)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    N, E = len(sp), len(ea["r"])
    dev = torch.device("cuda:0")
    t = lambda a, dt: torch.from_numpy(np.ascontiguousarray(a)).to(dev, dtype=dt)
    d = [t(ea["node_types"], torch.int32), t(ea["num_neigh"], torch.int32), t(ea["neigh_indices"], torch.int32),
         t(ea["neigh_types"], torch.int32), t(ea["xyz"], torch.float64), t(ea["r"], torch.float64)]
    xyz0, r0 = d[4].clone(), d[5].clone()
    oE = torch.zeros(N, dtype=torch.float64, device=dev); oF = torch.zeros(3 * E, dtype=torch.float64, device=dev)
    s = torch.cuda.Stream()

    def step():
        eng.compute_device(N, *[x.data_ptr() for x in d], E, oE.data_ptr(), oF.data_ptr(), s.cuda_stream)

    with torch.cuda.stream(s):
        step()
    torch.cuda.synchronize()
    refE, refF = oE.clone(), oF.clone()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        step()
    torch.cuda.synchronize()
    rng = np.random.default_rng(0)
    for rep in range(3):
        # eager work on other inputs in between: the same geometry scaled, which changes every intermediate
        scale = 1.0 - 0.01 * (rep + 1)
        d[4].copy_(xyz0 * scale); d[5].copy_(r0 * scale)
        with torch.cuda.stream(s):
            step()
        torch.cuda.synchronize()
        assert not torch.equal(oF, refF)
        d[4].copy_(xyz0); d[5].copy_(r0)
        oE.zero_(); oF.zero_()
        torch.cuda.synchronize()
        print(f"replay {rep}", flush=True)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(oE, refE) and torch.equal(oF, refF)


@pytest.mark.gpu
@pytest.mark.parametrize("L_max,big,one_table", [(0, False, False), (1, False, False), (0, True, False), (0, False, True)])
def test_device_resident_call_checks_its_inputs_on_the_device(gpu, tmp_models, L_max, big, one_table):
    """Arrays handed over as device addresses are checked inside the list preparation; when a check fails, the
    evaluation runs on emptied lists (no unchecked integer is used as an address), node energies and edge forces come
    back as NaN and the next synchronising call (synchronize, get_array, reduce_forces) raises.  Every kernel exits
    normally; the call after is unaffected, also when both are replays of one captured graph.
    `big`: more than 65 536 atoms, where the preparation is made of separate launches; `one_table`: the
    channel-slice kernels, whose forces come out of the sum over slices."""
    import torch
    from symmetrix_amd import neighbors, systems
    model = H.tiny_model(K=16 if big else 32, L_max=L_max, n_pts=48, seed=40 + L_max, r_cut=3.0 if big else 4.0,
                         pair=not one_table)
    path = H.write_model(model, tmp_models / f"guard{L_max}{int(big)}{int(one_table)}.json")
    if big:
        pos, cell, sp = systems.fcc_alloy((26, 26, 25), n_species=3, seed=1)     # 67 600 atoms
    else:
        pos, cell, sp = H.small_system(40, seed=5)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    N, E = len(sp), len(ea["r"])
    dev = torch.device("cuda:0")
    t = lambda a, dt: torch.from_numpy(np.ascontiguousarray(a)).to(dev, dtype=dt)
    names = ["node_types", "num_neigh", "neigh_indices", "neigh_types", "xyz", "r"]
    good = {k: t(ea[k], torch.float64 if k in ("xyz", "r") else torch.int32) for k in names}
    oE = torch.zeros(N, dtype=torch.float64, device=dev); oF = torch.zeros(3 * E, dtype=torch.float64, device=dev)
    eng = gpu(path, "float64")
    stream = torch.cuda.current_stream().cuda_stream

    def run(d):
        eng.compute_device(N, *[d[k].data_ptr() for k in names], E, oE.data_ptr(), oF.data_ptr(), stream)
        torch.cuda.synchronize()

    run(good)
    eng.synchronize()
    e_ref, f_ref = oE.clone(), oF.clone()
    F_ref = eng.reduce_forces(N, ea["neigh_indices"])
    assert torch.isfinite(e_ref).all() and torch.isfinite(f_ref).all()
    bad_cases = {"sender row": ("neigh_indices", 5, N + 3), "edge species": ("neigh_types", 0, 3),
                 "node species": ("node_types", 1, -1), "counts": ("num_neigh", 0, int(ea["num_neigh"][0]) + 1),
                 "edge length": ("r", 3, 2.0 * model["r_cut"])}
    for n_case, (what, (key, pos_, value)) in enumerate(bad_cases.items()):
        d = dict(good); d[key] = good[key].clone(); d[key][pos_] = value
        print(f"bad {what} (L_max {L_max}, {N} atoms)", flush=True)
        oF.zero_()
        run(d)
        assert torch.isnan(oE).all(), what
        assert torch.isnan(oF).all(), what
        with pytest.raises(ValueError):
            if n_case % 2 == 0:
                eng.synchronize()
            else:
                eng.reduce_forces(N, ea["neigh_indices"])     # the per-atom sums of NaN forces are not handed out silently
        eng.synchronize()                       # reported once
        run(good)
        eng.synchronize()
        assert torch.equal(oE, e_ref) and torch.equal(oF, f_ref), what
        assert np.array_equal(eng.reduce_forces(N, ea["neigh_indices"]), F_ref)
    if big:
        return
    # one captured graph, replayed on bad and then on good inputs: a skipped replay leaves nothing behind
    live = {k: good[k].clone() for k in names}
    s = torch.cuda.Stream()

    def step():
        eng.compute_device(N, *[live[k].data_ptr() for k in names], E, oE.data_ptr(), oF.data_ptr(), s.cuda_stream)

    with torch.cuda.stream(s):
        step()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        step()
    torch.cuda.synchronize()
    for rep in range(2):
        live["neigh_indices"][5] = N + 3
        torch.cuda.synchronize()
        print(f"graph replay {rep}: bad, then good", flush=True)
        g.replay()
        torch.cuda.synchronize()
        assert torch.isnan(oE).all() and torch.isnan(oF).all()
        live["neigh_indices"].copy_(good["neigh_indices"])
        oE.zero_(); oF.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(oE, e_ref) and torch.equal(oF, f_ref)
        with pytest.raises(ValueError):
            eng.synchronize()                   # the skipped replay is still reported, once
        eng.synchronize()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float64", "float32"])
def test_layer0_gradients_on_request_follow_the_calls(gpu, tmp_models, dtype):
    """With several polynomials per channel the whole-pipeline call keeps no M0_grad (its adjoint recomputes it); the
    array is formed when it is asked for, from the evaluation that ran last, and stage-level calls made afterwards
    (which do store gradients, as the reference's methods do) see consistent arrays.  Sequence: evaluation A, ask;
    evaluation B on fewer atoms, reverse_M0 as a stage call (needs the gradients of B), ask; evaluation A again:
    bit-identical to the first."""
    model = H.tiny_model(K=24, L_max=1, n_pts=64, seed=31, pair=False)
    path = H.write_model(model, tmp_models / "lazy_grad.json")
    eng = gpu(path, dtype)
    assert eng._int("contraction_tables") == 3
    tol = 1e-10 if dtype == "float64" else 2e-4
    runs = {}
    for tag, n in (("A", 60), ("B", 23)):
        pos, cell, sp = H.small_system(n, seed=n)
        nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
        orc = _oracle()(model)
        orc.compute_node_energies_forces(*H.call_args(ea))
        runs[tag] = (ea, orc)
    ea, orc = runs["A"]
    eng.compute_node_energies_forces(*H.call_args(ea))
    fA, eA = eng.node_forces.copy(), eng.node_energies.copy()
    assert np.abs(eng.M0_grad - orc.M0_grad).max() <= tol * max(1.0, np.abs(orc.M0_grad).max())
    ea, orc = runs["B"]
    eng.compute_node_energies_forces(*H.call_args(ea))
    a0_adj = eng.A0_adj.copy()
    assert np.abs(a0_adj - orc.A0_adj).max() <= tol * max(1.0, np.abs(orc.A0_adj).max())
    eng.reverse_M0(ea["num_nodes"], ea["node_types"])          # stage call: streams over stored gradients
    assert np.abs(eng.A0_adj - a0_adj).max() <= tol * max(1.0, np.abs(a0_adj).max())
    assert eng.M0_grad.shape == orc.M0_grad.shape
    assert np.abs(eng.M0_grad - orc.M0_grad).max() <= tol * max(1.0, np.abs(orc.M0_grad).max())
    ea, orc = runs["A"]
    eng.compute_node_energies_forces(*H.call_args(ea))
    assert np.array_equal(eng.node_forces, fA) and np.array_equal(eng.node_energies, eA)
    assert np.abs(eng.M0_grad - orc.M0_grad).max() <= tol * max(1.0, np.abs(orc.M0_grad).max())
