"""Host-side logic that needs no GPU: neighbour lists, the model generator's
structure, and that the C-ABI library loads and exports every declared symbol."""
import ctypes as C
import json
import os
import re

import numpy as np
import pytest

from symmetrix_amd import _lib, cg, modelgen, neighbors, systems
from tests import helpers as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("L,N,rc", [(6.0, 30, 5.0), (12.0, 100, 4.5), (4.0, 5, 5.0), (3.0, 1, 4.0)])
def test_neighbor_list_matches_brute_force(L, N, rc):
    rng = np.random.default_rng(int(L * 10 + N))
    pos = rng.uniform(0, L, size=(N, 3))
    cell = [L, L * 1.1, L * 0.9]
    a = neighbors.neighbor_list(pos, cell, rc)
    b = neighbors.brute_force_neighbor_list(pos, cell, rc)
    for k in ("i", "j", "S", "xyz", "r"):
        assert np.array_equal(a[k], b[k]), k          # integers and floats bit-exact
    # canonical order: (i, j, Sx, Sy, Sz) ascending, no duplicates
    key = np.stack([a["i"], a["j"], a["S"][:, 0], a["S"][:, 1], a["S"][:, 2]], axis=1)
    assert all(tuple(key[q]) < tuple(key[q + 1]) for q in range(len(key) - 1))
    assert np.all(a["r"] < rc)


def test_neighbor_list_symmetric_full_list():
    pos, cell, sp = systems.random_box(60, 0.1, [0.5, 0.5], seed=2)
    nl = neighbors.neighbor_list(pos, cell, 4.0)
    fwd = set(zip(nl["i"].tolist(), nl["j"].tolist(), map(tuple, nl["S"].tolist())))
    for i, j, S in fwd:
        assert (j, i, (-S[0], -S[1], -S[2])) in fwd
    ea = neighbors.edge_arrays(nl, sp)
    # the ASE caller counts neighbours over j (symmetrix_calc.py:80): same thing for a full list
    assert np.array_equal(ea["num_neigh"], np.bincount(nl["j"], minlength=len(pos)))


def test_empty_and_open_boundaries():
    pos = np.array([[0.0, 0.0, 0.0], [10.0, 0.0, 0.0]])
    nl = neighbors.neighbor_list(pos, [30.0, 30.0, 30.0], 3.0)
    assert len(nl["i"]) == 0 and nl["first_neigh"].tolist() == [0, 0, 0]
    nl = neighbors.neighbor_list(np.array([[0.5, 0.5, 0.5], [2.5, 0.5, 0.5]]), [3.0, 30.0, 30.0], 2.5, pbc=(False, True, True))
    assert len(nl["i"]) == 2                          # no image across the open direction


def test_no_atoms_and_image_shift_table():
    nl = neighbors.neighbor_list(np.zeros((0, 3)), [10.0, 10.0, 10.0], 4.0)
    assert len(nl["r"]) == 0 and list(nl["first_neigh"]) == [0]
    cell = np.array([[4.0, 0.0, 0.0], [1.0, 5.0, 0.0], [0.0, 0.0, 30.0]])
    ints, vecs = neighbors.image_shifts(cell, 4.5, pbc=(True, True, False))
    # two shells along a (height 4.0 below the cutoff), one along b, none along the open axis; lexicographic
    assert ints.shape == (15, 3) and np.array_equal(ints[0], [-2, -1, 0]) and np.array_equal(ints[-1], [2, 1, 0])
    assert [tuple(t) for t in ints] == sorted(tuple(t) for t in ints)
    assert np.array_equal(vecs, ints.astype(float) @ cell)
    # every shift the list uses is in the table
    pos = np.random.default_rng(0).uniform(0, 1, size=(12, 3)) @ cell
    used = {tuple(t) for t in neighbors.neighbor_list(pos, cell, 4.5, (True, True, False))["S"]}
    assert used <= {tuple(t) for t in ints}


def test_real_cg_couples_harmonics():
    rng = np.random.default_rng(0)
    u = rng.normal(size=(6, 3))
    Y = cg.real_sph_harm(u)
    for (l, l1, l2) in cg.tensor_product_paths(3, 1):
        Cg = cg.real_cg(l1, l2, l)
        out = np.einsum("na,nb,abc->nc", Y[:, l1 * l1:(l1 + 1) ** 2], Y[:, l2 * l2:(l2 + 1) ** 2], Cg)
        ratio = out / Y[:, l * l:(l + 1) ** 2]
        assert np.allclose(ratio, ratio.flat[0], rtol=1e-9)
        assert np.allclose((Cg ** 2).sum(axis=(0, 1)), 1.0)


def test_generator_emits_every_key_the_loader_reads():
    m = json.loads(json.dumps(H.tiny_model(K=3, L_max=1, n_pts=12)))
    keys = ["num_elements", "num_channels", "r_cut", "l_max", "L_max", "atomic_numbers", "atomic_energies", "has_zbl",
            "radial_spline_h", "radial_spline_values_0", "radial_spline_derivs_0", "radial_spline_values_1",
            "radial_spline_derivs_1", "H0_weights", "A0_weights", "A0_scaled", "M0_weights", "M0_monomials",
            "H1_weights", "Phi1_l", "Phi1_l1", "Phi1_l2", "Phi1_lme", "Phi1_clebsch_gordan", "Phi1_lelm1lm2",
            "A1_weights", "A1_scaled", "M1_weights", "M1_monomials", "H2_weights_for_H1", "H2_weights_for_M1",
            "readout_1_weights", "readout_2_weights_1", "readout_2_weights_2", "readout_2_scale_factor"]
    for k in keys:                                     # mace.cpp:912-1029
        assert k in m, k
    T, K = 3, 3
    assert np.array(m["radial_spline_values_0"]).shape == (T * (T + 1) // 2, 4 * K, 12)
    P = len(m["Phi1_l"])
    assert P == 10 and m["Phi1_l"] == sorted(m["Phi1_l"])          # non-decreasing, mace.cpp:619-640
    assert np.array(m["radial_spline_values_1"]).shape == (6, P * K, 12)
    assert [len(w) for w in m["A1_weights"]] == [n * K * K for n in (2, 3, 3, 2)]
    assert sorted(m["M0_monomials"].keys()) == ["0", "1", "2", "3"]
    assert len(m["M0_weights"]["2"]["3"]["1"]) == len(m["M0_monomials"]["3"])
    assert max(len(t) for t in m["M1_monomials"]) == 3
    assert max(m["Phi1_lme"]) == 39 and max(m["Phi1_lelm1lm2"]) == 87    # n_e = 40, n_r = 88
    # spline grid as the extractor's: knots on linspace(1e-12, r_cut, n)
    assert m["radial_spline_h"] == pytest.approx((m["r_cut"] - 1e-12) / 11)


def test_capi_library_exports_declared_symbols():
    """Every function declared in include/symmetrix_amd.h is exported by the built library."""
    header = open(os.path.join(ROOT, "include", "symmetrix_amd.h")).read()
    declared = set(re.findall(r"\b(smx_[a-zA-Z0-9_]+)\s*\(", header))
    declared.discard("smx_model")
    assert declared == set(_lib.EXPORTS)
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libsymmetrix_amd.so not built yet (python -c 'import __graft_entry__ as g; g.build()')")
    L = C.CDLL(_lib.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(L, name), name
    L.smx_stage_names.restype = C.c_char_p
    assert L.smx_stage_names().decode().split(";")[0] == "prep"


def test_capi_error_paths_without_gpu(tmp_path):
    """File errors are reported before any device is touched."""
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libsymmetrix_amd.so not built yet")
    L = _lib.lib()
    h = C.c_void_p()
    assert L.smx_model_load(str(tmp_path / "missing.json").encode(), 0, C.byref(h)) == -2
    assert b"cannot open" in L.smx_last_error()
    bad = tmp_path / "bad.json"
    bad.write_text('{"num_elements": 2, ')
    assert L.smx_model_load(str(bad).encode(), 0, C.byref(h)) == -2
    nokey = tmp_path / "nokey.json"
    nokey.write_text('{"num_elements": 2}')
    assert L.smx_model_load(str(nokey).encode(), 0, C.byref(h)) == -2
    assert b"missing key" in L.smx_last_error()
    assert L.smx_model_load(None, 0, C.byref(h)) == -1
    m = H.tiny_model(K=2, L_max=0, n_pts=8)
    m["M1_monomials"][0] = [0, 1, 2, 3]                      # degree 4: outside the device kernels
    p = H.write_model(m, tmp_path / "deg4.json")
    assert L.smx_model_load(p.encode(), 0, C.byref(h)) == -3
    assert b"degree 4" in L.smx_last_error()
    import torch
    if not torch.cuda.is_available():
        good = H.write_model(H.tiny_model(K=2, L_max=0, n_pts=8), tmp_path / "good.json")
        assert L.smx_model_load(good.encode(), 0, C.byref(h)) == -4   # no device: fails loudly, no CPU path
        with pytest.raises(RuntimeError):
            from symmetrix_amd.mace import MACE
            MACE(good)


def test_cpp_class_header_compiles():
    """include/symmetrix_amd/mace.hpp is a drop-in for libsymmetrix's mace.hpp for a C++20 caller: the statement
    forms the reference pair style applies to its evaluator compile unchanged (tests/cpp/reference_caller_syntax.cpp),
    and so does the LAMMPS-free half of this repository's pair style."""
    import subprocess
    inc = ["-I", os.path.join(ROOT, "include", "symmetrix_amd"), "-I", os.path.join(ROOT, "include")]
    for src in (os.path.join(ROOT, "tests", "cpp", "reference_caller_syntax.cpp"),
                os.path.join(ROOT, "pair_symmetrix_amd", "mace_evaluation.cpp")):
        r = subprocess.run(["g++", "-std=c++20", "-Wall", "-Wextra", "-fsyntax-only", *inc, src], capture_output=True)
        assert r.returncode == 0, r.stderr.decode()


@pytest.mark.parametrize("triclinic", [False, True])
def test_neighbor_list_of_atoms_outside_the_cell(triclinic):
    """Atoms translated by whole lattice vectors (as molecular dynamics leaves them: nothing wraps positions
    between steps, and the reference's calculator passes them on unwrapped, symmetrix_calc.py:77) keep the same
    neighbours: same (i, j) sets, the shifts differ by the translations, xyz and r agree to rounding.  The two
    atoms of a 10 A cell at x = 1.0 and x = 21.5 are 0.5 A apart."""
    cell = np.array([[10.0, 0, 0], [0, 10.0, 0], [0, 0, 10.0]])
    nl = neighbors.neighbor_list(np.array([[1.0, 5, 5], [21.5, 5, 5]]), cell, 3.0)
    assert len(nl["i"]) == 2 and np.allclose(nl["r"], 0.5)
    assert nl["S"].tolist() == [[-2, 0, 0], [2, 0, 0]] and np.allclose(nl["xyz"][0], [0.5, 0, 0])
    rng = np.random.default_rng(5)
    cell = np.array([[7.0, 0, 0], [1.5, 6.5, 0], [-0.8, 0.9, 7.5]]) if triclinic else np.diag([7.0, 6.5, 7.5])
    N = 25
    pos = rng.uniform(0, 1, size=(N, 3)) @ cell
    moves = rng.integers(-3, 4, size=(N, 3))
    moved = pos + moves @ cell
    a = neighbors.neighbor_list(pos, cell, 4.0)
    b = neighbors.neighbor_list(moved, cell, 4.0)
    c = neighbors.brute_force_neighbor_list(moved, cell, 4.0)
    assert len(a["i"]) > 0
    for other in (b, c):
        assert np.array_equal(a["i"], other["i"]) and np.array_equal(a["j"], other["j"])
        assert np.array_equal(a["S"] + moves[a["i"]] - moves[a["j"]], other["S"])
        assert np.allclose(a["xyz"], other["xyz"], rtol=0, atol=1e-12) and np.allclose(a["r"], other["r"], rtol=0, atol=1e-12)
    # open axis: no folding along it
    d = neighbors.neighbor_list(moved, cell, 4.0, pbc=(True, True, False))
    e = neighbors.brute_force_neighbor_list(moved, cell, 4.0, pbc=(True, True, False))
    assert np.array_equal(d["i"], e["i"]) and np.array_equal(d["j"], e["j"]) and np.array_equal(d["S"], e["S"])
    w, off = neighbors.wrap_positions(moved, cell)
    assert np.allclose(w + off @ cell, moved, atol=1e-12) and np.all((w @ np.linalg.inv(cell) > -1e-9) & (w @ np.linalg.inv(cell) < 1 + 1e-9))


def test_calculator_keeps_the_reference_signature():
    """symmetrix_calc.py:39: Symmetrix(model_file, dtype="float64", use_kokkos=True, **kwargs), and the keywords it
    forwards to the conversion of a torch checkpoint (:58-61) are accepted."""
    import inspect
    from symmetrix_amd.calc import Symmetrix, SymmetrixCalculator
    for cls in (Symmetrix, SymmetrixCalculator):
        sig = inspect.signature(cls.__init__)
        names = list(sig.parameters)
        assert names[:4] == ["self", "model_file", "dtype", "use_kokkos"]
        assert sig.parameters["dtype"].default == "float64" and sig.parameters["use_kokkos"].default is True
        assert any(p.kind is inspect.Parameter.VAR_KEYWORD for p in sig.parameters.values())
    assert SymmetrixCalculator.implemented_properties == ["energy", "free_energy", "energies", "forces", "stress"]
    assert SymmetrixCalculator.EXTRACT_KEYWORDS == ("species", "head", "num_spline_points")
    with pytest.raises(ValueError):
        SymmetrixCalculator("x.json", dtype="float16")


def test_compiled_monomial_tables_are_the_generators_output():
    """smx_poly_tables.inc (the monomial lists the straight-line contraction kernel is compiled for) is committed;
    it must equal what gen_poly_tables.py writes, and list for every output slot exactly the monomials a generated
    model carries, in the same order."""
    import importlib.util
    csrc = os.path.join(ROOT, "symmetrix_amd", "csrc")
    spec = importlib.util.spec_from_file_location("gen_poly_tables", os.path.join(csrc, "gen_poly_tables.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    with open(os.path.join(csrc, "smx_poly_tables.inc")) as f:
        assert f.read() == gen.render()
    from symmetrix_amd import modelgen
    model = modelgen.generate_model([1, 8], 2, 2, 4.0, num_spline_points=16, seed=0)
    tabs = gen.tables()
    assert len(tabs) == 9
    for LM, monos in model["M0_monomials"].items():
        assert [tuple([gen.ONE] * (3 - len(m)) + list(m)) for m in monos] == tabs[int(LM)]
    assert [tuple([gen.ONE] * (3 - len(m)) + list(m)) for m in model["M1_monomials"]] == tabs[0]


def test_contraction_slab_shapes_are_valid_for_every_channel_count(tmp_path):
    """The loader lays the coefficient slabs of the contraction kernel out with the function the launcher sizes its
    blocks with (smx_poly_shape.hpp, plain C++): for every channel count up to 512, one, four and nine polynomials
    and both precisions the shape must be one the kernel can run (channel block a multiple of 16 that tiles the
    padded channel count, at most 256 threads per pass, slabs of all resident blocks within the LDS of a CU)."""
    import subprocess
    exe = str(tmp_path / "poly_shape_check")
    r = subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-I", os.path.join(ROOT, "symmetrix_amd", "csrc"), "-o", exe,
                        os.path.join(ROOT, "tests", "cpp", "poly_shape_check.cpp")], capture_output=True)
    assert r.returncode == 0, r.stderr.decode()
    r = subprocess.run([exe], capture_output=True)
    out = r.stdout.decode()
    assert r.returncode == 0 and "BAD" not in out, out
    # the padded monomial counts in front of polynomials 1, 4, 9 (94 | 112 92 112 | 90 97 95 97 98, each to a multiple of 4)
    assert "offsets 96 412 900" in out
    # the headline shape: 96 channels, one polynomial, double: 32 channels and 24 KB per block, four blocks per CU
    assert "elem 8 NP 1 K 96: CB 32 AG 8 kblocks 3 blocks 4 slab 24576" in out
