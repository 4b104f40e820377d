"""The benchmark configurations that the other GPU tests do not run as such: the 192-atom H/C/O case at full size
against the oracle, the 25 002-atom water-like box through the pair style's ghost-node layout, the 50 000-atom
alloy's model on a small box against the oracle, and the capacity run's molecular-dynamics loop (positions moved on
the device, neighbour list searched or filtered on the device, evaluation on device-resident arrays) at a size that
takes seconds and at its full size of a million atoms."""
import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu
TOL = {"float64": dict(E=1e-10, F=1e-8), "float32": dict(E=1e-5, F=1e-4)}


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    from symmetrix_amd.mace import MACE
    return MACE


def _model_file(tmp_models, name, **override):
    import os
    from symmetrix_amd import modelgen
    cfg = dict(modelgen.CONFIGS[name]); cfg.update(override)
    tag = "_".join(f"{k}{v}" for k, v in sorted(override.items()))
    path = str(tmp_models / f"cfg_{name}_{tag}.json")
    if not os.path.exists(path):
        modelgen.write_model(path, **cfg)
    return path, cfg


@pytest.mark.parametrize("dtype", ["float64", "float32"])
@pytest.mark.parametrize("pair", [False, True], ids=["one_table", "pair_tables"])
def test_tiny_configuration_at_full_size_against_the_oracle(gpu, tmp_models, pair, dtype):
    """192 atoms H/C/O at 0.10 atoms/A^3, K = 32, r_cut 5.0 A, 256 spline points: the configuration the reference
    CPU path runs.  With one radial table (plain MACE) the channel-slice kernels serve both layers, with six pair
    tables the general ones do."""
    from oracle.oracle import OracleMACE
    from symmetrix_amd import neighbors, systems
    path, cfg = _model_file(tmp_models, "tiny", pair_dependent_radial=pair)
    pos, cell, sp = systems.config_system("tiny")
    assert len(pos) == 192
    nl = neighbors.neighbor_list(pos, cell, cfg["r_cut"]); ea = neighbors.edge_arrays(nl, sp)
    print(f"tiny: {len(pos)} atoms, {len(ea['r'])} edges, pair tables {pair}, {dtype}", flush=True)
    orc = OracleMACE(path)
    orc.compute_node_energies_forces(*H.call_args(ea))
    eng = gpu(path, dtype)
    eng.compute_node_energies_forces(*H.call_args(ea))
    Eo = orc.node_energies.sum()
    assert abs(eng.node_energies.sum() - Eo) <= TOL[dtype]["E"] * abs(Eo)
    assert np.abs(eng.node_forces - orc.node_forces).max() <= TOL[dtype]["F"]
    F = eng.reduce_forces(len(pos), nl["j"])
    assert np.abs(F - H.atom_forces(nl, orc.node_forces, len(pos))).max() <= TOL[dtype]["F"] * 10


@pytest.mark.parametrize("dtype", ["float64", "float32"])
def test_headline_configuration_at_full_size_against_the_oracle(gpu, tmp_models, dtype):
    """3 000 atoms H/C/N/O, K = 96, scalar hidden features, one radial table: the benchmark's headline workload,
    whole, against the oracle (about two seconds of CPU).  At this size the symmetric contraction takes two atom
    groups per block in double precision (96 channels fill three wavefronts only in pairs), which small cases never do."""
    from oracle.oracle import OracleMACE
    from symmetrix_amd import neighbors, systems
    path, cfg = _model_file(tmp_models, "off_small", pair_dependent_radial=False)
    pos, cell, sp = systems.config_system("off_small")
    assert len(pos) == 3000 and cfg["num_channels"] == 96
    nl = neighbors.neighbor_list(pos, cell, cfg["r_cut"]); ea = neighbors.edge_arrays(nl, sp)
    print(f"off_small: {len(pos)} atoms, {len(ea['r'])} edges, {dtype}", flush=True)
    orc = OracleMACE(path)
    orc.compute_node_energies_forces(*H.call_args(ea))
    eng = gpu(path, dtype)
    eng.compute_node_energies_forces(*H.call_args(ea))
    Eo = orc.node_energies.sum()
    assert abs(eng.node_energies.sum() - Eo) <= TOL[dtype]["E"] * abs(Eo)
    assert np.abs(eng.node_energies - orc.node_energies).max() <= TOL[dtype]["E"] * max(1.0, np.abs(orc.node_energies).max()) * 10
    assert np.abs(eng.node_forces - orc.node_forces).max() <= TOL[dtype]["F"]


@pytest.mark.parametrize("dtype", ["float64", "float32"])
@pytest.mark.parametrize("L_max", [0, 1])
@pytest.mark.parametrize("foreign", [False, True])
def test_contraction_blocks_of_several_atom_groups(gpu, tmp_models, L_max, dtype, foreign):
    """4 400 atoms with K = 32, one polynomial (scalar hidden features) and four.  The kernel of the standard product
    basis gives every block a run of several passes of eight atoms; with a monomial from outside that basis in every
    polynomial the general kernel runs, and packs two atom groups of 32 channels into one wavefront per variable group
    in either precision (single precision takes four atoms per thread and needs more than 4 096 atoms for it)."""
    from oracle.oracle import OracleMACE
    model = H.tiny_model(K=32, L_max=L_max, n_pts=64, seed=40 + L_max, pair=False)
    if foreign:
        H.add_foreign_monomials(model, seed=5)
    path = H.write_model(model, tmp_models / f"groups_{L_max}_{int(foreign)}.json")
    pos, cell, sp = H.small_system(4400, seed=9)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    print(f"case K=32 L_max={L_max} atoms=4400 edges={len(ea['r'])} {dtype}", flush=True)
    orc = OracleMACE(path)
    orc.compute_node_energies_forces(*H.call_args(ea))
    eng = gpu(path, dtype)
    assert eng._int("contraction_tables") == (0 if foreign else 3)
    eng.compute_node_energies_forces(*H.call_args(ea))
    Eo = orc.node_energies.sum()
    assert abs(eng.node_energies.sum() - Eo) <= TOL[dtype]["E"] * max(abs(Eo), np.abs(orc.node_energies).sum() * 1e-3)
    assert np.abs(eng.node_forces - orc.node_forces).max() <= TOL[dtype]["F"] * max(1.0, np.abs(orc.node_forces).max())


def test_contraction_runs_of_several_passes(gpu, tmp_models):
    """30 000 atoms with 16 channels and four polynomials per channel: more atoms than the contraction kernel of the
    standard product basis has thread slots on the chip, so every block walks its run of atoms in two (single
    precision) or three (double) passes with the coefficient slab it loaded once; values, the recomputing adjoint
    and the layer-1 launch against the oracle (about 20 s of CPU, once for both precisions)."""
    from oracle.oracle import OracleMACE
    model = H.tiny_model(K=16, L_max=1, n_pts=64, seed=77, pair=False)
    path = H.write_model(model, tmp_models / "passes.json")
    pos, cell, sp = H.small_system(30000, seed=5)
    nl, ea = H.edges_of(pos, cell, sp, model["r_cut"])
    print(f"case K=16 L_max=1 atoms=30000 edges={len(ea['r'])}", flush=True)
    orc = OracleMACE(path)
    orc.compute_node_energies_forces(*H.call_args(ea))
    Eo = orc.node_energies.sum()
    for dtype in ("float64", "float32"):
        eng = gpu(path, dtype)
        assert eng._int("contraction_tables") == 3
        eng.compute_node_energies_forces(*H.call_args(ea))
        assert abs(eng.node_energies.sum() - Eo) <= TOL[dtype]["E"] * max(abs(Eo), np.abs(orc.node_energies).sum() * 1e-3)
        assert np.abs(eng.node_energies - orc.node_energies).max() <= TOL[dtype]["E"] * max(1.0, np.abs(orc.node_energies).max()) * 10
        assert np.abs(eng.node_forces - orc.node_forces).max() <= TOL[dtype]["F"] * max(1.0, np.abs(orc.node_forces).max())
        for name in ("M0", "M1", "A0_adj", "M0_grad"):
            a, b = getattr(orc, name), getattr(eng, name)
            tol = 1e-10 if dtype == "float64" else 2e-4      # the bound test_gpu_parity.py puts on intermediates
            assert a.shape == b.shape and np.abs(a - b).max() <= tol * max(1.0, np.abs(a).max()), name


def test_water_box_with_ghost_nodes_at_full_size(gpu, tmp_models):
    """25 002 atoms, K = 128, hidden features up to l = 1, r_cut 5.0 A, through the full neighbour list with ghost
    atoms as extra nodes (the pair style's no_mpi_message_passing layout on one rank): node energies bit-equal to
    the owner-indexed layout, atom forces equal to rounding, Newton's third law; the same model on a 1 % box against
    the oracle in both layouts."""
    from oracle.oracle import OracleMACE
    from symmetrix_amd import neighbors, systems
    path, cfg = _model_file(tmp_models, "off_medium", pair_dependent_radial=False)
    pos, cell, sp = systems.config_system("off_medium")
    N = len(pos)
    assert N == 25002
    nl = neighbors.neighbor_list(pos, cell, cfg["r_cut"]); ea = neighbors.edge_arrays(nl, sp)
    ga = neighbors.ghost_edge_arrays(nl, sp)
    Nl, Ng = ga["num_local_nodes"], ga["num_ghost_nodes"]
    print(f"water box: {N} atoms, {len(ea['r'])} edges; ghost layout {Ng} ghost nodes, {len(ga['r'])} edges", flush=True)
    assert Nl == N and Ng > 5000
    eng = gpu(path, "float64")
    eng.compute_node_energies_forces(*H.call_args(ea))
    e_own = eng.node_energies.copy()
    F_own = eng.reduce_forces(N, nl["j"])
    assert np.abs(F_own.sum(0)).max() < 1e-8
    eng.compute_ghosted(Nl, Ng, ga["node_types"], ga["num_neigh"], ga["neigh_indices"], ga["neigh_types"], ga["xyz"], ga["r"])
    e_gh = eng.node_energies.copy()
    F_gh = eng.reduce_forces(N, ga["sender_atom"], ga["receiver_atom"])
    assert np.array_equal(e_gh, e_own)
    assert np.abs(F_gh - F_own).max() <= 1e-9 * max(1.0, np.abs(F_own).max())
    e32 = gpu(path, "float32")
    e32.compute_ghosted(Nl, Ng, ga["node_types"], ga["num_neigh"], ga["neigh_indices"], ga["neigh_types"], ga["xyz"], ga["r"])
    assert abs(e32.node_energies.sum() - e_own.sum()) <= 1e-5 * abs(e_own.sum())
    # hydrogens are placed without regard to other molecules, so some pairs are nearly on top of each other and their
    # forces reach hundreds of eV/A: the float32 bound of 1e-4 eV/A is taken relative to that scale here
    f_scale = max(1.0, np.abs(F_own).max())
    print(f"largest force component {f_scale:.1f} eV/A", flush=True)
    assert np.abs(e32.reduce_forces(N, ga["sender_atom"], ga["receiver_atom"]) - F_own).max() <= 1e-4 * f_scale
    # 1 % of the box (same recipe and density) against the oracle
    pos, cell, sp = systems.config_system("off_medium", scale=0.01)
    nl = neighbors.neighbor_list(pos, cell, cfg["r_cut"]); ea = neighbors.edge_arrays(nl, sp)
    ga = neighbors.ghost_edge_arrays(nl, sp)
    n = len(pos)
    print(f"1 % box: {n} atoms, {len(ea['r'])} edges, {ga['num_ghost_nodes']} ghost nodes", flush=True)
    orc = OracleMACE(path)
    orc.compute_node_energies_forces(*H.call_args(ea))
    F_ref = H.atom_forces(nl, orc.node_forces, n)
    for dtype, engine in (("float64", eng), ("float32", e32)):
        engine.compute_ghosted(n, ga["num_ghost_nodes"], ga["node_types"], ga["num_neigh"], ga["neigh_indices"],
                               ga["neigh_types"], ga["xyz"], ga["r"])
        Eo = orc.node_energies.sum()
        assert abs(engine.node_energies.sum() - Eo) <= TOL[dtype]["E"] * abs(Eo), dtype
        F = engine.reduce_forces(n, ga["sender_atom"], ga["receiver_atom"])
        fs = max(1.0, np.abs(orc.node_forces).max()) if dtype == "float32" else 1.0
        assert np.abs(F - F_ref).max() <= TOL[dtype]["F"] * 10 * fs, dtype
        engine.compute_node_energies_forces(*H.call_args(ea))
        assert np.abs(engine.node_forces - orc.node_forces).max() <= TOL[dtype]["F"] * fs, dtype


@pytest.mark.parametrize("dtype", ["float64", "float32"])
def test_capacity_loop_at_reduced_size(gpu, tmp_models, dtype):
    """The capacity run's loop on 49 920 atoms (4 x 4 x 4 copies of a 780-atom water box): before the first move
    all 64 copies of an atom get the same energy and force; then every step moves the atoms on the device by
    N(0, 0.01^2) A, searches the list anew every fifth step and filters the remembered pairs otherwise, and
    evaluates on the device-resident arrays.  After the last step the result is compared with an evaluation of a
    list built on the host from the final positions."""
    import torch
    from symmetrix_amd import neighbors, systems
    path, cfg = _model_file(tmp_models, "off_medium", pair_dependent_radial=False)
    dev = torch.device("cuda:0")
    reps, n_mol = 4, 260
    bpos, bcell, bsp = systems.water_box(n_mol, seed=0)
    nb = len(bpos)
    offs = np.array([[a, b, c] for a in range(reps) for b in range(reps) for c in range(reps)], dtype=np.float64) * bcell
    pos = (offs[:, None, :] + bpos[None, :, :]).reshape(-1, 3)
    species = np.tile(bsp, reps ** 3).astype(np.int32)
    cell = bcell * reps
    N = len(pos)
    r_cut, skin = cfg["r_cut"], 0.6
    dpos = torch.from_numpy(np.ascontiguousarray(pos)).to(dev)
    dty = torch.from_numpy(species).to(dev)
    eng = gpu(path, dtype)
    dnl = neighbors.DeviceNeighborList()
    stream = torch.cuda.current_stream().cuda_stream
    out_E = torch.zeros(N, dtype=torch.float64, device=dev)

    def evaluate(E):
        p = dnl.ptr
        out_F = torch.zeros(3 * E, dtype=torch.float64, device=dev)
        eng.compute_device(N, dty.data_ptr(), p["num_neigh"], p["neigh_indices"], p["neigh_types"], p["xyz"], p["r"], E,
                           out_E.data_ptr(), out_F.data_ptr(), stream)
        F = eng.reduce_forces_device(N, p["neigh_indices"])
        return out_E.cpu().numpy().copy(), F

    E = dnl.build(N, dpos.data_ptr(), dty.data_ptr(), cell, r_cut, skin=skin)
    print(f"capacity loop: {N} atoms, {E} edges, {dtype}", flush=True)
    en, F = evaluate(E)
    e_rep, f_rep = en.reshape(reps ** 3, nb), F.reshape(reps ** 3, nb, 3)
    e_scale, f_scale = np.abs(e_rep[0]).max(), np.abs(f_rep[0]).max()
    etol, ftol = (1e-11, 1e-9) if dtype == "float64" else (2e-5, 2e-4)
    assert np.abs(e_rep - e_rep[0]).max() <= etol * e_scale
    assert np.abs(f_rep - f_rep[0]).max() <= ftol * max(1.0, f_scale)
    gen = torch.Generator(device=dev); gen.manual_seed(0)
    for it in range(12):
        dpos.add_(torch.randn(dpos.shape, dtype=torch.float64, device=dev, generator=gen), alpha=0.01)
        if it % 5 == 0:
            E = dnl.build(N, dpos.data_ptr(), dty.data_ptr(), cell, r_cut, skin=skin)
        else:
            E = dnl.update(dpos.data_ptr(), dty.data_ptr(), r_cut)
        en, F = evaluate(E)
        assert np.isfinite(en).all() and np.isfinite(F).all()
        if it % 4 == 0:
            print(f"  step {it}: {E} edges, E = {en.sum():.6f}", flush=True)
    # the final state from a list built on the host (atoms that left the cell are folded in there)
    final = dpos.cpu().numpy()
    nl = neighbors.neighbor_list(final, cell, r_cut); ea = neighbors.edge_arrays(nl, species)
    assert len(ea["r"]) == E
    eng.compute_node_energies_forces(*H.call_args(ea))
    e_host = eng.node_energies
    F_host = eng.reduce_forces(N, nl["j"])
    tol = TOL[dtype]
    fs = max(1.0, np.abs(F).max()) if dtype == "float32" else 1.0
    assert abs(e_host.sum() - en.sum()) <= tol["E"] * abs(en.sum())
    assert np.abs(F_host - F).max() <= tol["F"] * 10 * fs


@pytest.mark.parametrize("dtype", ["float64", "float32"])
def test_alloy_configuration_model_against_the_oracle(gpu, tmp_models, dtype):
    """The model of the 50 000-atom alloy workload (5 species, K = 128, hidden features up to l = 1, 10 Bessel
    functions, r_cut 6.0 A, 256 spline points) on a 4 x 4 x 3-cell box of the same lattice, displacements and species
    draw (192 atoms, about 80 neighbours each; the box is shorter than two cutoffs along z, so a pair also meets
    through a periodic image), against the oracle."""
    from oracle.oracle import OracleMACE
    from symmetrix_amd import neighbors, systems
    path, cfg = _model_file(tmp_models, "mp_medium", pair_dependent_radial=False)
    assert cfg["num_channels"] == 128 and cfg["L_max"] == 1 and cfg["r_cut"] == 6.0
    pos, cell, sp = systems.config_system("mp_medium", scale=0.004)
    assert len(pos) == 192 and len(set(sp.tolist())) == 5
    nl = neighbors.neighbor_list(pos, cell, cfg["r_cut"]); ea = neighbors.edge_arrays(nl, sp)
    print(f"alloy model: {len(pos)} atoms, {len(ea['r'])} edges, {dtype}", flush=True)
    orc = OracleMACE(path)
    orc.compute_node_energies_forces(*H.call_args(ea))
    eng = gpu(path, dtype)
    eng.compute_node_energies_forces(*H.call_args(ea))
    Eo = orc.node_energies.sum()
    assert abs(eng.node_energies.sum() - Eo) <= TOL[dtype]["E"] * abs(Eo)
    assert np.abs(eng.node_energies - orc.node_energies).max() <= TOL[dtype]["E"] * max(1.0, np.abs(orc.node_energies).max()) * 10
    assert np.abs(eng.node_forces - orc.node_forces).max() <= TOL[dtype]["F"]
    F = eng.reduce_forces(len(pos), nl["j"])
    assert np.abs(F - H.atom_forces(nl, orc.node_forces, len(pos))).max() <= TOL[dtype]["F"] * 10


def test_capacity_configuration_at_full_size(gpu, tmp_models):
    """The capacity configuration at its size: the l <= 1 water model on 1 000 128 atoms (4 x 4 x 4 copies of a
    15 627-atom water box, about 5.4e7 edges), float32 features.  Device list search, evaluation, two steps with the
    cutoff filter and one with a new search, every atom moved by N(0, 0.01^2) A per step on the device.  Before the
    first move the 64 copies of an atom must agree in energy and force (equal up to summation order: the copies'
    edges are the same vectors); afterwards energies and forces stay finite and the energy moves smoothly.  The
    adjoint messages (2 KB per edge) do not fit the staging buffer, so the receiver-chunked path runs."""
    import torch
    from symmetrix_amd import neighbors, systems
    free_b, _ = torch.cuda.mem_get_info()
    if free_b < 200e9:
        pytest.skip(f"needs about 185 GB of free HBM, {free_b / 1e9:.0f} GB are free")
    path, cfg = _model_file(tmp_models, "off_medium", pair_dependent_radial=False)
    dev = torch.device("cuda:0")
    reps, n_mol = 4, 5209
    bpos, bcell, bsp = systems.water_box(n_mol, seed=0)
    nb = len(bpos)
    offs = np.array([[a, b, c] for a in range(reps) for b in range(reps) for c in range(reps)], dtype=np.float64) * bcell
    pos = (offs[:, None, :] + bpos[None, :, :]).reshape(-1, 3)
    species = np.tile(bsp, reps ** 3).astype(np.int32)
    cell = bcell * reps
    N = len(pos)
    assert N == 1000128
    r_cut, skin = cfg["r_cut"], 0.6
    dpos = torch.from_numpy(np.ascontiguousarray(pos)).to(dev)
    dty = torch.from_numpy(species).to(dev)
    del pos
    eng = gpu(path, "float32")
    dnl = neighbors.DeviceNeighborList()
    stream = torch.cuda.current_stream().cuda_stream
    out_E = torch.zeros(N, dtype=torch.float64, device=dev)
    out_F = None

    def evaluate(E):
        nonlocal out_F
        if out_F is None or out_F.numel() < 3 * E:
            out_F = torch.zeros(int(3 * E * 1.02), dtype=torch.float64, device=dev)
        p = dnl.ptr
        eng.compute_device(N, dty.data_ptr(), p["num_neigh"], p["neigh_indices"], p["neigh_types"], p["xyz"], p["r"], E,
                           out_E.data_ptr(), out_F.data_ptr(), stream)
        eng.synchronize()
        return eng.reduce_forces_device(N, p["neigh_indices"])

    E = dnl.build(N, dpos.data_ptr(), dty.data_ptr(), cell, r_cut, skin=skin)
    print(f"capacity configuration: {N} atoms, {E} edges", flush=True)
    assert E > 5.0e7
    F = evaluate(E)
    free_after, total_b = torch.cuda.mem_get_info()
    print(f"  first evaluation done, {(total_b - free_after) / 1e9:.0f} GB of HBM in use", flush=True)
    assert (total_b - free_after) < 288e9
    en = out_E.cpu().numpy()
    e_rep, f_rep = en.reshape(reps ** 3, nb), F.reshape(reps ** 3, nb, 3)
    e_scale, f_scale = np.abs(e_rep[0]).max(), np.abs(f_rep[0]).max()
    e_dev, f_dev = np.abs(e_rep - e_rep[0]).max(), np.abs(f_rep - f_rep[0]).max()
    print(f"  64 copies: energy differs by {e_dev:.2e} (scale {e_scale:.2f}), force by {f_dev:.2e} (scale {f_scale:.1f})", flush=True)
    # float32 features: 1e-5 relative in energy, 1e-4 eV/A in force relative to the largest force of the box (the
    # recipe drops hydrogens next to other molecules: forces of a hundred eV/A)
    assert e_dev <= 2e-5 * e_scale and f_dev <= 2e-4 * max(1.0, f_scale)
    assert np.abs(F.sum(0)).max() <= 1e-6 * N ** 0.5 * max(1.0, f_scale)     # Newton's third law
    e_prev = en.sum()
    gen = torch.Generator(device=dev); gen.manual_seed(0)
    for it, search in enumerate((False, False, True)):
        dpos.add_(torch.randn(dpos.shape, dtype=torch.float64, device=dev, generator=gen), alpha=0.01)
        if search:
            E = dnl.build(N, dpos.data_ptr(), dty.data_ptr(), cell, r_cut, skin=skin)
        else:
            E = dnl.update(dpos.data_ptr(), dty.data_ptr(), r_cut)
        F = evaluate(E)
        e_now = float(out_E.sum().item())
        print(f"  step {it} ({'search' if search else 'filter'}): {E} edges, E = {e_now:.3f}", flush=True)
        assert np.isfinite(F).all() and np.isfinite(e_now)
        assert abs(e_now - e_prev) <= 0.05 * abs(e_prev)
        e_prev = e_now
    del eng, dnl, out_F, out_E, dpos, dty
    torch.cuda.empty_cache()
