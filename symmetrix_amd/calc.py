"""Calculator face: energy, per-atom energies, forces and stress of an atomic
configuration, the work of `Symmetrix.calculate`
(symmetrix/source/symmetrix/symmetrix_calc.py:72-102), without requiring ASE.

`SymmetrixCalculator.compute(positions, cell, atomic_numbers)` builds the
canonical neighbour list on the device (the counterpart of the
neighbor_list('ijdD') call at symmetrix_calc.py:77-83; bit-identical to the
numpy builder of this package, which `neighbor_list="host"` selects), calls the
engine on the device-resident edge arrays and reduces per-edge forces to atoms
on the device.  When ASE is importable, `Symmetrix` is an
`ase.calculators.calculator.Calculator` with the reference's constructor
signature and `implemented_properties`.
"""
from __future__ import annotations

import numpy as np

from . import neighbors
from .mace import MACE


class SymmetrixCalculator:
    implemented_properties = ["energy", "free_energy", "energies", "forces", "stress"]

    # keywords the reference hands to its on-the-fly conversion of a torch checkpoint (symmetrix_calc.py:58-61)
    EXTRACT_KEYWORDS = ("species", "head", "num_spline_points")

    def __init__(self, model_file, dtype="float64", use_kokkos=True, neighbor_list="device", **kwargs):
        """Signature and defaults of the reference's `Symmetrix.__init__` (symmetrix_calc.py:39).  `use_kokkos`
        selects between two back ends there; here there is one, for both dtypes, and the flag is ignored."""
        if dtype not in ("float32", "float64"):
            raise ValueError(f"Unsupported dtype '{dtype}'. Supported dtypes are 'float64' and 'float32'.")
        if neighbor_list not in ("device", "host"):
            raise ValueError("neighbor_list is 'device' or 'host'")
        self.use_kokkos = use_kokkos
        self.extract_kwargs = {k: v for k, v in kwargs.items() if k in self.EXTRACT_KEYWORDS}
        unknown = sorted(set(kwargs) - set(self.EXTRACT_KEYWORDS))
        if unknown:
            raise TypeError(f"unexpected keyword arguments {unknown}")
        try:
            self.evaluator = MACE(str(model_file), dtype)
        except RuntimeError as exc:
            # The reference converts a torch-MACE checkpoint here (symmetrix_calc.py:54-68); that needs mace-torch,
            # e3nn and ase, and this package holds no extractor: say what to run instead of failing on the parse error.
            raise RuntimeError(
                f"'{model_file}' is not a symmetrix JSON model ({exc}).  Convert the checkpoint once with the "
                f"reference's extractor, e.g. `symmetrix_extract_mace {model_file}` with {self.extract_kwargs or 'its defaults'}, "
                f"and pass the JSON file it writes.") from exc
        self.cutoff = self.evaluator.r_cut
        self.results = {}
        self._nlist = neighbors.DeviceNeighborList() if neighbor_list == "device" else None

    def compute(self, positions, cell, atomic_numbers, pbc=(True, True, True)):
        Z = [int(z) for z in atomic_numbers]
        table = self.evaluator.atomic_numbers
        try:
            species = np.array([table.index(z) for z in Z], dtype=np.int32)
        except ValueError as exc:
            raise ValueError("an atom's element is not in the model") from exc
        ev = self.evaluator
        n_atoms = len(Z)
        if self._nlist is not None:
            E = self._nlist.build_host(positions, species, cell, self.cutoff, pbc)
            p = self._nlist.ptr
            ev.compute_device(n_atoms, p["node_types"], p["num_neigh"], p["neigh_indices"], p["neigh_types"], p["xyz"],
                              p["r"], E)
            ev.synchronize()
            energies = ev.node_energies
            if E:
                forces, virial = ev.reduce_forces_device(n_atoms, p["neigh_indices"], virial=True)
            else:
                forces, virial = np.zeros((n_atoms, 3)), np.zeros(6)
        else:
            nl = neighbors.neighbor_list(positions, cell, self.cutoff, pbc)
            ea = neighbors.edge_arrays(nl, species)
            ev.compute_node_energies_forces(ea["num_nodes"], ea["node_types"], ea["num_neigh"], ea["neigh_indices"],
                                            ea["neigh_types"], ea["xyz"], ea["r"])
            energies = ev.node_energies
            forces, virial = ev.reduce_forces(n_atoms, nl["j"], virial=True)
        cell = np.asarray(cell, dtype=np.float64)
        volume = abs(np.linalg.det(np.diag(cell) if cell.shape == (3,) else cell))
        # symmetrix_calc.py:102: stress = -(pair_forces^T xyz)/V in Voigt order xx,yy,zz,yz,xz,xy
        stress = -np.array([virial[0], virial[1], virial[2], virial[5], virial[4], virial[3]]) / volume
        self.results = {"energy": float(energies.sum()), "free_energy": float(energies.sum()),
                        "energies": energies, "forces": forces, "stress": stress}
        return self.results


try:  # pragma: no cover - ase is not installed in the build image
    from ase.calculators.calculator import Calculator, all_changes

    class Symmetrix(Calculator):
        implemented_properties = SymmetrixCalculator.implemented_properties

        def __init__(self, model_file, dtype="float64", use_kokkos=True, **kwargs):
            Calculator.__init__(self, **kwargs)     # symmetrix_calc.py:40: every keyword goes to the base class
            extract = {k: v for k, v in kwargs.items() if k in SymmetrixCalculator.EXTRACT_KEYWORDS}
            self._impl = SymmetrixCalculator(model_file, dtype, use_kokkos, **extract)
            self.use_kokkos = use_kokkos
            self.evaluator = self._impl.evaluator
            self.cutoff = self._impl.cutoff

        def calculate(self, atoms=None, properties=("energy",), system_changes=all_changes):
            Calculator.calculate(self, atoms, properties, system_changes)
            self.results = dict(self._impl.compute(self.atoms.get_positions(), self.atoms.get_cell().array,
                                                   self.atoms.get_atomic_numbers(), self.atoms.get_pbc()))
except ImportError:
    Symmetrix = SymmetrixCalculator
