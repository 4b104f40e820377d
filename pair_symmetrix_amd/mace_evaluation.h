// Engine-facing half of `pair_style symmetrix/mace`, free of LAMMPS types: what the reference pair
// style does between its "begin mace evaluation" and "end mace evaluation" marks, plus the scatter
// of per-edge forces to atoms (pair_symmetrix/pair_symmetrix_mace.cpp:319-368, 444-546, 660-744),
// written over the C++ face of the engine (include/symmetrix_amd/mace.hpp).
#pragma once

#include <functional>
#include <span>
#include <vector>

#include "symmetrix_amd/mace.hpp"

namespace symmetrix_amd {

// Flat edge arrays of one step, receiver blocks in node order (pair_symmetrix_mace.cpp:268-315,
// 404-440, 596-658).  Local nodes come first; ghost nodes (mode no_mpi_message_passing only) follow.
// neigh_indices: row of the sender in the H1 array of the mode in use; node_i / neigh_j: atom rows
// (LAMMPS local + ghost numbering) of receiver and sender, used by the force scatter.
struct EdgeList {
    int num_local_nodes = 0, num_ghost_nodes = 0;
    std::vector<int> node_types, num_neigh, neigh_indices, neigh_types;
    std::vector<double> xyz, r;
    std::vector<int> node_i, neigh_j;
    int num_nodes() const { return num_local_nodes + num_ghost_nodes; }
    void clear();
};

// Halo exchange of the mode mpi_message_passing: rows[atom row][num_LM * num_channels].  `forward` fills
// the ghost rows from their owners (comm->forward_comm, pair_symmetrix_mace.cpp:470); `reverse` adds the
// ghost rows to their owners (comm->reverse_comm, :489).
struct HaloExchange {
    std::function<void(std::vector<double>& rows)> forward, reverse;
};

// no_domain_decomposition (:319-320): senders are owners, one call.
void evaluate_no_domain_decomposition(MACE& mace, const EdgeList& e);

// mpi_message_passing (:444-495): the stage sequence with the two exchanges in the middle.  num_atom_rows =
// nlocal + nghost; H1 / H1_adj are the pair style's exchange buffers, indexed by atom row.
void evaluate_mpi_message_passing(MACE& mace, const EdgeList& e, int num_atom_rows, const HaloExchange& halo,
                                  std::vector<double>& H1, std::vector<double>& H1_adj);

// no_mpi_message_passing (:660-698).  `staged` false: one call into the engine, which runs layer 0 on all nodes
// and layer 1 on the local ones; `staged` true: the reference's stage-by-stage sequence (same result, more
// launches and host round trips; kept for cross-checking).
void evaluate_no_mpi_message_passing(MACE& mace, const EdgeList& e, bool staged = false);

// Sum of node energies of the local nodes (:324-332, 499-502, 702-704).  With `eatom`, node ii's energy is written
// to eatom[node_i[ii]], the atom row of the node (the reference writes eatom[ii], :329-331, 504-507: the same entry
// while ilist[ii] == ii).
double total_energy(MACE& mace, const EdgeList& e, double* eatom = nullptr);

// f[node_i] -= f_ij, f[neigh_j] += f_ij over all edges (:334-347, 509-522, 710-723) into f[num_atom_rows][3],
// and the global virial in LAMMPS order xx, yy, zz, xy, xz, yz (:349-368) when virial is not null.  Both are
// accumulated into.  Runs on the device (smx_reduce_forces: fixed summation order, no atomics); only the
// per-atom forces and six numbers cross PCIe.
void scatter_forces(MACE& mace, const EdgeList& e, int num_atom_rows, double* f, double* virial);

}  // namespace symmetrix_amd
