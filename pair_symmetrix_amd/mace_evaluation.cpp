#include "mace_evaluation.h"

#include <algorithm>
#include <stdexcept>

namespace symmetrix_amd {

void EdgeList::clear()
{
    num_local_nodes = num_ghost_nodes = 0;
    node_types.clear(); num_neigh.clear(); neigh_indices.clear(); neigh_types.clear();
    xyz.clear(); r.clear(); node_i.clear(); neigh_j.clear();
}

void evaluate_no_domain_decomposition(MACE& mace, const EdgeList& e)
{
    mace.compute_node_energies_forces(e.num_local_nodes, e.node_types, e.num_neigh, e.neigh_indices, e.neigh_types,
                                      e.xyz, e.r);
}

namespace {
// outputs start from zero; the ZBL term goes in first (pair_symmetrix_mace.cpp:444-452, 660-670)
void begin_evaluation(MACE& mace, const EdgeList& e, int num_energy_nodes)
{
    mace.node_energies.assign((std::size_t)num_energy_nodes, 0.0);
    mace.node_forces.assign(e.xyz.size(), 0.0);
    if (mace.has_zbl)
        mace.zbl.compute_ZBL(num_energy_nodes, e.node_types, e.num_neigh, e.neigh_types, mace.atomic_numbers, e.r, e.xyz,
                             mace.node_energies, mace.node_forces);
}
}  // namespace

void evaluate_mpi_message_passing(MACE& mace, const EdgeList& e, int num_atom_rows, const HaloExchange& halo,
                                  std::vector<double>& H1, std::vector<double>& H1_adj)
{
    if (e.num_ghost_nodes != 0) throw std::invalid_argument("mpi_message_passing takes local nodes only");
    const int N = e.num_local_nodes;
    const std::size_t w = (std::size_t)mace.num_LM * mace.num_channels;
    begin_evaluation(mace, e, N);
    mace.compute_Y(e.xyz);
    mace.compute_R0(N, e.node_types, e.num_neigh, e.neigh_types, e.r);
    mace.compute_A0(N, e.node_types, e.num_neigh, e.neigh_types);
    mace.compute_A0_scaled(N, e.node_types, e.num_neigh, e.neigh_types, e.r);
    mace.compute_M0(N, e.node_types);
    mace.compute_H1(N);
    // rows of the local nodes go to their atom rows, the exchange fills the ghost rows (:462-471)
    H1.assign((std::size_t)num_atom_rows * w, 0.0);
    {
        const symmetrix_amd::Mirror& h = mace.H1;
        for (int ii = 0; ii < N; ++ii)
            std::copy(h.begin() + (std::size_t)ii * w, h.begin() + (std::size_t)(ii + 1) * w, H1.begin() + (std::size_t)e.node_i[ii] * w);
    }
    if (halo.forward) halo.forward(H1);
    mace.H1 = H1;
    mace.compute_R1(N, e.node_types, e.num_neigh, e.neigh_types, e.r);
    mace.compute_Phi1(N, e.num_neigh, e.neigh_j);
    mace.compute_A1(N);
    mace.compute_A1_scaled(N, e.node_types, e.num_neigh, e.neigh_types, e.r);
    mace.compute_M1(N, e.node_types);
    mace.compute_H2(N, e.node_types);
    mace.compute_readouts(N, e.node_types);
    mace.reverse_H2(N, e.node_types, false);
    mace.reverse_M1(N, e.node_types);
    mace.reverse_A1_scaled(N, e.node_types, e.num_neigh, e.neigh_types, e.xyz, e.r, false);
    mace.reverse_A1(N);
    mace.reverse_Phi1(N, e.num_neigh, e.neigh_j, e.xyz, e.r, false, false);
    // adjoint rows of the ghosts go back to their owners (:487-490)
    H1_adj = mace.H1_adj;
    if (halo.reverse) halo.reverse(H1_adj);
    // back from atom rows to node rows (the reference hands the atom-row array over as it is, which is the same
    // thing when node ii is atom ii)
    {
        std::vector<double> by_node((std::size_t)N * w);
        for (int ii = 0; ii < N; ++ii)
            std::copy(H1_adj.begin() + (std::size_t)e.node_i[ii] * w, H1_adj.begin() + (std::size_t)(e.node_i[ii] + 1) * w,
                      by_node.begin() + (std::size_t)ii * w);
        mace.H1_adj = std::move(by_node);
    }
    mace.reverse_H1(N);
    mace.reverse_M0(N, e.node_types);
    mace.reverse_A0_scaled(N, e.node_types, e.num_neigh, e.neigh_types, e.xyz, e.r);
    mace.reverse_A0(N, e.node_types, e.num_neigh, e.neigh_types, e.xyz, e.r);
}

void evaluate_no_mpi_message_passing(MACE& mace, const EdgeList& e, bool staged)
{
    const int Nl = e.num_local_nodes, Na = e.num_nodes();
    if (!staged) {
        mace.compute_node_energies_forces_ghosted(Nl, e.num_ghost_nodes, e.node_types, e.num_neigh, e.neigh_indices,
                                                  e.neigh_types, e.xyz, e.r);
        return;
    }
    begin_evaluation(mace, e, Nl);
    mace.compute_Y(e.xyz);
    mace.compute_R0(Na, e.node_types, e.num_neigh, e.neigh_types, e.r);
    mace.compute_A0(Na, e.node_types, e.num_neigh, e.neigh_types);
    mace.compute_A0_scaled(Na, e.node_types, e.num_neigh, e.neigh_types, e.r);
    mace.compute_M0(Na, e.node_types);
    mace.compute_H1(Na);
    mace.compute_R1(Nl, e.node_types, e.num_neigh, e.neigh_types, e.r);
    mace.compute_Phi1(Nl, e.num_neigh, e.neigh_indices);
    mace.compute_A1(Nl);
    mace.compute_A1_scaled(Nl, e.node_types, e.num_neigh, e.neigh_types, e.r);
    mace.compute_M1(Nl, e.node_types);
    mace.compute_H2(Nl, e.node_types);
    mace.compute_readouts(Nl, e.node_types);
    mace.reverse_H2(Nl, e.node_types, false);
    mace.reverse_M1(Nl, e.node_types);
    mace.reverse_A1_scaled(Nl, e.node_types, e.num_neigh, e.neigh_types, e.xyz, e.r, false);
    mace.reverse_A1(Nl);
    mace.reverse_Phi1(Nl, e.num_neigh, e.neigh_indices, e.xyz, e.r, false, false);
    mace.reverse_H1(Na);
    mace.reverse_M0(Na, e.node_types);
    mace.reverse_A0_scaled(Na, e.node_types, e.num_neigh, e.neigh_types, e.xyz, e.r);
    mace.reverse_A0(Na, e.node_types, e.num_neigh, e.neigh_types, e.xyz, e.r);
}

double total_energy(MACE& mace, const EdgeList& e, double* eatom)
{
    const symmetrix_amd::Mirror& en = mace.node_energies;
    double sum = 0.0;
    for (int ii = 0; ii < e.num_local_nodes; ++ii) {
        sum += en[ii];
        if (eatom) eatom[e.node_i[ii]] = en[ii];
    }
    return sum;
}

void scatter_forces(MACE& mace, const EdgeList& e, int num_atom_rows, double* f, double* virial)
{
    if (num_atom_rows <= 0) return;
    std::vector<double> fa((std::size_t)3 * num_atom_rows, 0.0);
    double v[6] = {0, 0, 0, 0, 0, 0};
    mace.flush();
    symmetrix_amd::check(smx_reduce_forces(mace.handle(), num_atom_rows, e.neigh_j.data(), e.node_i.data(), fa.data(),
                                           virial ? v : nullptr));
    for (std::size_t q = 0; q < fa.size(); ++q) f[q] += fa[q];
    if (virial)
        for (int q = 0; q < 6; ++q) virial[q] += v[q];
}

}  // namespace symmetrix_amd
