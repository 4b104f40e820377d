// Compile-only check (g++ -std=c++20 -fsyntax-only): the statement forms a caller written against the
// reference's libsymmetrix/source/mace.hpp applies to its evaluator -- std::unique_ptr<MACE>, members resized,
// filled, assigned from and to std::vector<double>, indexed, `mace->zbl.compute_ZBL(...)` with the members as
// output spans, every stage method with std::vector arguments -- as the pair style's stage-by-stage modes use
// them (pair_symmetrix/pair_symmetrix_mace.cpp:444-546, 660-744).
#include <algorithm>
#include <memory>
#include <vector>

#include "mace.hpp"

double reference_style_calls(const char* file, int num_nodes, std::vector<int>& node_types, std::vector<int>& num_neigh,
                             std::vector<int>& neigh_j, std::vector<int>& neigh_types, std::vector<double>& xyz,
                             std::vector<double>& r)
{
    std::unique_ptr<MACE> mace = std::make_unique<MACE>(file);
    std::vector<double> H1, H1_adj;
    const double r_cut_squared = mace->r_cut * mace->r_cut;
    const int comm_forward = mace->num_LM * mace->num_channels;
    auto iter = std::find(mace->atomic_numbers.begin(), mace->atomic_numbers.end(), 8);
    (void)iter; (void)comm_forward;

    mace->node_energies.resize(num_nodes);
    std::fill(mace->node_energies.begin(), mace->node_energies.end(), 0.0);
    mace->node_forces.resize(xyz.size());
    std::fill(mace->node_forces.begin(), mace->node_forces.end(), 0.0);
    if (mace->has_zbl)
        mace->zbl.compute_ZBL(num_nodes, node_types, num_neigh, neigh_types, mace->atomic_numbers, r, xyz,
                              mace->node_energies, mace->node_forces);
    mace->compute_Y(xyz);
    mace->compute_R0(num_nodes, node_types, num_neigh, neigh_types, r);
    mace->compute_A0(num_nodes, node_types, num_neigh, neigh_types);
    mace->compute_A0_scaled(num_nodes, node_types, num_neigh, neigh_types, r);
    mace->compute_M0(num_nodes, node_types);
    mace->compute_H1(num_nodes);
    H1.resize(2 * num_nodes * mace->num_LM * mace->num_channels);
    for (int k = 0; k < mace->num_LM * mace->num_channels; ++k) H1[k] = mace->H1[k];
    mace->H1 = H1;
    mace->compute_R1(num_nodes, node_types, num_neigh, neigh_types, r);
    mace->compute_Phi1(num_nodes, num_neigh, neigh_j);
    mace->compute_A1(num_nodes);
    mace->compute_A1_scaled(num_nodes, node_types, num_neigh, neigh_types, r);
    mace->compute_M1(num_nodes, node_types);
    mace->compute_H2(num_nodes, node_types);
    mace->compute_readouts(num_nodes, node_types);
    mace->reverse_H2(num_nodes, node_types, false);
    mace->reverse_M1(num_nodes, node_types);
    mace->reverse_A1_scaled(num_nodes, node_types, num_neigh, neigh_types, xyz, r, false);
    mace->reverse_A1(num_nodes);
    mace->reverse_Phi1(num_nodes, num_neigh, neigh_j, xyz, r, false, false);
    H1_adj = mace->H1_adj;
    mace->H1_adj = H1_adj;
    mace->reverse_H1(num_nodes);
    mace->reverse_M0(num_nodes, node_types);
    mace->reverse_A0_scaled(num_nodes, node_types, num_neigh, neigh_types, xyz, r);
    mace->reverse_A0(num_nodes, node_types, num_neigh, neigh_types, xyz, r);
    mace->compute_node_energies_forces(num_nodes, node_types, num_neigh, neigh_j, neigh_types, xyz, r);
    double e = r_cut_squared;
    for (int ii = 0; ii < num_nodes; ++ii) e += mace->node_energies[ii];
    return e + mace->node_forces[0];
}
