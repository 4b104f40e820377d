// Header-only C++ face of the engine: `class MACE` with the public members and
// method signatures of the reference's class (libsymmetrix/source/mace.hpp:12-169),
// implemented over the C ABI of symmetrix_amd.h.  A caller written against the
// reference (the LAMMPS pair style, the pybind module) compiles against this
// header and links libsymmetrix_amd.so instead of libsymmetrix.
//
// Differences a caller can observe:
//   - intermediates live on the device; the public std::vector members
//     (node_energies, node_forces, H1, H1_adj) are host mirrors refreshed after
//     each call that writes them, and pushed with push_H1()/push_H1_adj() after
//     the caller overwrote them (the LAMMPS halo exchange,
//     pair_symmetrix_mace.cpp:462-471, 488-490);
//   - errors of the C ABI become std::invalid_argument (argument/range errors,
//     as libsymmetrix/source/cubic_spline.cpp:19-20) or std::runtime_error.
#pragma once

#include <span>
#include <stdexcept>
#include <string>
#include <vector>

#include "../symmetrix_amd.h"

class MACE {
public:
    explicit MACE(std::string filename, int precision = SMX_FP64)
    {
        check(smx_model_load(filename.c_str(), precision, &m_));
        check(smx_model_get_int(m_, "num_elements", &num_elements));
        check(smx_model_get_int(m_, "num_channels", &num_channels));
        check(smx_model_get_int(m_, "l_max", &l_max));
        check(smx_model_get_int(m_, "num_lm", &num_lm));
        check(smx_model_get_int(m_, "L_max", &L_max));
        check(smx_model_get_int(m_, "num_LM", &num_LM));
        check(smx_model_get_int(m_, "num_lme", &num_lme));
        check(smx_model_get_int(m_, "num_lelm1lm2", &num_lelm1lm2));
        int z = 0;
        check(smx_model_get_int(m_, "has_zbl", &z));
        has_zbl = z != 0;
        check(smx_model_get_double(m_, "r_cut", &r_cut));
        atomic_numbers.resize(num_elements);
        atomic_energies.resize(num_elements);
        int n = 0;
        check(smx_model_get_atomic_numbers(m_, atomic_numbers.data(), num_elements, &n));
        check(smx_model_get_atomic_energies(m_, atomic_energies.data(), num_elements, &n));
    }
    ~MACE() { smx_model_free(m_); }
    MACE(const MACE&) = delete;
    MACE& operator=(const MACE&) = delete;

    // Basic model information (mace.hpp:19-26)
    int num_elements = 0, num_channels = 0;
    double r_cut = 0.0;
    int l_max = 0, num_lm = 0, L_max = 0, num_LM = 0;
    int num_lelm1lm2 = 0, num_lme = 0;
    std::vector<int> atomic_numbers;
    std::vector<double> atomic_energies;
    bool has_zbl = false;

    // Host mirrors of the members callers read or overwrite (mace.hpp:29, 107)
    std::vector<double> node_energies, node_forces, H1, H1_adj;

    void compute_node_energies_forces(const int num_nodes, std::span<const int> node_types,
                                      std::span<const int> num_neigh, std::span<const int> neigh_indices,
                                      std::span<const int> neigh_types, std::span<const double> xyz,
                                      std::span<const double> r)
    {
        check(smx_compute_node_energies_forces(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_indices.data(),
                                               neigh_types.data(), xyz.data(), r.data(), (long)r.size()));
        pull("node_energies", node_energies);
        pull("node_forces", node_forces);
    }
    // Ghost atoms as extra nodes that go through layer 0 only: the stage sequence of
    // PairSymmetrixMACE::compute_no_mpi_message_passing (pair_symmetrix_mace.cpp:660-698) as one call.
    // No counterpart among the reference's methods.
    void compute_node_energies_forces_ghosted(const int num_local_nodes, const int num_ghost_nodes,
                                              std::span<const int> node_types, std::span<const int> num_neigh,
                                              std::span<const int> neigh_indices, std::span<const int> neigh_types,
                                              std::span<const double> xyz, std::span<const double> r)
    {
        check(smx_compute_ghosted(m_, num_local_nodes, num_ghost_nodes, node_types.data(), num_neigh.data(),
                                  neigh_indices.data(), neigh_types.data(), xyz.data(), r.data(), (long)r.size()));
        pull("node_energies", node_energies);
        pull("node_forces", node_forces);
    }
    void compute_R0(const int num_nodes, std::span<const int> node_types, std::span<const int> num_neigh,
                    std::span<const int> neigh_types, std::span<const double> r)
    { check(smx_compute_R0(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), r.data(), (long)r.size())); }
    void compute_R1(const int num_nodes, std::span<const int> node_types, std::span<const int> num_neigh,
                    std::span<const int> neigh_types, std::span<const double> r)
    { check(smx_compute_R1(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), r.data(), (long)r.size())); }
    void compute_Y(std::span<const double> xyz) { check(smx_compute_Y(m_, xyz.data(), (long)xyz.size())); }
    void compute_A0(const int num_nodes, std::span<const int> node_types, std::span<const int> num_neigh,
                    std::span<const int> neigh_types)
    { check(smx_compute_A0(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), (long)neigh_types.size())); }
    void reverse_A0(const int num_nodes, std::span<const int> node_types, std::span<const int> num_neigh,
                    std::span<const int> neigh_types, std::span<const double> xyz, std::span<const double> r)
    {
        check(smx_reverse_A0(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), xyz.data(), r.data(), (long)r.size()));
        pull("node_forces", node_forces);
    }
    // density normalisation: no-ops for models without it (mace.cpp:280, 307, 688, 716)
    void compute_A0_scaled(const int num_nodes, std::span<const int> node_types, std::span<const int> num_neigh,
                           std::span<const int> neigh_types, std::span<const double> r)
    {
        check(smx_compute_A0_scaled(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), r.data(), (long)r.size()));
    }
    void reverse_A0_scaled(const int num_nodes, std::span<const int> node_types, std::span<const int> num_neigh,
                           std::span<const int> neigh_types, std::span<const double> xyz, std::span<const double> r)
    {
        check(smx_reverse_A0_scaled(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), xyz.data(), r.data(), (long)r.size()));
        pull("node_forces", node_forces);
    }
    void compute_A1_scaled(const int num_nodes, std::span<const int> node_types, std::span<const int> num_neigh,
                           std::span<const int> neigh_types, std::span<const double> r)
    {
        check(smx_compute_A1_scaled(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), r.data(), (long)r.size()));
    }
    void reverse_A1_scaled(const int num_nodes, std::span<const int> node_types, std::span<const int> num_neigh,
                           std::span<const int> neigh_types, std::span<const double> xyz, std::span<const double> r,
                           bool zero_dxyz = true)
    {
        check(smx_reverse_A1_scaled(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), xyz.data(), r.data(), (long)r.size(), zero_dxyz ? 1 : 0));
        pull("node_forces", node_forces);
    }
    void compute_M0(const int num_nodes, std::span<const int> node_types) { check(smx_compute_M0(m_, num_nodes, node_types.data())); }
    void reverse_M0(const int num_nodes, std::span<const int> node_types) { check(smx_reverse_M0(m_, num_nodes, node_types.data())); }
    void compute_H1(const int num_nodes) { check(smx_compute_H1(m_, num_nodes)); pull("H1", H1); }
    void reverse_H1(const int num_nodes) { check(smx_reverse_H1(m_, num_nodes)); }
    void compute_Phi1(const int num_nodes, std::span<const int> num_neigh, std::span<const int> neigh_indices)
    { check(smx_compute_Phi1(m_, num_nodes, num_neigh.data(), neigh_indices.data(), (long)neigh_indices.size())); }
    void reverse_Phi1(const int num_nodes, std::span<const int> num_neigh, std::span<const int> neigh_indices,
                      std::span<const double> xyz, std::span<const double> r, bool zero_dxyz = true, bool zero_H1_adj = true)
    {
        check(smx_reverse_Phi1(m_, num_nodes, num_neigh.data(), neigh_indices.data(), xyz.data(), r.data(), (long)r.size(),
                               zero_dxyz, zero_H1_adj));
        pull("node_forces", node_forces);
        pull("H1_adj", H1_adj);
    }
    void compute_A1(const int num_nodes) { check(smx_compute_A1(m_, num_nodes)); }
    void reverse_A1(const int num_nodes) { check(smx_reverse_A1(m_, num_nodes)); }
    void compute_M1(const int num_nodes, std::span<const int> node_types) { check(smx_compute_M1(m_, num_nodes, node_types.data())); }
    void reverse_M1(const int num_nodes, std::span<const int> node_types) { check(smx_reverse_M1(m_, num_nodes, node_types.data())); }
    void compute_H2(const int num_nodes, std::span<const int> node_types) { check(smx_compute_H2(m_, num_nodes, node_types.data())); }
    void reverse_H2(const int num_nodes, std::span<const int> node_types, bool zero_H1_adj = true)
    { check(smx_reverse_H2(m_, num_nodes, node_types.data(), zero_H1_adj)); pull("H1_adj", H1_adj); }
    void compute_readouts(const int num_nodes, std::span<const int> node_types)
    {
        check(smx_compute_readouts(m_, num_nodes, node_types.data()));
        pull("node_energies", node_energies);
        pull("H1_adj", H1_adj);
    }

    // after the caller overwrote a mirror (halo exchange), send it to the device
    void push_H1() { check(smx_set_array(m_, "H1", H1.data(), (long)H1.size())); }
    void push_H1_adj() { check(smx_set_array(m_, "H1_adj", H1_adj.data(), (long)H1_adj.size())); }
    void push_node_energies() { check(smx_set_array(m_, "node_energies", node_energies.data(), (long)node_energies.size())); }
    void push_node_forces() { check(smx_set_array(m_, "node_forces", node_forces.data(), (long)node_forces.size())); }
    std::vector<double> get(const char* name) { std::vector<double> v; pull(name, v); return v; }
    void set(const char* name, std::span<const double> v) { check(smx_set_array(m_, name, v.data(), (long)v.size())); }
    smx_model* handle() { return m_; }

private:
    smx_model* m_ = nullptr;
    void pull(const char* name, std::vector<double>& v)
    {
        long n = 0;
        check(smx_get_array(m_, name, nullptr, 0, &n));
        v.resize((size_t)n);
        if (n) check(smx_get_array(m_, name, v.data(), n, &n));
    }
    static void check(int code)
    {
        if (code == SMX_OK) return;
        const std::string msg = smx_last_error();
        if (code == SMX_EINVAL || code == SMX_ERANGE) throw std::invalid_argument(msg);
        throw std::runtime_error(msg);
    }
};
