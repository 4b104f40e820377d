// Header-only C++ face of the engine: `class MACE` with the public members and
// method signatures of the reference's class (libsymmetrix/source/mace.hpp:12-169),
// implemented over the C ABI of symmetrix_amd.h.  A caller written against the
// reference (the LAMMPS pair style, the pybind module) compiles against this
// header and links libsymmetrix_amd.so instead of libsymmetrix.
//
// Differences a caller can observe:
//   - intermediates live on the device.  The public members the reference's
//     callers read and overwrite in place (node_energies, node_forces, H1,
//     H1_adj; pair_symmetrix/pair_symmetrix_mace.cpp:444-471, 488-490, 506-520)
//     are `Mirror` objects with the std::vector<double> operations those callers
//     use.  A mirror copies from the device the first time the host touches it
//     after a stage wrote it, and to the device before the next stage that reads
//     it if the host may have written it in between; stages that run back to
//     back move nothing over PCIe;
//   - `zbl.compute_ZBL(...)` (libsymmetrix/source/zbl.hpp:26-34) runs on the
//     device and adds to the model's own node_energies / node_forces; spans that
//     are not those two members are copied in and out;
//   - errors of the C ABI become std::invalid_argument (argument/range errors,
//     as libsymmetrix/source/cubic_spline.cpp:19-20) or std::runtime_error.
#pragma once

#include <algorithm>
#include <cstddef>
#include <initializer_list>
#include <span>
#include <stdexcept>
#include <string>
#include <vector>

#include "../symmetrix_amd.h"

namespace symmetrix_amd {

inline void check(int code)
{
    if (code == SMX_OK) return;
    const std::string msg = smx_last_error();
    if (code == SMX_EINVAL || code == SMX_ERANGE) throw std::invalid_argument(msg);
    throw std::runtime_error(msg);
}

// Host view of one device array of the model.  `host_valid`: the host copy holds the latest
// values; `dev_valid`: the device copy does.  Any access through a non-const member function
// may be a write, so it invalidates the device copy.
class Mirror {
public:
    using value_type = double;
    using iterator = double*;
    using const_iterator = const double*;

    Mirror(smx_model* const* model, const char* name) : model_(model), name_(name) {}
    Mirror(const Mirror&) = delete;
    Mirror& operator=(const Mirror&) = delete;

    std::size_t size() const { pull(); return h_.size(); }
    bool empty() const { return size() == 0; }
    void resize(std::size_t n) { pull(); h_.resize(n); dev_valid_ = false; }
    void resize(std::size_t n, double v) { pull(); h_.resize(n, v); dev_valid_ = false; }
    void assign(std::size_t n, double v) { h_.assign(n, v); host_valid_ = true; dev_valid_ = false; }
    double* data() { touch(); return h_.data(); }
    const double* data() const { pull(); return h_.data(); }
    iterator begin() { touch(); return h_.data(); }
    iterator end() { touch(); return h_.data() + h_.size(); }
    const_iterator begin() const { pull(); return h_.data(); }
    const_iterator end() const { pull(); return h_.data() + h_.size(); }
    double& operator[](std::size_t i) { touch(); return h_[i]; }
    const double& operator[](std::size_t i) const { pull(); return h_[i]; }
    Mirror& operator=(const std::vector<double>& v) { h_ = v; host_valid_ = true; dev_valid_ = false; return *this; }
    Mirror& operator=(std::vector<double>&& v) { h_ = std::move(v); host_valid_ = true; dev_valid_ = false; return *this; }
    operator const std::vector<double>&() const { pull(); return h_; }

    // ---- used by class MACE and ZBL
    // make the device copy current (before a stage that reads it)
    void to_device()
    {
        if (dev_valid_) return;
        const bool zeros = std::all_of(h_.begin(), h_.end(), [](double x) { return x == 0.0; });
        if (zeros) check(smx_fill_array(*model_, name_, (long)h_.size(), 0.0));
        else check(smx_set_array(*model_, name_, h_.data(), (long)h_.size()));
        dev_valid_ = true;
    }
    // a stage wrote the device copy
    void device_wrote() { dev_valid_ = true; host_valid_ = false; }
    const double* host_address() const { return h_.data(); }

private:
    void pull() const
    {
        if (host_valid_) return;
        long n = 0;
        check(smx_get_array(*model_, name_, nullptr, 0, &n));
        h_.resize((std::size_t)n);
        if (n) check(smx_get_array(*model_, name_, h_.data(), n, &n));
        host_valid_ = true;
    }
    void touch() { pull(); dev_valid_ = false; }

    smx_model* const* model_;
    const char* name_;
    mutable std::vector<double> h_;
    mutable bool host_valid_ = true;
    bool dev_valid_ = true;
};

}  // namespace symmetrix_amd

class MACE;

// The `zbl` member of the reference class (libsymmetrix/source/mace.hpp:39) with the one method
// its callers use.
class ZBL {
public:
    explicit ZBL(MACE* owner) : owner_(owner) {}
    inline void compute_ZBL(const int num_nodes, std::span<const int> node_types, std::span<const int> num_neigh,
                            std::span<const int> neigh_types, std::span<const int> atomic_numbers,
                            std::span<const double> r, std::span<const double> xyz, std::span<double> node_energies,
                            std::span<double> node_forces);

private:
    MACE* owner_;
};

class MACE {
public:
    using Mirror = symmetrix_amd::Mirror;

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
    ZBL zbl{this};

    // The members callers read or overwrite (mace.hpp:29, 107)
    Mirror node_energies{&m_, "node_energies"}, node_forces{&m_, "node_forces"}, H1{&m_, "H1"}, H1_adj{&m_, "H1_adj"};

    void compute_node_energies_forces(const int num_nodes, std::span<const int> node_types,
                                      std::span<const int> num_neigh, std::span<const int> neigh_indices,
                                      std::span<const int> neigh_types, std::span<const double> xyz,
                                      std::span<const double> r)
    {
        check(smx_compute_node_energies_forces(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_indices.data(),
                                               neigh_types.data(), xyz.data(), r.data(), (long)r.size()));
        wrote({&node_energies, &node_forces, &H1, &H1_adj});
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
        wrote({&node_energies, &node_forces, &H1, &H1_adj});
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
        reads({&node_forces});
        check(smx_reverse_A0(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), xyz.data(), r.data(), (long)r.size()));
        wrote({&node_forces});
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
        reads({&node_forces});
        check(smx_reverse_A0_scaled(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), xyz.data(), r.data(), (long)r.size()));
        wrote({&node_forces});
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
        reads({&node_forces});
        check(smx_reverse_A1_scaled(m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), xyz.data(), r.data(), (long)r.size(), zero_dxyz ? 1 : 0));
        wrote({&node_forces});
    }
    void compute_M0(const int num_nodes, std::span<const int> node_types) { check(smx_compute_M0(m_, num_nodes, node_types.data())); }
    void reverse_M0(const int num_nodes, std::span<const int> node_types) { check(smx_reverse_M0(m_, num_nodes, node_types.data())); }
    void compute_H1(const int num_nodes) { check(smx_compute_H1(m_, num_nodes)); wrote({&H1}); }
    void reverse_H1(const int num_nodes) { reads({&H1_adj}); check(smx_reverse_H1(m_, num_nodes)); }
    void compute_Phi1(const int num_nodes, std::span<const int> num_neigh, std::span<const int> neigh_indices)
    {
        reads({&H1});
        check(smx_compute_Phi1(m_, num_nodes, num_neigh.data(), neigh_indices.data(), (long)neigh_indices.size()));
    }
    void reverse_Phi1(const int num_nodes, std::span<const int> num_neigh, std::span<const int> neigh_indices,
                      std::span<const double> xyz, std::span<const double> r, bool zero_dxyz = true, bool zero_H1_adj = true)
    {
        reads({&H1, &node_forces, &H1_adj});
        check(smx_reverse_Phi1(m_, num_nodes, num_neigh.data(), neigh_indices.data(), xyz.data(), r.data(), (long)r.size(),
                               zero_dxyz, zero_H1_adj));
        wrote({&node_forces, &H1_adj});
    }
    void compute_A1(const int num_nodes) { check(smx_compute_A1(m_, num_nodes)); }
    void reverse_A1(const int num_nodes) { check(smx_reverse_A1(m_, num_nodes)); }
    void compute_M1(const int num_nodes, std::span<const int> node_types) { check(smx_compute_M1(m_, num_nodes, node_types.data())); }
    void reverse_M1(const int num_nodes, std::span<const int> node_types) { check(smx_reverse_M1(m_, num_nodes, node_types.data())); }
    void compute_H2(const int num_nodes, std::span<const int> node_types)
    { reads({&H1}); check(smx_compute_H2(m_, num_nodes, node_types.data())); }
    void reverse_H2(const int num_nodes, std::span<const int> node_types, bool zero_H1_adj = true)
    {
        reads({&H1, &H1_adj});
        check(smx_reverse_H2(m_, num_nodes, node_types.data(), zero_H1_adj));
        wrote({&H1_adj});
    }
    void compute_readouts(const int num_nodes, std::span<const int> node_types)
    {
        reads({&H1, &node_energies});
        check(smx_compute_readouts(m_, num_nodes, node_types.data()));
        wrote({&node_energies, &H1_adj});
    }

    // any other named intermediate (the def_readwrite members of the pybind class, symmetrix/source/cpp/mace.cpp:14-34)
    std::vector<double> get(const char* name)
    {
        reads({&node_energies, &node_forces, &H1, &H1_adj});
        std::vector<double> v;
        long n = 0;
        check(smx_get_array(m_, name, nullptr, 0, &n));
        v.resize((size_t)n);
        if (n) check(smx_get_array(m_, name, v.data(), n, &n));
        return v;
    }
    void set(const char* name, std::span<const double> v)
    {
        reads({&node_energies, &node_forces, &H1, &H1_adj});
        check(smx_set_array(m_, name, v.data(), (long)v.size()));
        wrote({&node_energies, &node_forces, &H1, &H1_adj});
    }
    // device copies of the four members made current (before a raw C-ABI call on handle())
    void flush() { reads({&node_energies, &node_forces, &H1, &H1_adj}); }
    smx_model* handle() { return m_; }

private:
    friend class ZBL;
    smx_model* m_ = nullptr;
    static void check(int code) { symmetrix_amd::check(code); }
    static void reads(std::initializer_list<Mirror*> l) { for (Mirror* m : l) m->to_device(); }
    static void wrote(std::initializer_list<Mirror*> l) { for (Mirror* m : l) m->device_wrote(); }
};

inline void ZBL::compute_ZBL(const int num_nodes, std::span<const int> node_types, std::span<const int> num_neigh,
                             std::span<const int> neigh_types, std::span<const int> atomic_numbers,
                             std::span<const double> r, std::span<const double> xyz, std::span<double> node_energies,
                             std::span<double> node_forces)
{
    MACE& o = *owner_;
    if (!o.has_zbl) throw std::invalid_argument("compute_ZBL called on a model without ZBL (has_zbl is false)");
    if (atomic_numbers.size() != o.atomic_numbers.size() ||
        !std::equal(atomic_numbers.begin(), atomic_numbers.end(), o.atomic_numbers.begin()))
        throw std::invalid_argument("compute_ZBL: atomic_numbers must be the model's own species table");
    if (node_energies.size() < (std::size_t)num_nodes || node_forces.size() < xyz.size() || xyz.size() != 3 * r.size())
        throw std::invalid_argument("compute_ZBL: output spans shorter than the node or edge count");
    const bool own = node_energies.data() == o.node_energies.host_address() && node_forces.data() == o.node_forces.host_address();
    if (!own) {
        o.node_energies = std::vector<double>(node_energies.begin(), node_energies.end());
        o.node_forces = std::vector<double>(node_forces.begin(), node_forces.end());
    }
    MACE::reads({&o.node_energies, &o.node_forces});
    MACE::check(smx_compute_ZBL(o.m_, num_nodes, node_types.data(), num_neigh.data(), neigh_types.data(), r.data(),
                                xyz.data(), (long)r.size()));
    MACE::wrote({&o.node_energies, &o.node_forces});
    if (!own) {
        const symmetrix_amd::Mirror& e = o.node_energies;
        const symmetrix_amd::Mirror& f = o.node_forces;
        std::copy(e.begin(), e.begin() + std::min(e.size(), node_energies.size()), node_energies.begin());
        std::copy(f.begin(), f.begin() + std::min(f.size(), node_forces.size()), node_forces.begin());
    }
}
