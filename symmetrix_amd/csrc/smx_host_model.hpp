// Host-side representation of a symmetrix JSON model, prepared for upload.
//
// Follows MACE::load_from_json (libsymmetrix/source/mace.cpp:905-1030) key by
// key.  Differences from the reference's in-memory form, all exact:
//   - identical radial tables of different species pairs are stored once
//     (plain MACE has a species-independent radial network, so every pair of
//     the file usually carries the same numbers);
//   - the symmetric-contraction polynomials are kept as sorted monomial rows
//     (degree <= 3) instead of one product graph per (species, LM, channel):
//     the graph of multivariate_polynomial.cpp:10-101 depends only on the
//     monomial list, and a polynomial's value does not depend on the order of
//     its products.
#pragma once

#include <string>
#include <vector>

namespace smx {

// One polynomial family P[type][k](x_0..x_15): monomials grouped in rows that
// share their first two factors.  Index 16 denotes the constant 1, so that a
// monomial (a) is stored as (16,16,a) and (a,b) as (16,a,b).
constexpr int POLY_GROUPS = 4;         // wavefront groups of the contraction kernel that share one atom group
constexpr int POLY_SPARE_CHUNKS = 2;   // the kernel reads entries this many chunks ahead
struct PolySpec {
    int num_entries = 0;                         // distinct monomials
    std::vector<int> row_i0, row_i1, row_start;  // row_start has num_rows+1 entries
    std::vector<int> entry_var;                  // third factor of each entry
    std::vector<double> coef;                    // [T][num_entries][K]
    // The same polynomial seen from each variable v: dP/dx_v = sum over the
    // entries of list v of coef[mono] * x[fa] * x[fb] (a monomial appears once per
    // occurrence of v in it).  The first list_nfirst[v] entries of list v are the
    // monomials whose first factor is v, so P = sum_v x_v * (their partial sum).
    std::vector<int> list_start;                 // [17]
    std::vector<int> list_nfirst;                // [16]
    std::vector<int> list_fa, list_fb, list_mono;
    // Device form of the lists: entries packed as mono | fa << 16 | fb << 24, each
    // half-list (first-factor entries of v, then the rest of v) padded to a
    // multiple of four with entries that point at an all-zero coefficient row
    // (index num_entries), plus spare chunks at the end for the prefetch.  The
    // variables follow each other in the order v = g, g + POLY_GROUPS, ... for
    // g = 0 .. POLY_GROUPS-1, so that each group's chunks are contiguous.
    std::vector<int> packed;                     // [4 * (total chunks + POLY_SPARE_CHUNKS)]
    std::vector<int> chunks;                     // [32]: chunks of (v, first part), (v, rest), same order
    // The same coefficients laid out for the compile-time monomial table `table` of the standard product basis
    // (smx_poly_tables.inc): [T][table length][K], zero where the file has no such monomial; table = -1 when the
    // file holds a monomial outside the table (the general kernel then runs).
    int table = -1;
    std::vector<double> table_coef;
};

struct HostModel {
    int T = 0, K = 0, l_max = 0, num_lm = 0, L_max = 0, num_LM = 0;
    double r_cut = 0.0;
    std::vector<int> atomic_numbers;
    std::vector<double> atomic_energies;

    bool has_zbl = false;
    double zbl_a_exp = 0, zbl_a_prefactor = 0;
    std::vector<double> zbl_c, zbl_covalent_radii;
    int zbl_p = 0;

    // radial spline sets: coefficient tables [(nodes-1)][4][nspl] per unique table
    double spl_h = 0.0;
    int spl_nodes = 0, num_pairs = 0;
    int nspl0 = 0, nspl1 = 0;
    std::vector<int> pair_table0, pair_table1;       // [num_pairs] -> unique table
    std::vector<std::vector<double>> tables0, tables1;

    std::vector<double> H0_weights;                  // [T][K]
    std::vector<double> A0_weights;                  // [T][l_max+1][K][K]
    bool A0_scaled = false, A1_scaled = false;
    double A0_spline_h = 0, A1_spline_h = 0;
    int A0_spline_nodes = 0, A1_spline_nodes = 0;
    std::vector<double> A0_spline_c, A1_spline_c;    // [pair][nodes-1][4]

    std::vector<PolySpec> P0;                        // [num_LM]
    PolySpec P1;

    std::vector<double> H1_weights;                  // [L_max+1][K][K]

    int num_paths = 0, num_lme = 0, num_lelm1lm2 = 0;
    std::vector<int> Phi1_l, Phi1_l1, Phi1_l2, Phi1_lme, Phi1_lelm1lm2;
    std::vector<double> Phi1_cg;
    std::vector<int> num_e;                          // [l_max+1]
    // coupling entries regrouped for the kernels: B[b] = sum C * Y[lm1] with
    // b = boff(path) + m*(2*l2+1) + m2
    int num_B = 0;
    std::vector<int> B_start, B_lm1;
    std::vector<double> B_c;

    std::vector<std::vector<double>> A1_weights;     // [l] -> [num_e[l]*K][K]
    std::vector<double> H2_weights_for_H1;           // [T][K][K]
    std::vector<double> H2_weights_for_M1;           // [K][K]
    std::vector<double> readout_1_weights;           // [K]
    std::vector<double> readout_2_w1, readout_2_w2;  // [16][K], [16]
    double readout_2_scale = 1.0;
};

// Throws smx::JsonError (file problems) or std::runtime_error prefixed with
// "unsupported:" (models outside what the kernels implement).
HostModel load_host_model(const std::string& path);

}  // namespace smx
