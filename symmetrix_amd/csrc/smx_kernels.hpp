// Launch interface of the gfx950 kernels (definitions in smx_kernels_*.hip).
#pragma once

#include <hip/hip_runtime.h>

#include "smx_poly_shape.hpp"

namespace smx {

// ---------------------------------------------------------------------------
// Edge aggregation (forward) and its adjoint.  One templated pair of kernels
// serves layer 0 (MACE::compute_A0 / reverse_A0 without the channel-mixing
// linear, libsymmetrix/source/mace.cpp:158-178, 238-269) and layer 1
// (compute_Phi1 / reverse_Phi1, mace.cpp:453-605): per edge
//     out[i, lme, k] += R_path(lme)[k](r_ij) * sum_m2 B_ij[lme, m2] * H[g_ij, l2^2+m2, k]
// with B_ij[.,.] = sum_m1 C * Y_m1(r_ij) the Clebsch-Gordan-contracted
// harmonics of the edge, H the gathered sender row (H0_weights[type_j] for
// layer 0, H1[neigh_index] for layer 1) and R the radial spline set of the
// species pair.  Y, B and R are recomputed per edge inside the kernels and
// never stored.
template <typename F>
struct AggParams {
    int num_nodes;
    int K;
    const int* first_neigh;   // [num_nodes+1] CSR offsets of the receiver-sorted edge list
    const int* node_types;    // [num_nodes]
    const int* neigh_types;   // [E]
    const int* gather;        // [E] row of Hsrc per edge
    const double* xyz;        // [E][3]
    const double* r;          // [E]
    const F* Hsrc;            // [rows][NLM][K]
    const F* tab;             // [table][nodes-1][4][P*K]
    const F* tabK;            // the same numbers with the coefficients of a spline adjacent, [table][nodes-1][P][K][4] (general edge kernels)
    const int* pair_table;    // [T(T+1)/2] -> table
    int T;
    int spl_nodes;
    double spl_h;
    double spl_inv_h;         // 1 / spl_h
    const int* B_start;       // [NB+1] rows of the coupling list
    const int* B_lm1;
    const double* B_c;
    F* out;                   // fwd: [num_nodes][NE][K]
    const F* d_out;           // bwd: adjoint of out
    double* forces;           // bwd: [E][3]
    int accumulate_forces;    // bwd: add to forces instead of overwriting
    F* msg;                   // bwd: [E][NLM][K] adjoint message to the sender row, or null
    double* fpart;            // bwd: [channel groups][E][3] partial forces, needed when agg_bwd_groups() > 1
    long num_edges;
    int num_terms;            // entries of B_lm1 / B_c
    // bwd, general kernel only: receivers [node_begin, num_nodes) are processed and the message of edge e goes to
    // row e - msg_edge_begin of msg (edge lists too long for one staging buffer are taken in receiver chunks)
    int node_begin;
    long msg_edge_begin;
};

template <typename F> hipError_t launch_agg_fwd(int L_max_H, const AggParams<F>& p, hipStream_t s);
template <typename F> hipError_t launch_agg_bwd(int L_max_H, const AggParams<F>& p, hipStream_t s);
// number of channel groups launch_agg_bwd splits K into; with more than one, the forces come out as
// fpart[group][E][3] and launch_fpart_reduce adds them up
template <typename F> int agg_bwd_groups(int L_max_H, int K);

// Channel-slice variant of the same two stages for scalar hidden features
// (L_max = 0 path structure: output slot lm is fed by path l(lm) and harmonic lm
// only, with a per-slot coupling constant cdiag[lm]).  tabS is the radial table
// regrouped per slice: [slice][table][interval][W] with row content
// [4 coefficients][4 paths][CH channels] padded to W elements.
template <typename F>
struct SliceParams {
    AggParams<F> a;
    const F* tabS;
    const F* tabF;     // forward kernel of 32-byte slices: rows [4 paths][2 halves][4 lanes][16 bytes], or null
    int W;             // padded row length in elements
    int CH;            // channels per slice
    double cdiag[16];
    double* fpart;     // bwd: [slices][E][3] partial forces
    long E;
    int num_cus;
    const int* order;     // [num_nodes] receivers by decreasing degree: entry 4t+q is row q of task t
    int units_per_die, slot_lines, num_units, receiver_groups;   // set by the launchers: block -> (slice, receiver group)
    long fpart_carry;     // bwd, one lane per edge: edges [0, fpart_carry) add what fpart already holds (an earlier stage's partial forces)
    int edge_lanes;       // bwd: one lane per edge (tabS rows padded to slice_edge_row_elements, CH * sizeof(F) = 32)
};
// row length (elements) and LDS bytes of the adjoint kernel with one lane per edge
template <typename F> int slice_edge_row_elements();
template <typename F> size_t slice_edge_lds_bytes(int spl_nodes);
// padded row length W (elements) of the per-slice table for CH channels, 0 if the kernels cannot take that CH
template <typename F> int slice_row_elements(int CH);
template <typename F> hipError_t launch_slice_fwd(const SliceParams<F>& p, hipStream_t s);
template <typename F> hipError_t launch_slice_bwd(const SliceParams<F>& p, hipStream_t s);
// forces (+)= sum over slices of fpart, slices added in ascending order
// (`copy`, if not null, receives the same sums: the caller's output array of the whole-pipeline call;
// `guard`, if not null and raised, makes every force NaN instead: the evaluation was skipped)
hipError_t launch_fpart_reduce(long edges, long E, int nslices, const double* fpart, double* forces, int accumulate,
                               double* copy, hipStream_t s, const int* guard = nullptr);

// H1_adj[j] (+)= sum over edges with sender j of msg[e], in ascending edge order.
// H_adj[j] (+)= sum of msg[e - e_lo] over the edges e of sender j with e_lo <= e < e_hi, in ascending edge order
template <typename F>
hipError_t launch_sender_reduce(int rows, int width, const int* sstart, const int* slist, const F* msg, F* H_adj,
                                int zero_first, long e_lo, long e_hi, hipStream_t s);
// The same sum for rows of K scalar features, followed by M_adj[rows][K] = H_adj . W^T (W [K][K], row n holding
// the weights of input channel n: reverse_H1 of an L_max = 0 model) in the same launch; K as sender_reduce_linear_ok
bool sender_reduce_linear_ok(int K);
template <typename F>
hipError_t launch_sender_reduce_linear(int rows, int K, const int* sstart, const int* slist, const F* msg, F* H_adj,
                                       int zero_first, const F* W, F* M_adj, hipStream_t s);

// ---------------------------------------------------------------------------
// Neighbour list on the device (smx_kernels_nlist.hip)
struct NlGrid {
    double lo[3], hi[3];     // bounding box of the positions
    double inv_bs[3];        // 1 / bin size
    int nb[3];               // bins per axis
};
hipError_t launch_nl_bbox(const double* pos, int N, double* part, int nblocks, hipStream_t s);
hipError_t launch_nl_bins(const double* pos, int N, const NlGrid& g, int* atom_bin, int* bin_count, hipStream_t s);
hipError_t launch_nl_bin_fill(int N, const int* atom_bin, const int* bin_start, int* bin_cursor, int* bin_atoms,
                              hipStream_t s);
hipError_t launch_nl_search(bool fill, const double* pos, int N, const NlGrid& g, const int* bin_start,
                            const int* bin_atoms, int num_shifts, const double* shift_vec, int zero_shift,
                            double r_cut, int* count, const int* first, long long* keys, hipStream_t s);
hipError_t launch_nl_sort(int N, const int* cfirst, const long long* keys, long long* sorted, hipStream_t s);
hipError_t launch_nl_filter(bool emit, const double* pos, const int* types, int N, const int* cfirst,
                            const long long* sorted, int num_shifts, const double* shift_vec, const int* shift_int,
                            double r_cut, int* count, const int* first, int* neigh_indices, int* neigh_types,
                            int* neigh_shift, double* xyz, double* r, hipStream_t s);

// ---------------------------------------------------------------------------
// Pair terms of the edge length alone (smx_kernels_pair.hip)
struct ZblParams {
    int T;
    const double* a_pair;      // [T][T] screening length of the species pair
    const double* rmax_pair;   // [T][T] envelope radius: sum of the covalent radii
    const double* zz_pair;     // [T][T] Z_i * Z_j
    double c[4];
    int p;
};
struct PairSpline {
    const double* c;           // [pairs][nodes-1][4], unordered pairs (a <= b) row-major upper triangle
    double h;
    int nodes;
};
// node_energies[i] += sum_j V(r_ij), node_forces[ij] -= V'(r_ij) xyz_ij / r_ij      (zbl.cpp:96-125)
hipError_t launch_zbl(int N, const int* first_neigh, const int* node_types, const int* neigh_types, const double* xyz,
                      const double* r, const ZblParams& z, double* energies, double* forces, hipStream_t s);
// A[i] /= 1 + sum_j s(r_ij), divisor kept (mace.cpp:273-297, 681-705); bit 4 of *flags: r outside the spline
template <typename F>
hipError_t launch_scale_fwd(int N, const int* first_neigh, const int* node_types, const int* neigh_types, const double* r,
                            const PairSpline& sp, int T, F* A, int width, double* divisor, int* flags, hipStream_t s);
// adjoint of the above (mace.cpp:299-346, 707-757): forces += ..., A_adj /= divisor
template <typename F>
hipError_t launch_scale_bwd(int N, const int* first_neigh, const int* node_types, const int* neigh_types,
                            const double* xyz, const double* r, const PairSpline& sp, int T, const F* A, F* A_adj,
                            int width, const double* divisor, double* forces, int* flags, hipStream_t s);

// ---------------------------------------------------------------------------
// Integer list preparation
hipError_t launch_scan_exclusive(const int* in, int* out, int n, int* block_sums, hipStream_t s);  // out[n] = total
// order[N]: receivers by decreasing degree
hipError_t launch_degree_order(int N, const int* first_neigh, int* order, hipStream_t s);
// counters_are_zero: 0 = clear count and cursor first, 1 = they are zero, 2 = the histogram is already in count and
// rank[E] holds every entry's place inside its bucket (launch_node_lists_count);
// count and cursor are zero again when the launches have run
// Guard of a device-resident evaluation, carried by the last launch of the sender-list build: when the checks of
// this evaluation raised the status word, first_neigh[n_first] and tstart[n_tstart] are zeroed (no edges, no species
// groups: the kernels that follow then touch no unchecked index) and the status is ORed into the sticky word the
// host reads later.  Raised or not, the status is copied into the `live` word, which the kernels after this launch
// read (energies and forces become NaN); the status word itself is cleared again by the readout kernel of the same
// evaluation, after every reader of it has run, so that a replayed graph starts clean.  status == nullptr: no guard.
struct InputGuard {
    const int* status = nullptr;
    int* live = nullptr;
    int* sticky = nullptr;
    int* first_neigh = nullptr; int n_first = 0;
    int* tstart = nullptr; int n_tstart = 0;
};
// What launch_node_lists_count checks besides the sender rows when status is not null: species of nodes and edges,
// edge lengths inside (0, r_cut), no negative count, counts adding up to num_edges (all nodes) and to the key
// count (the first num_local_nodes nodes).  Bits: 1 = index or count, 2 = edge length.
struct InputChecks {
    int* status = nullptr;
    const int* neigh_types = nullptr;
    const double* r = nullptr;
    double r_cut = 0.0;
    long num_edges = 0;
    int num_local_nodes = 0;
};
hipError_t launch_sender_lists(const int* gather, int E, int rows, int* count, int* sstart, int* cursor,
                               int* slist, int* block_sums, int counters_are_zero, const int* rank, hipStream_t s,
                               const InputGuard& guard = InputGuard());
hipError_t launch_check_counts(const int* num_neigh, int N, const int* first_neigh, int num_local_nodes, long num_edges,
                               long num_local_edges, int* status, hipStream_t s);
// first_neigh, degree order, species groups and `zero_n` cleared counters in one single-block launch
// (N <= 65536; larger systems use the separate launches, where the extra launches do not matter)
hipError_t launch_node_lists(const int* num_neigh, int N, int* first_neigh, int* order, const int* node_types, int T,
                             int* tstart, int* perm, int* zero_p, long zero_n, hipStream_t s);
// launch_node_lists plus the sender histogram count[rows] of `key[n]` in the same launch, with rank[n] = the place
// each entry took in its bucket; the counters must be zero on entry (every sender-list build leaves them so)
hipError_t launch_node_lists_count(const int* num_neigh, int N, int* first_neigh, int* order, const int* node_types, int T,
                                   int* tstart, int* perm, const int* key, long n, int rows, int* count, int* rank,
                                   const InputChecks& chk, hipStream_t s);
hipError_t launch_type_groups(const int* node_types, int N, int T, int* tcount, int* tstart, int* cursor,
                              int* perm, int* block_sums, hipStream_t s);
// flags[0] |= 1 if any index is outside [0, limit)
hipError_t launch_check_range(const int* v, long n, int limit, int* flags, hipStream_t s);
hipError_t launch_check_r(const double* r, long n, double r_cut, int* flags, hipStream_t s);

// ---------------------------------------------------------------------------
// Symmetric contraction (MACE::compute_M0 / compute_M1, mace.cpp:348-370, 759-777):
// value and gradient of NP polynomials of the 16 A_lm of one channel.
template <typename F>
struct PolyParams {
    int num_nodes, K, NP;              // NP polynomials (num_LM for M0, 1 for M1)
    const F* A;                        // [N][16][K]
    F* M;                              // [N][NP][K]
    F* M_grad;                         // [N][NP][16][K]
    // per polynomial (device arrays of length NP): per-variable entry lists, packed
    // mono | fa << 16 | fb << 24 in chunks of four (padding entries address the
    // all-zero row `num_entries`), and the chunk counts [32] = (v, first part), (v, rest)
    const int4* const* packed;
    const int* const* chunks;
    const F* const* coef;              // coef[p]: [T][num_entries + 1][K]
    const int* num_entries;            // monomials per polynomial
    const int* perm; const int* tstart; int T;   // atoms grouped by species
    // Standard product basis: when every polynomial p of the launch has its monomials inside compile-time table p
    // (smx_poly_tables.inc), the coefficients as [T][channel blocks] slabs in the layout of poly_spec_shape and the
    // straight-line kernel runs; else null.
    const F* table_slabs;
    int num_cus;
    // with table_slabs only: 0 values and gradients; 1 values only (M_grad unused); 2 adjoint,
    // A_adj[N][16][K] = sum_p M_adj[N][NP][K] * dM_p/dA recomputed from A (M and M_grad unused)
    int mode;
    const F* M_adj;
    F* A_adj;
};

template <typename F> hipError_t launch_poly(const PolyParams<F>& p, hipStream_t s);
// the table_slabs branch of launch_poly (smx_kernels_poly.hip)
template <typename F> hipError_t launch_poly_spec(const PolyParams<F>& p, hipStream_t s);

// A_adj[i,lm,k] = sum_LM M_grad[i,LM,lm,k] * M_adj[i,LM,k]   (reverse_M0 / reverse_M1)
template <typename F>
hipError_t launch_poly_reverse(int N, int NP, int K, const F* M_grad, const F* M_adj, F* A_adj, hipStream_t s);

// ---------------------------------------------------------------------------
// Dense channel mixing on the matrix cores.  A launch holds up to four
// independent products (blockIdx.z), each
//   C[row(node,s)][n] (+)= sum_k A[row(node,s)][k] * W[type(node)][k][n]   (or W^T)
//                          (+ sum_k A2[node][k] * W2[type(node)][k][n] when A2 is set)
// rows are (node, s) with s < sub; row (node,s) of A starts at
// A + node*a_node_stride + a_off + s*a_sub_stride and is Kd long.
template <typename TA, typename TC, typename CT>
struct GemmProb {
    const TA* A; long a_node_stride, a_off, a_sub_stride;
    TC* C; long c_node_stride, c_off, c_sub_stride;
    const CT* W; long w_type_stride, w_off;   // w_type_stride 0: one matrix for all species
    int transW;              // 0: W block is [Kd][Nn]; 1: W block is [Nn][Kd]
    int accumulate;          // 1: C += ...
    int Kd, Nn, sub;         // inner size, output columns, rows per node
    // optional second product into the same rows (sub must be 1): row of A2 starts at A2 + node*a2_node_stride
    const TA* A2; long a2_node_stride;
    // optional per-node factor of the first operand: A[row(node,s)][k] * Ascale[node*ascale_node_stride + k]
    // (row-streaming kernel only; not together with A2)
    const TA* Ascale; long ascale_node_stride;
    const CT* W2; long w2_type_stride;
    int transW2, Kd2;
};
template <typename TA, typename TC, typename CT>
struct GemmParams {
    int num_nodes;
    const int* perm;         // [num_nodes] nodes grouped by species, or null when no weight depends on the species
    const int* tstart;       // [T+1]
    int T;
    int nprob;
    int vec_ok;              // set by launch_gemm: every offset and size is a multiple of four elements
    GemmProb<TA, TC, CT> prob[4];
};
template <typename TA, typename TC, typename CT>
hipError_t launch_gemm(const GemmParams<TA, TC, CT>& p, hipStream_t s);
// whether a product with inner size Kd, Nn output columns and elements of `elem` bytes can take Ascale
bool gemm_scaled_operand_ok(int Kd, int Nn, size_t elem);

// ---------------------------------------------------------------------------
// Readout tail (MACE::compute_readouts, mace.cpp:876-903) in one launch: node_energies[i] (+)= E0[type] +
// w1 . H1[i, l=0] + MLP_{K->16->1}(H2[i]) with W1[16][K], H2_adj = gradient of the network, H1_adj[rows][num_LM][K]
// seeded with w1 in the scalar block of the first N rows and zero elsewhere.  guard / guard_clear / guard_forces: as
// in TailParams below.
template <typename F>
hipError_t launch_readout_fused(int N, int rows, int K, int num_LM, const int* node_types, const double* atomic_energies,
                                const double* w1, const double* W1, const double* w2, double scale, const F* H1,
                                const double* H2, double* H2_adj, F* H1_adj, double* node_energies, int zero_energies,
                                double* energies_copy, const int* guard, int* guard_clear, double* guard_forces,
                                long guard_forces_n, hipStream_t s);
// H2 (mace.cpp:820-845), the readout tail and reverse_H2 (mace.cpp:847-874) in one launch; K a multiple of 16
// up to 128 (tail_fused_ok).  Atoms grouped by species (perm, tstart); H1_adj [rows][num_LM][K] is written
// whole (seed plus the adjoint of H2 in the scalar block, zero elsewhere), M1_adj [N][K] too.
template <typename F>
struct TailParams {
    int N, rows, K, num_LM, T;
    const int* perm; const int* tstart;
    const double* E0; const double* w1; const double* W1; const double* w2; double scale;
    const F* H1; const F* M1;
    const double* W_H1;      // [T][K][K]
    const double* W_M1;      // [K][K]
    double* H2; double* H2_adj; F* H1_adj; F* M1_adj;
    double* node_energies; int zero_energies; double* energies_copy;
    const int* guard;        // live status of a device-resident evaluation (or null): raised -> energies are NaN
    int* guard_clear;        // the word the input checks of the next evaluation raise (or null): cleared here
    double* guard_forces;    // raised guard: these guard_forces_n edge-force components become NaN as well (the
    long guard_forces_n;     // adjoint kernels of a skipped evaluation see no edges and write none)
};
bool tail_fused_ok(int K);
template <typename F> hipError_t launch_tail_fused(const TailParams<F>& p, hipStream_t s);
template <typename T> hipError_t launch_fill(T* p, long n, T v, hipStream_t s);
template <typename TS, typename TD> hipError_t launch_convert(const TS* src, TD* dst, long n, hipStream_t s);

// Y[E][16], Y_grad[E][3][16] as the reference stores them (mace.cpp:118-148); inspection only
hipError_t launch_sph_harm(const double* xyz, long E, double* Y, double* Y_grad, hipStream_t s);
// R[E][nspl] spline values (mace.cpp:66-116); inspection only
template <typename F>
hipError_t launch_radial(int N, const int* first_neigh, const int* node_types, const int* neigh_types,
                         const double* r, const F* tab, const int* pair_table, int T, int nodes, double h,
                         int nspl, double* R, hipStream_t s);

// atom_forces[j] += f_e, atom_forces[i] -= f_e in a fixed order per atom, virial sums
hipError_t launch_force_scatter(int num_atoms, const int* recv_start, const int* recv_list,
                                const int* send_start, const int* send_list, const double* forces,
                                double* atom_forces, hipStream_t s);
hipError_t launch_virial(long E, const double* xyz, const double* forces, double* partial, int nblocks,
                         hipStream_t s);

}  // namespace smx
