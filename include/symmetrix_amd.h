/*
 * symmetrix_amd.h -- C ABI of the MI355X (gfx950) MACE energy+forces engine.
 *
 * Drop-in boundary for the hot path of wcwitt/symmetrix: everything the
 * reference's `class MACE` (libsymmetrix/source/mace.hpp:12-169) offers to its
 * three callers -- the pybind module (symmetrix/source/cpp/mace.cpp:12-243), the
 * LAMMPS pair style (pair_symmetrix/pair_symmetrix_mace.cpp:319-320, :444-495,
 * :662-698) and the ASE calculator (symmetrix/source/symmetrix/symmetrix_calc.py:
 * 72-102) -- is reachable through the functions below with plain pointers and
 * sizes.  `include/symmetrix_amd/mace.hpp` wraps them in a header-compatible
 * C++ `class MACE`; `symmetrix_amd/mace.py` wraps them for Python.
 *
 * Conventions
 *   - Every function returns 0 on success and a negative SMX_E* code on
 *     failure; smx_last_error() returns the message of the calling thread's
 *     last failure (the reference throws C++ exceptions instead,
 *     libsymmetrix/source/cubic_spline.cpp:19-20, mace.cpp:908-909).
 *   - Arrays named like the reference's members have the reference's layout
 *     (row-major, channel index fastest).  Host getters/setters always speak
 *     double, whatever precision the engine holds internally.
 *   - One model object is not re-entrant (as the reference's, whose scratch
 *     state lives in members): one thread at a time per model.
 *   - There is no CPU fallback: every compute entry point needs a gfx950
 *     device and fails with SMX_ENODEVICE without one.
 */
#ifndef SYMMETRIX_AMD_H
#define SYMMETRIX_AMD_H

#ifdef __cplusplus
extern "C" {
#endif

typedef struct smx_model smx_model;

enum {
    SMX_OK = 0,
    SMX_EINVAL = -1,    /* bad argument (null pointer, negative size, index out of range) */
    SMX_EFILE = -2,     /* model file missing, malformed JSON, missing or ill-typed key */
    SMX_EUNSUPPORTED = -3, /* model outside what the kernels implement (see message) */
    SMX_ENODEVICE = -4, /* no usable gfx950 device */
    SMX_EHIP = -5,      /* HIP runtime error (message carries hipGetErrorString) */
    SMX_ERANGE = -6,    /* spline argument out of range: r <= 0, r >= r_cut or not finite */
    SMX_ENOMEM = -7
};

/* smx_model_load flags */
enum {
    SMX_FP64 = 0,          /* everything in double, as the reference CPU path */
    SMX_FP32_FEATURES = 1  /* features, tables and weights in float; positions, H2,
                              readouts, energies and force sums in double (the split of
                              MACEKokkos<float>, libsymmetrix/source/mace_kokkos.hpp:34-181) */
};

const char* smx_last_error(void);

/* MACE::MACE(std::string) / MACE::load_from_json, mace.cpp:12-15, 905-1030.
 * Reads the symmetrix JSON model file and uploads tables and weights to the
 * current HIP device. */
int smx_model_load(const char* json_path, int flags, smx_model** out);
void smx_model_free(smx_model* m);

/* Public scalar members of class MACE, mace.hpp:19-26,115: keys "num_elements",
 * "num_channels", "l_max", "num_lm", "L_max", "num_LM", "has_zbl", "num_lme",
 * "num_lelm1lm2", "precision" (0/1); "r_cut".  Beyond the reference:
 * "num_radial_tables_0/1" (radial tables per layer) and "contraction_tables"
 * (bit 0 / bit 1 set when the symmetric contraction of layer 0 / layer 1 has all
 * its monomials inside the standard product basis and runs the kernel compiled
 * for it; a file with other monomials takes the general kernel). */
int smx_model_get_int(const smx_model* m, const char* key, int* out);
int smx_model_get_double(const smx_model* m, const char* key, double* out);
/* atomic_numbers[T], atomic_energies[T], mace.hpp:25-26.  *n receives the length. */
int smx_model_get_atomic_numbers(const smx_model* m, int* out, int cap, int* n);
int smx_model_get_atomic_energies(const smx_model* m, double* out, int cap, int* n);

/* MACE::compute_node_energies_forces, mace.cpp:17-64.  Host arrays, exactly the
 * reference's arguments plus explicit lengths: node_types[num_nodes],
 * num_neigh[num_nodes], neigh_indices[num_edges], neigh_types[num_edges],
 * xyz[3*num_edges] (x_j - x_i), r[num_edges].  Results stay on the device until
 * fetched with smx_get_array("node_energies" / "node_forces"). */
int smx_compute_node_energies_forces(smx_model* m, int num_nodes,
                                     const int* node_types, const int* num_neigh,
                                     const int* neigh_indices, const int* neigh_types,
                                     const double* xyz, const double* r, long num_edges);

/* Same computation with every array already resident in device memory and the
 * work enqueued on `stream` (a hipStream_t, or NULL for the default stream).
 * d_node_energies[num_nodes] and d_node_forces[3*num_edges] may be NULL, in
 * which case results are only kept inside the model.  Does not synchronise. */
int smx_compute_device(smx_model* m, int num_nodes,
                       const int* d_node_types, const int* d_num_neigh,
                       const int* d_neigh_indices, const int* d_neigh_types,
                       const double* d_xyz, const double* d_r, long num_edges,
                       double* d_node_energies, double* d_node_forces, void* stream);

/* The same computation for a caller that holds ghost atoms as extra nodes, the mode no_mpi_message_passing of the
 * pair style (pair_symmetrix_mace.cpp:557-748): the first num_local_nodes nodes are evaluated in full, the
 * num_ghost_nodes nodes after them go through layer 0 only (R0, A0, M0, H1 and their adjoints, :674-698), so that
 * neigh_indices of local receivers may point at ghost nodes.  Arrays are laid out as for
 * smx_compute_node_energies_forces over all num_local_nodes + num_ghost_nodes nodes, local nodes and their edges
 * first; neigh_indices of edges that belong to ghost receivers are not read.  Results: node_energies[num_local_nodes],
 * node_forces[3*num_edges] (ghost receivers' edges carry their layer-0 share).  The device variant needs the number of
 * edges of the local receivers as well, writes d_node_energies[num_local_nodes] and d_node_forces[3*num_edges] when
 * they are not NULL, and does not synchronise. */
int smx_compute_ghosted(smx_model* m, int num_local_nodes, int num_ghost_nodes, const int* node_types,
                        const int* num_neigh, const int* neigh_indices, const int* neigh_types, const double* xyz,
                        const double* r, long num_edges);
int smx_compute_ghosted_device(smx_model* m, int num_local_nodes, int num_ghost_nodes, const int* d_node_types,
                               const int* d_num_neigh, const int* d_neigh_indices, const int* d_neigh_types,
                               const double* d_xyz, const double* d_r, long num_edges, long num_local_edges,
                               double* d_node_energies, double* d_node_forces, void* stream);

/* Number of rows of H1 a following layer-1 call may index (ghost rows of the
 * LAMMPS modes, pair_symmetrix_mace.cpp:462-471, 674-698).  Defaults to the
 * num_nodes of the last compute_H1. */
int smx_set_num_H1_rows(smx_model* m, int rows);

/* Stage-level entry points, one per public method of class MACE
 * (mace.hpp:29-164).  Edge geometry is remembered from the last
 * smx_compute_Y (xyz) and smx_compute_R0/R1 (r, types), as the reference
 * remembers Y, R0 and R1. */
int smx_compute_Y(smx_model* m, const double* xyz, long n3);                             /* mace.cpp:118-148 */
int smx_compute_R0(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                   const int* neigh_types, const double* r, long num_edges);            /* mace.cpp:66-90 */
int smx_compute_R1(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                   const int* neigh_types, const double* r, long num_edges);            /* mace.cpp:92-116 */
int smx_compute_A0(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                   const int* neigh_types, long num_edges);                             /* mace.cpp:150-201 */
int smx_reverse_A0(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                   const int* neigh_types, const double* xyz, const double* r, long num_edges); /* mace.cpp:203-271 */
/* Density normalisation of the A-basis and its adjoint; no-ops for models with A0_scaled / A1_scaled false.
 * SMX_ERANGE ("Out of bounds in CubicSpline::evaluate.") where the reference throws std::invalid_argument. */
int smx_compute_A0_scaled(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                          const int* neigh_types, const double* r, long num_edges);     /* mace.cpp:273-297 */
int smx_reverse_A0_scaled(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                          const int* neigh_types, const double* xyz, const double* r, long num_edges); /* mace.cpp:299-346 */
int smx_compute_A1_scaled(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                          const int* neigh_types, const double* r, long num_edges);     /* mace.cpp:681-705 */
int smx_reverse_A1_scaled(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                          const int* neigh_types, const double* xyz, const double* r, long num_edges,
                          int zero_dxyz);                                               /* mace.cpp:707-757 */
int smx_compute_M0(smx_model* m, int num_nodes, const int* node_types);                 /* mace.cpp:348-370 */
int smx_reverse_M0(smx_model* m, int num_nodes, const int* node_types);                 /* mace.cpp:372-395 */
int smx_compute_H1(smx_model* m, int num_nodes);                                        /* mace.cpp:397-423 */
int smx_reverse_H1(smx_model* m, int num_nodes);                                        /* mace.cpp:425-451 */
int smx_compute_Phi1(smx_model* m, int num_nodes, const int* num_neigh,
                     const int* neigh_indices, long num_edges);                         /* mace.cpp:453-502 */
int smx_reverse_Phi1(smx_model* m, int num_nodes, const int* num_neigh, const int* neigh_indices,
                     const double* xyz, const double* r, long num_edges,
                     int zero_dxyz, int zero_H1_adj);                                   /* mace.cpp:504-605 */
int smx_compute_A1(smx_model* m, int num_nodes);                                        /* mace.cpp:607-642 */
int smx_reverse_A1(smx_model* m, int num_nodes);                                        /* mace.cpp:644-679 */
int smx_compute_M1(smx_model* m, int num_nodes, const int* node_types);                 /* mace.cpp:759-777 */
int smx_reverse_M1(smx_model* m, int num_nodes, const int* node_types);                 /* mace.cpp:779-794 */
int smx_compute_H2(smx_model* m, int num_nodes, const int* node_types);                 /* mace.cpp:796-832 */
int smx_reverse_H2(smx_model* m, int num_nodes, const int* node_types, int zero_H1_adj);/* mace.cpp:834-874 */
int smx_compute_readouts(smx_model* m, int num_nodes, const int* node_types);           /* mace.cpp:876-903 */
/* ZBL::compute_ZBL, libsymmetrix/source/zbl.hpp:26-34 / zbl.cpp:96-125, as the pair style calls it on
 * mace->zbl before the stage sequence (pair_symmetrix/pair_symmetrix_mace.cpp:449-452, 667-670): adds the pair
 * repulsion of every edge to the model's node_energies[num_nodes] and node_forces[3*num_edges] (the arrays of
 * smx_get_array / smx_set_array / smx_fill_array; entries beyond their present length start at zero).  The species
 * table is the model's own atomic_numbers.  A no-op for models with has_zbl false. */
int smx_compute_ZBL(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh, const int* neigh_types,
                    const double* r, const double* xyz, long num_edges);

/* Read/write access to the named intermediates, the def_readwrite members of
 * the pybind class (symmetrix/source/cpp/mace.cpp:14-34): "node_energies",
 * "node_forces", "A0", "A0_adj", "M0", "M0_adj", "H1", "H1_adj", "Phi1",
 * "Phi1_adj", "A1", "A1_adj", "M1", "M1_adj", "H2", "H2_adj", "H0_weights"
 * (num_elements * num_channels values), plus "Y", "Y_grad", "R0", "R1"
 * (read-only: evaluated on demand from the remembered geometry and never
 * stored, so assigning R0 / R1 is refused with SMX_EUNSUPPORTED where the
 * pybind class allows it), "M0_grad" and "M1_grad" (read-only).
 * smx_get_array copies min(cap, size) doubles to `out` and stores the full
 * size in *n; out may be NULL to query the size. */
int smx_get_array(smx_model* m, const char* name, double* out, long cap, long* n);
int smx_set_array(smx_model* m, const char* name, const double* in, long n);
/* A settable array sized to n entries that all hold `value`, without a transfer from the host: what
 * `v.resize(n); std::fill(v.begin(), v.end(), value)` does to a member of the reference class
 * (pair_symmetrix_mace.cpp:444-447). */
int smx_fill_array(smx_model* m, const char* name, long n, double value);

/* Upper bound in bytes (default 32 GiB) for the buffer that stages the per-edge adjoint messages of reverse_Phi1
 * (mace.cpp:579-604) in models with l <= 1 hidden features.  Longer edge lists are processed in receiver chunks that
 * reuse the buffer; results do not depend on the limit.  No counterpart in the reference, which holds no per-edge
 * staging. */
int smx_set_staging_limit(smx_model* m, long bytes);

/* Per-stage timing with HIP events on the stream the kernels run on.  When
 * enabled, every stage of the next compute is bracketed by events;
 * smx_get_stage_times synchronises and returns elapsed milliseconds per stage.
 * Stage names come back as a ';'-separated list from smx_stage_names. */
int smx_set_profiling(smx_model* m, int enabled);
const char* smx_stage_names(void);
int smx_get_stage_times(smx_model* m, float* ms, int cap, int* n);

/* Blocks until all work enqueued for this model has finished. */
int smx_synchronize(smx_model* m);

/* Caller-side helpers, device resident (counterparts of the force and virial
 * scatter of pair_symmetrix_mace.cpp:334-368 and symmetrix_calc.py:93-102):
 * atom_forces[num_atoms][3] = sum over edges of +f_ij on sender j and -f_ij on
 * receiver i; virial[6] = sum xyz (x) f_ij in LAMMPS order xx,yy,zz,xy,xz,yz.
 * receiver_atom/sender_atom map edge ends to atom rows; NULL receiver_atom
 * means the receiver of edge block i is atom i.  Uses the forces of the last
 * compute.  Outputs are host arrays. */
int smx_reduce_forces(smx_model* m, int num_atoms, const int* sender_atom, const int* receiver_atom,
                      double* atom_forces, double* virial);
/* The same with sender_atom a device array (e.g. neigh_indices of smx_nlist_arrays) and receiver i = atom i. */
int smx_reduce_forces_device(smx_model* m, int num_atoms, const int* d_sender_atom, double* atom_forces,
                             double* virial);

/* The reduction of smx_reduce_forces_device for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same
 * inputs (the forces of the model's last evaluation, d_sender_atom[num_edges] on the device, receiver i = atom i),
 * outputs in device memory (d_atom_forces[3*num_atoms], d_virial[6]; either may be NULL), work enqueued on `stream`
 * without synchronising.  The per-atom sender lists and the partial virial sums live in a fixed array of about
 * 20 MiB that every GPU holds from the first model load to the end of the process, so sizes beyond
 * SMX_NOALLOC_MAX_ATOMS atoms or SMX_NOALLOC_MAX_EDGES edges are refused with SMX_EINVAL, and calls that overlap on
 * one GPU race (all of them share that GPU's array).  `stream` must be the stream of the evaluation whose forces
 * are reduced, or be ordered after it by the caller (an event wait): the call reads the model's node_forces and
 * edge arrays without any ordering of its own.  The model's GPU must be the current device (SMX_EINVAL otherwise).
 * A sender index outside [0, num_atoms) cannot be reported without a synchronisation: the outputs are NaN then, as
 * they are after an evaluation that its input checks skipped.  Calls no hipMalloc / hipFree and no allocating
 * routine. */
#define SMX_NOALLOC_MAX_ATOMS 262144
#define SMX_NOALLOC_MAX_EDGES 4194304
int smx_reduce_forces_device_noalloc(smx_model* m, int num_atoms, const int* d_sender_atom, double* d_atom_forces,
                                     double* d_virial, void* stream);

/* Full neighbour list built on the device, counterpart of the edge construction of
 * pair_symmetrix_mace.cpp:246-315 (ghost images, r^2 < r_cut^2) and of the ASE caller's
 * neighbor_list('ijdD') (symmetrix_calc.py:77-83), in the canonical order of this library: receivers
 * ascending, senders ascending within a receiver, images of one sender in the order of the shift list.
 * The caller lists the periodic images to consider: shift_int[num_shifts][3] (integer cell shifts, in
 * lexicographic order; (0,0,0) marks the shift for which a pair i == j is no edge) and
 * shift_vec[num_shifts][3] = shift . cell in Cartesian coordinates (host arrays).  d_positions[num_atoms][3]
 * and d_types[num_atoms] (may be NULL) are device arrays.  Edge vectors are (x_j + shift) - x_i and
 * r = sqrt((d0*d0 + d1*d1) + d2*d2), every operation rounded once.  Pairs closer than r_list >= r_cut are
 * remembered (r_list - r_cut is the skin that smx_nlist_update relies on; the shift list must cover r_list); the
 * edges are those closer than r_cut.  The arrays stay on the device and belong to the list object until the next
 * build or update; their addresses can be handed to smx_compute_device. */
typedef struct smx_nlist smx_nlist;
smx_nlist* smx_nlist_create(void);
void smx_nlist_free(smx_nlist* nl);
int smx_nlist_build(smx_nlist* nl, int num_atoms, const double* d_positions, const int* d_types, int num_shifts,
                    const int* shift_int, const double* shift_vec, double r_list, double r_cut, void* stream,
                    long* num_edges);
/* Same list from new positions without a new search: the pairs found within r_list by the last build are
 * re-measured and those inside r_cut kept, in the same canonical order (the cutoff filter that the LAMMPS caller
 * applies to its skin list every step, pair_symmetrix_mace.cpp:287-315).  Equal to a fresh build at r_cut as long
 * as no pair outside r_list at build time has come inside r_cut since. */
int smx_nlist_update(smx_nlist* nl, const double* d_positions, const int* d_types, double r_cut, void* stream,
                     long* num_edges);
/* Variants for callers that hold positions and species in host memory (the ASE calculator,
 * symmetrix_calc.py:72-83): the list object keeps device copies (smx_nlist_inputs returns their addresses, to be
 * handed to smx_compute_device as node_types) and the calls synchronise.  An update reuses the species of the
 * last build. */
int smx_nlist_build_host(smx_nlist* nl, int num_atoms, const double* positions, const int* types, int num_shifts,
                         const int* shift_int, const double* shift_vec, double r_list, double r_cut, long* num_edges);
int smx_nlist_update_host(smx_nlist* nl, const double* positions, double r_cut, long* num_edges);
int smx_nlist_inputs(smx_nlist* nl, const double** d_positions, const int** d_types);
int smx_nlist_arrays(smx_nlist* nl, const int** num_neigh, const int** first_neigh, const int** neigh_indices,
                     const int** neigh_types, const int** neigh_shift, const double** xyz, const double** r);
int smx_nlist_copy_to_host(smx_nlist* nl, int* num_neigh, int* neigh_indices, int* neigh_types, int* neigh_shift,
                           double* xyz, double* r);

#ifdef __cplusplus
}
#endif
#endif
