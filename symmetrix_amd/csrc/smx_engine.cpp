// Host orchestration and C ABI of the MACE energy+forces engine.
//
// Pipeline (the stage list of MACE::compute_node_energies_forces,
// libsymmetrix/source/mace.cpp:17-64), one HIP kernel or one batched MFMA
// launch per stage, all on one stream, nothing computed on the host:
//
//   prep        CSR offsets, sender lists, species groups        (integers only)
//   agg0_fwd    Phi0 = sum_j R0 Y H0                             mace.cpp:158-178
//   A0_lin      A0 = Phi0 . A0_weights[type][l]        (MFMA)    mace.cpp:180-199
//   M0          symmetric contraction + gradient                 mace.cpp:348-370
//   H1          H1 = M0 . H1_weights[l]                (MFMA)    mace.cpp:397-423
//   agg1_fwd    Phi1 = CG . sum_j R1 Y H1[j]                     mace.cpp:453-502
//   A1          A1 = Phi1 . A1_weights[l]              (MFMA)    mace.cpp:607-642
//   M1          symmetric contraction + gradient                 mace.cpp:759-777
//   H2          H2 = H1[l=0].W[type] + M1.W            (MFMA)    mace.cpp:796-832
//   readout     energies, H1_adj seed, H2_adj          (MFMA)    mace.cpp:876-903
//   rev_H2, rev_M1, rev_A1, agg1_bwd, sender_reduce, rev_H1, rev_M0,
//   rev_A0_lin, agg0_bwd                                         mace.cpp:54-63
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/symmetrix_amd.h"
#include "smx_host_model.hpp"
#include "smx_internal.hpp"
#include "smx_json.hpp"
#include "smx_kernels.hpp"
#include "smx_paths.hpp"

namespace smx {

struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};

static thread_local std::string g_last_error;

#define HIPCHK(expr)                                                                                   \
    do {                                                                                               \
        hipError_t e_ = (expr);                                                                        \
        if (e_ != hipSuccess)                                                                          \
            throw ::smx::Error(e_ == hipErrorOutOfMemory ? SMX_ENOMEM : SMX_EHIP,                      \
                        std::string(#expr) + ": " + hipGetErrorString(e_));                            \
    } while (0)

// growable device array with std::vector::resize semantics (contents kept, new tail zeroed)
template <typename T>
struct DVec {
    T* p = nullptr;
    size_t n = 0, cap = 0;
    ~DVec() { if (p) (void)hipFree(p); }
    DVec() = default;
    DVec(const DVec&) = delete;
    DVec& operator=(const DVec&) = delete;
    void reserve(size_t m, hipStream_t s, bool keep)
    {
        if (m <= cap) return;
        // headroom against regrowth when the edge count drifts: an eighth, a sixty-fourth for buffers beyond 1 GiB
        const size_t newcap = m + (m * sizeof(T) > ((size_t)1 << 30) ? m / 64 : m / 8) + 64;
        T* q = nullptr;
        if (p && !(keep && n)) {
            // nothing to carry over: release first, so that the two sizes never coexist
            HIPCHK(hipStreamSynchronize(s));
            HIPCHK(hipFree(p));
            p = nullptr; cap = 0; n = 0;
        }
        HIPCHK(hipMalloc(&q, newcap * sizeof(T)));
        if (p) {
            HIPCHK(hipMemcpyAsync(q, p, n * sizeof(T), hipMemcpyDeviceToDevice, s));
            HIPCHK(hipStreamSynchronize(s));
            HIPCHK(hipFree(p));
        }
        p = q;
        cap = newcap;
    }
    // size to m elements; previous contents are undefined afterwards
    void size_to(size_t m, hipStream_t s) { reserve(m ? m : 1, s, false); n = m; }
    // std::vector::resize
    void resize(size_t m, hipStream_t s)
    {
        reserve(m ? m : 1, s, true);
        if (m > n) HIPCHK(hipMemsetAsync(p + n, 0, (m - n) * sizeof(T), s));
        n = m;
    }
    void upload(const T* host, size_t m, hipStream_t s)
    {
        size_to(m, s);
        if (m) HIPCHK(hipMemcpyAsync(p, host, m * sizeof(T), hipMemcpyHostToDevice, s));
    }
};

template <typename T, typename S>
static void upload_as(DVec<T>& d, const std::vector<S>& h, hipStream_t s)
{
    std::vector<T> tmp(h.begin(), h.end());
    d.upload(tmp.data(), tmp.size(), s);
    HIPCHK(hipStreamSynchronize(s));  // tmp goes out of scope
}

static const char* kStageNames =
    "prep;agg0_fwd;A0_lin;M0;H1;agg1_fwd;A1;M1;H2;readout;rev_H2;rev_M1;rev_A1;agg1_bwd;sender_reduce;"
    "rev_H1;rev_M0;rev_A0_lin;agg0_bwd;force_sum1;force_sum0";
enum Stage { ST_PREP, ST_AGG0F, ST_A0LIN, ST_M0, ST_H1, ST_AGG1F, ST_A1, ST_M1, ST_H2, ST_READOUT, ST_REVH2,
             ST_REVM1, ST_REVA1, ST_AGG1B, ST_SRED, ST_REVH1, ST_REVM0, ST_REVA0LIN, ST_AGG0B, ST_FSUM1, ST_FSUM0, ST_COUNT };

struct EngineBase {
    virtual ~EngineBase()
    {
        for (int i = 0; i < ST_COUNT; ++i) {
            if (ev0[i]) (void)hipEventDestroy(ev0[i]);
            if (ev1[i]) (void)hipEventDestroy(ev1[i]);
        }
    }
    HostModel hm;
    int precision = 0;
    int poly_tables = 0;            // bit 0 / bit 1: layer 0 / layer 1 contraction runs the table-specialised kernel
    int contraction_tables() const { return poly_tables; }
    int device = 0;                 // ordinal of the GPU the model was loaded on
    hipStream_t stream = nullptr;   // stream of the current call
    bool profiling = false;
    hipEvent_t ev0[ST_COUNT] = {}, ev1[ST_COUNT] = {};
    bool ev_used[ST_COUNT] = {};
    int H1_rows_override = -1;
    size_t msg_limit_bytes = (size_t)32 << 30;   // staging buffer of the layer-1 adjoint messages

    virtual void compute(int N, const int* node_types, const int* num_neigh, const int* neigh_indices,
                         const int* neigh_types, const double* xyz, const double* r, long E, bool on_device,
                         double* d_energies, double* d_forces, int N_local, long E_local) = 0;
    virtual void stage(const char* name, int N, const int* node_types, const int* num_neigh,
                       const int* neigh_indices, const int* neigh_types, const double* xyz, const double* r,
                       long E, int flag_a, int flag_b) = 0;
    virtual void get_array(const char* name, double* out, long cap, long* n) = 0;
    virtual void set_array(const char* name, const double* in, long n) = 0;
    virtual void fill_array(const char* name, long n, double value) = 0;
    virtual void forces_view(ForcesView* v) = 0;
    virtual void check_device_status() = 0;
    virtual void reduce_forces(int num_atoms, const int* sender_atom, const int* receiver_atom,
                               double* atom_forces, double* virial, bool sender_on_device) = 0;

    void stage_begin(int st)
    {
        if (!profiling) return;
        if (!ev0[st]) { HIPCHK(hipEventCreate(&ev0[st])); HIPCHK(hipEventCreate(&ev1[st])); }
        HIPCHK(hipEventRecord(ev0[st], stream));
    }
    void stage_end(int st)
    {
        if (!profiling) return;
        HIPCHK(hipEventRecord(ev1[st], stream));
        ev_used[st] = true;
    }
};

template <typename F>
struct Engine : EngineBase {
    // ---- model on device
    DVec<F> tab0, tab1, tabK0, tabK1, H0, A0w, H1w, A1w;
    DVec<int> pair_table0, pair_table1;
    DVec<int> B0_start, B0_lm1, B1_start, B1_lm1;
    DVec<double> B0_c, B1_c;
    std::vector<long> A1w_off;   // per l
    // channel-slice tables (see smx_kernels_slice.hip); CH = 0 disables the path for that layer
    DVec<F> tabS0, tabS1;
    int slice_CH0 = 0, slice_CH1 = 0, slice_W = 0, num_cus = 0;
    // the same slices with the row padding of the adjoint kernel that gives every edge a lane of its own
    // (empty when the forward table already has that row length, or when the kernel does not apply)
    DVec<F> tabE0, tabE1;
    DVec<F> tabF0, tabF1;   // forward-kernel layout of the same slices (when a slice is 32 bytes of channels)
    bool edge_lanes = false;
    double cdiag1[16] = {};
    DVec<double> fpart;
    DVec<double> H2w_H1, H2w_M1, ro1, ro2_w1, ro2_w2, E0;
    struct DevPoly {
        DVec<int> packed, chunks;
        DVec<F> coef;
        int num_entries = 0;
    };
    std::vector<std::unique_ptr<DevPoly>> P0;
    DevPoly P1;
    // pointer tables for the polynomial kernel: [0..num_LM) = P0, then P1
    DVec<const int4*> pp_packed;
    DVec<const int*> pp_chunks;
    DVec<const F*> pp_coef;
    DVec<F> M0_slabs, M1_slabs;   // coefficients of the straight-line contraction kernel (poly_spec_shape layout)
    DVec<int> pp_nent;
    bool M0_tables = false, M1_tables = false;   // every polynomial of the layer maps onto its compile-time table

    // ---- geometry of the current edge list (device)
    DVec<int> g_node_types, g_num_neigh, g_neigh_indices, g_neigh_types;
    DVec<double> g_xyz, g_r;
    const int *node_types = nullptr, *num_neigh = nullptr, *neigh_indices = nullptr, *neigh_types = nullptr;
    const double *xyz = nullptr, *r = nullptr;
    long E = 0;
    long E1 = 0;   // leading edges whose receivers take part in layer 1 (all of them unless ghost nodes follow)
    int N_geo = 0;
    DVec<int> first_neigh, recv_order, scan_tmp, s_count, s_start, s_list, t_count, t_start, t_cursor, t_perm, flags;
    int sender_rows = 0;
    // pair terms: ZBL constants per species pair, density-normalisation splines, divisors of the last forward pass
    DVec<double> zbl_a, zbl_rmax, zbl_zz, A0spl, A1spl, div0, div1;
    ZblParams zbl_params() const
    {
        ZblParams z{};
        z.T = hm.T; z.a_pair = zbl_a.p; z.rmax_pair = zbl_rmax.p; z.zz_pair = zbl_zz.p;
        for (int q = 0; q < 4; ++q) z.c[q] = hm.zbl_c[q];
        z.p = hm.zbl_p;
        return z;
    }
    PairSpline scale_spline(int layer) const
    {
        PairSpline sp{};
        sp.c = layer == 0 ? A0spl.p : A1spl.p;
        sp.h = layer == 0 ? hm.A0_spline_h : hm.A1_spline_h;
        sp.nodes = layer == 0 ? hm.A0_spline_nodes : hm.A1_spline_nodes;
        return sp;
    }
    // caller's output arrays of the running whole-pipeline call; the kernel that forms the final values writes
    // them too and clears the pointer, otherwise a copy is enqueued at the end
    double* energies_copy = nullptr;
    double* forces_copy = nullptr;
    bool senders_counted = false;   // the sender histogram (and s_rank) was formed by the fused node-list launch
    DVec<int> s_rank;               // place of every edge inside its sender's bucket
    long counters_clean = 0;        // leading entries of s_count known to be zero

    // ---- state (mace.hpp members)
    DVec<F> Phi0, A0, A0_adj, M0, M0_grad, M0_adj, H1, H1_adj, Phi1, dPhi1, A1, A1_adj, M1, M1_grad, M1_adj, msg;
    DVec<double> H2, H2_adj, node_energies, node_forces, scratch_d;

    int K() const { return hm.K; }
    int NLM() const { return hm.num_LM; }
    int NE() const { return hm.num_lme; }

    explicit Engine(HostModel&& m, int prec)
    {
        hm = std::move(m);
        precision = prec;
        HIPCHK(hipGetDevice(&device));
        hipStream_t s = nullptr;
        auto cat = [](const std::vector<std::vector<double>>& t) {
            std::vector<double> out;
            for (auto& v : t) out.insert(out.end(), v.begin(), v.end());
            return out;
        };
        upload_as(tab0, cat(hm.tables0), s);
        upload_as(tab1, cat(hm.tables1), s);
        upload_as(pair_table0, hm.pair_table0, s);
        upload_as(pair_table1, hm.pair_table1, s);
        upload_as(H0, hm.H0_weights, s);
        upload_as(A0w, hm.A0_weights, s);
        upload_as(H1w, hm.H1_weights, s);
        {
            std::vector<double> all;
            for (auto& w : hm.A1_weights) { A1w_off.push_back((long)all.size()); all.insert(all.end(), w.begin(), w.end()); }
            upload_as(A1w, all, s);
        }
        build_slices(s);
        // the general edge kernels read the tables as [interval][path][channel][4 coefficients]: one load instruction
        // of a wavefront (one path, consecutive channels) then covers contiguous memory; layers served by the slice
        // kernels need no copy
        auto regroup = [&](const std::vector<std::vector<double>>& tables, int nspl, DVec<F>& dst) {
            const int R = hm.spl_nodes - 1, Kc = hm.K, Pn = nspl / Kc;
            std::vector<double> out((size_t)tables.size() * R * nspl * 4);
            size_t o = 0;
            for (auto& t : tables)
                for (int n = 0; n < R; ++n)
                    for (int pth = 0; pth < Pn; ++pth)
                        for (int k = 0; k < Kc; ++k)
                            for (int q = 0; q < 4; ++q) out[o++] = t[((size_t)n * 4 + q) * nspl + pth * Kc + k];
            upload_as(dst, out, s);
        };
        if (!slice_CH0) regroup(hm.tables0, hm.nspl0, tabK0);
        if (!slice_CH1) regroup(hm.tables1, hm.nspl1, tabK1);
        // layer 0 couples Y_lm straight into output slot lm
        {
            std::vector<int> st(17), lm(16);
            std::vector<double> c(16, 1.0);
            for (int q = 0; q < 16; ++q) { st[q] = q; lm[q] = q; }
            st[16] = 16;
            upload_as(B0_start, st, s); upload_as(B0_lm1, lm, s); upload_as(B0_c, c, s);
        }
        upload_as(B1_start, hm.B_start, s);
        upload_as(B1_lm1, hm.B_lm1, s);
        upload_as(B1_c, hm.B_c, s);
        upload_as(H2w_H1, hm.H2_weights_for_H1, s);
        upload_as(H2w_M1, hm.H2_weights_for_M1, s);
        upload_as(ro1, hm.readout_1_weights, s);
        upload_as(ro2_w1, hm.readout_2_w1, s);
        upload_as(ro2_w2, hm.readout_2_w2, s);
        upload_as(E0, hm.atomic_energies, s);
        if (hm.has_zbl) {
            // zbl.cpp:22-35: screening length and envelope radius of every ordered species pair
            const int T = hm.T;
            std::vector<double> a((size_t)T * T), rm((size_t)T * T), zz((size_t)T * T);
            for (int i = 0; i < T; ++i)
                for (int j = 0; j < T; ++j) {
                    const int Zi = hm.atomic_numbers[i], Zj = hm.atomic_numbers[j];
                    if (Zi < 0 || Zj < 0 || Zi >= (int)hm.zbl_covalent_radii.size() || Zj >= (int)hm.zbl_covalent_radii.size())
                        throw Error(SMX_EFILE, "model file: zbl_covalent_radii does not cover the atomic numbers of the model");
                    a[(size_t)i * T + j] = hm.zbl_a_prefactor * 0.529 / (std::pow((double)Zi, hm.zbl_a_exp) + std::pow((double)Zj, hm.zbl_a_exp));
                    rm[(size_t)i * T + j] = hm.zbl_covalent_radii[Zi] + hm.zbl_covalent_radii[Zj];
                    zz[(size_t)i * T + j] = (double)Zi * (double)Zj;
                }
            upload_as(zbl_a, a, s); upload_as(zbl_rmax, rm, s); upload_as(zbl_zz, zz, s);
        }
        if (hm.A0_scaled) upload_as(A0spl, hm.A0_spline_c, s);
        if (hm.A1_scaled) upload_as(A1spl, hm.A1_spline_c, s);
        auto up_poly = [&](DevPoly& d, const PolySpec& p) {
            upload_as(d.packed, p.packed, s); upload_as(d.chunks, p.chunks, s);
            upload_as(d.coef, p.coef, s);
            d.num_entries = p.num_entries;
        };
        std::vector<const int4*> vpk;
        std::vector<const int*> vch;
        std::vector<const F*> vco;
        std::vector<int> vne;
        auto reg = [&](DevPoly& d) {
            vpk.push_back(reinterpret_cast<const int4*>(d.packed.p)); vch.push_back(d.chunks.p);
            vco.push_back(d.coef.p); vne.push_back(d.num_entries);
        };
        for (int LM = 0; LM < hm.num_LM; ++LM) {
            P0.emplace_back(new DevPoly());
            up_poly(*P0.back(), hm.P0[LM]);
            reg(*P0.back());
        }
        up_poly(P1, hm.P1);
        reg(P1);
        pp_packed.upload(vpk.data(), vpk.size(), s); pp_chunks.upload(vch.data(), vch.size(), s);
        pp_coef.upload(vco.data(), vco.size(), s);
        pp_nent.upload(vne.data(), vne.size(), s);
        M0_tables = hm.num_LM == 1 || hm.num_LM == 4 || hm.num_LM == 9;
        for (int LM = 0; LM < hm.num_LM; ++LM) M0_tables = M0_tables && hm.P0[LM].table == LM;
        M1_tables = hm.P1.table == 0;
        M0_tables = M0_tables && poly_spec_shape((int)sizeof(F), hm.K, hm.num_LM).CB > 0;
        M1_tables = M1_tables && poly_spec_shape((int)sizeof(F), hm.K, 1).CB > 0;
        // slabs of the straight-line kernel: [species][channel block][monomial / V][CB][V]
        auto slabs = [&](DVec<F>& dst, const PolySpec* polys, int NP) {
            const PolySpecShape sh = poly_spec_shape((int)sizeof(F), hm.K, NP);
            constexpr int V = 16 / (int)sizeof(F);
            const size_t slab = sh.slab_bytes / sizeof(F);
            std::vector<F> h((size_t)hm.T * sh.kblocks * slab, F(0));
            for (int P = 0; P < NP; ++P) {
                const int tn = kPolyTableLen[polys[P].table], m0 = poly_spec_offset(P);
                for (int t = 0; t < hm.T; ++t)
                    for (int i = 0; i < tn; ++i)
                        for (int k = 0; k < hm.K; ++k) {
                            const int m = m0 + i, kb = k / sh.CB, kloc = k % sh.CB;
                            h[((size_t)t * sh.kblocks + kb) * slab + ((size_t)(m / V) * sh.CB + kloc) * V + m % V] =
                                (F)polys[P].table_coef[((size_t)t * tn + i) * hm.K + k];
                        }
            }
            dst.upload(h.data(), h.size(), s);
            HIPCHK(hipStreamSynchronize(s));   // h goes out of scope
        };
        if (num_cus == 0) {
            hipDeviceProp_t prop;
            HIPCHK(hipGetDeviceProperties(&prop, device));
            num_cus = prop.multiProcessorCount;
        }
        if (M0_tables) slabs(M0_slabs, hm.P0.data(), hm.num_LM);
        if (M1_tables) slabs(M1_slabs, &hm.P1, 1);
        poly_tables = (M0_tables ? 1 : 0) | (M1_tables ? 2 : 0);
        flags.resize(8, s);
        HIPCHK(hipStreamSynchronize(s));
    }

    // ---- input checks of device-resident evaluations.  flags[0]: host-array calls (read back at once);
    // flags[1]: sticky status of device-resident calls, read by the next synchronising call; flags[2]: the word the
    // checks of the running device-resident evaluation raise; flags[3]: its copy for the kernels after the list
    // preparation ("live": raised -> energies and forces are NaN).  The evaluation clears flags[2] again in its
    // readout launch, after the last reader, so every evaluation, eager or a replayed graph, starts from a clean word.
    long device_calls = 0;
    int* guard_status = nullptr;   // check word of the running evaluation (nullptr: host-array call, checked already)
    bool guard_clear_enqueued = false;   // ... and a launch that clears it again is in the stream
    const int* guard_live() const { return guard_status ? flags.p + 3 : nullptr; }
    InputGuard input_guard(int N)
    {
        InputGuard g;
        if (!guard_status) return g;
        g.status = guard_status;
        g.live = flags.p + 3;
        g.sticky = flags.p + 1;
        g.first_neigh = first_neigh.p; g.n_first = N + 1;
        g.tstart = t_start.p; g.n_tstart = hm.T + 1;
        return g;
    }
    void check_device_status() override
    {
        if (!device_calls) return;
        int f = 0;
        HIPCHK(hipMemcpyAsync(&f, flags.p + 1, sizeof(int), hipMemcpyDeviceToHost, stream));
        HIPCHK(hipStreamSynchronize(stream));
        if (!f) return;
        HIPCHK(launch_fill<int>(flags.p + 1, 1, 0, stream));
        if (f & 1)
            throw Error(SMX_EINVAL, "a device-resident evaluation was skipped: node_types / neigh_types / neigh_indices hold an "
                                    "index outside the model or the node range, or num_neigh does not add up to the number "
                                    "of edges (its node energies and forces are NaN)");
        throw Error(SMX_ERANGE, "a device-resident evaluation was skipped: an edge length lies outside (0, r_cut) "
                                "(its node energies and forces are NaN)");
    }

    // Regroup a radial table per channel slice, or return 0 when the slice path does not apply.
    int build_slice_table(const std::vector<std::vector<double>>& tables, int nspl, DVec<F>& dst, DVec<F>& edst, DVec<F>& fdst,
                          hipStream_t s)
    {
        // One radial table only (species-independent radial functions, as models without a distance transform
        // have).  A slice kernel holds one table at a time: with several, every table is a pass over all edges of
        // which only its share does work, and already at three tables (two species) the general kernels, which read
        // whichever table an edge needs from L2, are faster (0.92 against 1.32 ms per step at 3 000 atoms).
        const int R = hm.spl_nodes - 1, Kc = hm.K;
        if (nspl != 4 * Kc || tables.size() != 1) return 0;
        hipDeviceProp_t prop;
        int dev = 0;
        HIPCHK(hipGetDevice(&dev));
        HIPCHK(hipGetDeviceProperties(&prop, dev));
        num_cus = prop.multiProcessorCount;
        // LDS a single workgroup may use (opt-in limit where the runtime reports one)
        size_t lds_cap = prop.sharedMemPerBlock;
        if ((size_t)prop.sharedMemPerBlockOptin > lds_cap) lds_cap = prop.sharedMemPerBlockOptin;
        if (lds_cap > 160 * 1024) lds_cap = 160 * 1024;
        for (int CH = sizeof(F) == 8 ? 4 : 8; CH >= 2; CH /= 2) {
            // row = [4 coefficients][4 paths][CH channels], padded as the kernels of this precision want it
            const int W = slice_row_elements<F>(CH);
            if (W == 0) continue;
            if ((size_t)R * W * sizeof(F) > lds_cap) continue;
            const int S = (Kc + CH - 1) / CH;
            std::vector<F> buf((size_t)S * R * W, F(0));
            for (int sl = 0; sl < S; ++sl)
                for (int n = 0; n < R; ++n)
                    for (int q = 0; q < 4; ++q)
                        for (int pth = 0; pth < 4; ++pth)
                            for (int c = 0; c < CH; ++c) {
                                const int k = sl * CH + c;
                                if (k < Kc)
                                    buf[((size_t)sl * R + n) * W + (q * 4 + pth) * CH + c] =
                                        (F)tables[0][((size_t)n * 4 + q) * nspl + pth * Kc + k];
                            }
            dst.upload(buf.data(), buf.size(), s);
            HIPCHK(hipStreamSynchronize(s));
            slice_W = W;
            // adjoint kernel with one lane per edge: CH channels are 32 bytes, table slice and the staged adjoint
            // rows of twelve wavefronts fit the LDS
            edge_lanes = CH * sizeof(F) == 32 && slice_edge_lds_bytes<F>(hm.spl_nodes) <= lds_cap;
            if (edge_lanes) {
                const int We = slice_edge_row_elements<F>();
                std::vector<F> eb((size_t)S * R * We, F(0));
                for (size_t rowi = 0; rowi < (size_t)S * R; ++rowi)
                    std::copy(buf.begin() + rowi * W, buf.begin() + rowi * W + 16 * CH, eb.begin() + rowi * We);
                edst.upload(eb.data(), eb.size(), s);
                HIPCHK(hipStreamSynchronize(s));
                // forward kernel of such slices: per row [4 paths][2 halves][4 lanes][channels of the lane][2], the pair
                // being coefficients (2 half, 2 half + 1)
                const int cpln = CH / 4, Wf = 512 / (int)sizeof(F);
                std::vector<F> fb((size_t)S * R * Wf, F(0));
                for (int sl = 0; sl < S; ++sl)
                    for (int n = 0; n < R; ++n)
                        for (int pth = 0; pth < 4; ++pth)
                            for (int hf = 0; hf < 2; ++hf)
                                for (int ln = 0; ln < 4; ++ln)
                                    for (int c = 0; c < cpln; ++c)
                                        for (int j = 0; j < 2; ++j) {
                                            const int k = sl * CH + ln * cpln + c;
                                            if (k < Kc)
                                                fb[((size_t)sl * R + n) * Wf + ((((pth * 2 + hf) * 4 + ln) * cpln + c) * 2 + j)] =
                                                    (F)tables[0][((size_t)n * 4 + 2 * hf + j) * nspl + pth * Kc + k];
                                        }
                fdst.upload(fb.data(), fb.size(), s);
                HIPCHK(hipStreamSynchronize(s));
            }
            return CH;
        }
        return 0;
    }
    void build_slices(hipStream_t s)
    {
        slice_CH0 = build_slice_table(hm.tables0, hm.nspl0, tabS0, tabE0, tabF0, s);
        if (hm.L_max == 0) {
            // layer 1 qualifies when every output slot lm is fed by harmonic lm alone
            bool diag = hm.num_B == 16;
            for (int b = 0; diag && b < 16; ++b) {
                cdiag1[b] = 0.0;
                for (int t = hm.B_start[b]; t < hm.B_start[b + 1]; ++t) {
                    if (hm.B_lm1[t] != b) diag = false;
                    else cdiag1[b] += hm.B_c[t];
                }
            }
            if (diag) {
                slice_CH1 = build_slice_table(hm.tables1, hm.nspl1, tabS1, tabE1, tabF1, s);
            }
        }
    }
    SliceParams<F> slice_params(int layer, int N, bool adjoint = false)
    {
        SliceParams<F> p{};
        p.a = agg_params(layer, N);
        p.tabS = layer == 0 ? tabS0.p : tabS1.p;
        p.W = slice_W;
        if (!adjoint && edge_lanes) p.tabF = layer == 0 ? tabF0.p : tabF1.p;
        if (adjoint && edge_lanes) {
            p.edge_lanes = 1;
            DVec<F>& te = layer == 0 ? tabE0 : tabE1;
            if (te.p) { p.tabS = te.p; p.W = slice_edge_row_elements<F>(); }
        }
        p.CH = layer == 0 ? slice_CH0 : slice_CH1;
        for (int q = 0; q < 16; ++q) p.cdiag[q] = layer == 0 ? 1.0 : cdiag1[q];
        p.E = E;
        p.num_cus = num_cus;
        p.order = recv_order.p;
        return p;
    }

    // ------------------------------------------------------------------
    // geometry handling
    void set_geometry_ptrs(int N, const int* nt, const int* nn, const int* ni, const int* nty, const double* x,
                           const double* rr, long E_, bool on_device)
    {
        hipStream_t s = stream;
        if (on_device) {
            if (nt) node_types = nt;
            if (nn) num_neigh = nn;
            if (ni) neigh_indices = ni;
            if (nty) neigh_types = nty;
            if (x) xyz = x;
            if (rr) r = rr;
        } else {
            if (nt) { g_node_types.upload(nt, N, s); node_types = g_node_types.p; }
            if (nn) { g_num_neigh.upload(nn, N, s); num_neigh = g_num_neigh.p; }
            if (ni) { g_neigh_indices.upload(ni, E_, s); neigh_indices = g_neigh_indices.p; }
            if (nty) { g_neigh_types.upload(nty, E_, s); neigh_types = g_neigh_types.p; }
            if (x) { g_xyz.upload(x, 3 * E_, s); xyz = g_xyz.p; }
            if (rr) { g_r.upload(rr, E_, s); r = g_r.p; }
        }
        if (E_ >= 0) { E = E_; E1 = E_; }
    }
    void build_first_neigh(int N)
    {
        hipStream_t s = stream;
        first_neigh.size_to((size_t)N + 1, s);
        scan_tmp.size_to((size_t)N / 1024 + 2, s);
        HIPCHK(launch_scan_exclusive(num_neigh, first_neigh.p, N, scan_tmp.p, s));
        recv_order.size_to((size_t)N, s);
        HIPCHK(launch_degree_order(N, first_neigh.p, recv_order.p, s));
        N_geo = N;
    }
    void build_type_groups(int N)
    {
        hipStream_t s = stream;
        const int T = hm.T;
        t_count.size_to(T, s); t_start.size_to((size_t)T + 1, s); t_cursor.size_to(T, s); t_perm.size_to(N, s);
        scan_tmp.size_to((size_t)std::max(N, T) / 1024 + 2, s);
        HIPCHK(launch_type_groups(node_types, N, T, t_count.p, t_start.p, t_cursor.p, t_perm.p, scan_tmp.p, s));
    }
    void build_sender_lists(int rows)
    {
        hipStream_t s = stream;
        s_count.size_to((size_t)2 * rows, s); s_start.size_to((size_t)rows + 1, s);
        s_list.size_to((size_t)E1, s);
        scan_tmp.size_to((size_t)rows / 1024 + 2, s);
        HIPCHK(launch_sender_lists(neigh_indices, (int)E1, rows, s_count.p, s_start.p, s_count.p + rows, s_list.p, scan_tmp.p,
                                   senders_counted ? 2 : 0, senders_counted ? s_rank.p : nullptr, s, input_guard(N_geo)));
        senders_counted = false;
        counters_clean = 2L * rows;   // every build leaves its counters and cursors at zero
        sender_rows = rows;
    }
    // Host-path validation of what the reference leaves unchecked (mace.cpp:17-64 trusts
    // its caller; cubic_spline_set.cpp:54 reads past the table for r >= r_cut).
    void validate(int N, int rows)
    {
        hipStream_t s = stream;
        HIPCHK(hipMemsetAsync(flags.p, 0, sizeof(int), s));
        HIPCHK(launch_check_range(node_types, N, hm.T, flags.p, s));
        HIPCHK(launch_check_range(neigh_types, E, hm.T, flags.p, s));
        HIPCHK(launch_check_range(neigh_indices, E1, rows, flags.p, s));
        HIPCHK(launch_check_r(r, E, hm.r_cut, flags.p, s));
        int f = 0;
        HIPCHK(hipMemcpyAsync(&f, flags.p, sizeof(int), hipMemcpyDeviceToHost, s));
        HIPCHK(hipStreamSynchronize(s));
        if (f & 1) throw Error(SMX_EINVAL, "node_types / neigh_types / neigh_indices hold an index outside the model or the node range");
        if (f & 2) throw Error(SMX_ERANGE, "an edge length lies outside (0, r_cut): the radial spline tables do not cover it");
    }
    // stage-level calls: check whichever integer arrays this call brought
    void validate_stage_inputs(int N, bool have_nt, bool have_ni, bool have_nty, bool have_r)
    {
        hipStream_t s = stream;
        HIPCHK(hipMemsetAsync(flags.p, 0, sizeof(int), s));
        if (have_nt) HIPCHK(launch_check_range(node_types, N, hm.T, flags.p, s));
        if (have_nty) HIPCHK(launch_check_range(neigh_types, E, hm.T, flags.p, s));
        if (have_ni) {
            const size_t rows_now = H1.n / ((size_t)hm.num_LM * hm.K);
            HIPCHK(launch_check_range(neigh_indices, E, (int)std::max<size_t>(rows_now, (size_t)N), flags.p, s));
        }
        if (have_r) HIPCHK(launch_check_r(r, E, hm.r_cut, flags.p, s));
        int f = 0;
        HIPCHK(hipMemcpyAsync(&f, flags.p, sizeof(int), hipMemcpyDeviceToHost, s));
        HIPCHK(hipStreamSynchronize(s));
        if (f & 1) throw Error(SMX_EINVAL, "node_types / neigh_types / neigh_indices hold an index outside the model or the node range");
        if (f & 2) throw Error(SMX_ERANGE, "an edge length lies outside (0, r_cut): the radial spline tables do not cover it");
    }
    int edges_from_counts_check(int N, const int* host_num_neigh, long E_)
    {
        long tot = 0;
        for (int i = 0; i < N; ++i) {
            if (host_num_neigh[i] < 0) throw Error(SMX_EINVAL, "negative num_neigh entry");
            tot += host_num_neigh[i];
        }
        if (tot != E_) throw Error(SMX_EINVAL, "sum(num_neigh) does not match the number of edges");
        return 0;
    }

    // ------------------------------------------------------------------
    AggParams<F> agg_params(int layer, int N)
    {
        AggParams<F> p{};
        p.num_nodes = N; p.K = hm.K;
        p.first_neigh = first_neigh.p; p.node_types = node_types; p.neigh_types = neigh_types;
        p.xyz = xyz; p.r = r; p.T = hm.T; p.spl_nodes = hm.spl_nodes; p.spl_h = hm.spl_h; p.spl_inv_h = 1.0 / hm.spl_h;
        p.num_edges = E;
        if (layer == 0) {
            p.gather = neigh_types; p.Hsrc = H0.p; p.tab = tab0.p; p.tabK = tabK0.p; p.pair_table = pair_table0.p;
            p.B_start = B0_start.p; p.B_lm1 = B0_lm1.p; p.B_c = B0_c.p; p.num_terms = (int)B0_c.n;
        } else {
            p.gather = neigh_indices; p.Hsrc = H1.p; p.tab = tab1.p; p.tabK = tabK1.p; p.pair_table = pair_table1.p;
            p.B_start = B1_start.p; p.B_lm1 = B1_lm1.p; p.B_c = B1_c.p; p.num_terms = (int)B1_c.n;
        }
        return p;
    }
    void need(const void* p, const char* what)
    {
        if (!p) throw Error(SMX_EINVAL, std::string("stage called before its inputs exist: ") + what);
    }

    // ---- stages ------------------------------------------------------
    void st_agg0_fwd(int N)
    {
        need(xyz, "xyz (compute_Y)"); need(r, "r (compute_R0)"); need(first_neigh.p, "num_neigh");
        Phi0.size_to((size_t)N * 16 * K(), stream);
        if (slice_CH0) {
            auto sp = slice_params(0, N);
            sp.a.out = Phi0.p;
            HIPCHK(launch_slice_fwd<F>(sp, stream));
            return;
        }
        auto p = agg_params(0, N);
        p.out = Phi0.p;
        HIPCHK(launch_agg_fwd<F>(0, p, stream));
    }
    template <typename TA, typename TC, typename CT>
    GemmParams<TA, TC, CT> gemm_base(int N, bool typed)
    {
        GemmParams<TA, TC, CT> g{};
        g.num_nodes = N;
        if (typed) { need(t_perm.p, "species groups"); g.perm = t_perm.p; g.tstart = t_start.p; g.T = hm.T; }
        return g;
    }
    template <typename TA, typename TC, typename CT>
    static GemmProb<TA, TC, CT> gemm_prob(const TA* A, long a_node_stride, long a_off, long a_sub_stride, TC* C,
                                          long c_node_stride, long c_off, long c_sub_stride, const CT* W,
                                          long w_type_stride, long w_off, int transW, int accumulate, int Kd, int Nn,
                                          int sub)
    {
        GemmProb<TA, TC, CT> q{};
        q.A = A; q.a_node_stride = a_node_stride; q.a_off = a_off; q.a_sub_stride = a_sub_stride;
        q.C = C; q.c_node_stride = c_node_stride; q.c_off = c_off; q.c_sub_stride = c_sub_stride;
        q.W = W; q.w_type_stride = w_type_stride; q.w_off = w_off; q.transW = transW; q.accumulate = accumulate;
        q.Kd = Kd; q.Nn = Nn; q.sub = sub;
        return q;
    }
    // A0[i, l-block] = Phi0[i, l-block] . A0_weights[type_i][l]  (reverse: transposed weights)
    // `from_M0`: the adjoint product takes M0_grad . M0_adj (one polynomial per channel) as its operand
    // instead of a stored A0_adj
    void st_A0_lin(int N, bool reverse, bool from_M0 = false)
    {
        const int k = K();
        const F* src = reverse ? (from_M0 ? M0_grad.p : A0_adj.p) : Phi0.p;
        if (reverse) Phi0.size_to((size_t)N * 16 * k, stream); else A0.size_to((size_t)N * 16 * k, stream);
        F* dst = reverse ? Phi0.p : A0.p;
        auto g = gemm_base<F, F, F>(N, true);
        g.nprob = 4;
        for (int l = 0; l < 4; ++l) {
            g.prob[l] = gemm_prob<F, F, F>(src, 16L * k, (long)l * l * k, k, dst, 16L * k, (long)l * l * k, k, A0w.p,
                                           4L * k * k, (long)l * k * k, reverse ? 1 : 0, 0, k, k, 2 * l + 1);
            if (from_M0) { g.prob[l].Ascale = M0_adj.p; g.prob[l].ascale_node_stride = k; }
        }
        HIPCHK((launch_gemm<F, F, F>(g, stream)));
    }
    // density normalisation of A0 / A1 and its adjoint; no-ops for models without it (mace.cpp:280, 688)
    void st_scale(int layer, int N, bool reverse)
    {
        if (!(layer == 0 ? hm.A0_scaled : hm.A1_scaled)) return;
        need(r, "r"); need(first_neigh.p, "num_neigh"); need(node_types, "node_types"); need(neigh_types, "neigh_types");
        DVec<double>& dv = layer == 0 ? div0 : div1;
        DVec<F>& A = layer == 0 ? A0 : A1;
        DVec<F>& Aa = layer == 0 ? A0_adj : A1_adj;
        const int width = 16 * K();
        if (A.n < (size_t)N * width) throw Error(SMX_EINVAL, "density normalisation called before its A-basis exists");
        if (!reverse) {
            dv.size_to((size_t)N, stream);
            HIPCHK(launch_scale_fwd<F>(N, first_neigh.p, node_types, neigh_types, r, scale_spline(layer), hm.T, A.p, width,
                                       dv.p, flags.p, stream));
        } else {
            need(xyz, "xyz");
            if (dv.n < (size_t)N || Aa.n < (size_t)N * width)
                throw Error(SMX_EINVAL, "adjoint of the density normalisation called before its forward pass");
            node_forces.resize((size_t)3 * E, stream);
            HIPCHK(launch_scale_bwd<F>(N, first_neigh.p, node_types, neigh_types, xyz, r, scale_spline(layer), hm.T, A.p,
                                       Aa.p, width, dv.p, node_forces.p, flags.p, stream));
        }
    }
    void check_spline_flag()
    {
        int f = 0;
        HIPCHK(hipMemcpyAsync(&f, flags.p, sizeof(int), hipMemcpyDeviceToHost, stream));
        HIPCHK(hipStreamSynchronize(stream));
        if (f & 4) {
            HIPCHK(hipMemsetAsync(flags.p, 0, sizeof(int), stream));
            throw Error(SMX_ERANGE, "Out of bounds in CubicSpline::evaluate.");
        }
    }
    void st_zbl(int N)
    {
        if (!hm.has_zbl) return;
        HIPCHK(launch_zbl(N, first_neigh.p, node_types, neigh_types, xyz, r, zbl_params(), node_energies.p,
                          node_forces.p, stream));
    }
    // Layer 0 with several polynomials per channel and the standard product basis: the evaluation keeps no
    // gradients (16 numbers per polynomial and channel: four times the variables at l <= 1, nine times at l <= 2,
    // written once and read once); the adjoint stage evaluates them again from the variables instead.
    bool recompute_M0_grad() const { return M0_tables && NLM() > 1; }
    // mode 0: values and gradients; 1: values only; 2: layer-0 adjoint from the variables (A0_adj from A0, M0_adj)
    void st_poly(int N, bool layer1, int mode = 0)
    {
        PolyParams<F> p{};
        p.num_nodes = N; p.K = K(); p.mode = mode;
        const int off = layer1 ? NLM() : 0;
        p.NP = layer1 ? 1 : NLM();
        if (layer1) {
            M1.size_to((size_t)N * K(), stream); M1_grad.size_to((size_t)N * 16 * K(), stream);
            p.A = A1.p; p.M = M1.p; p.M_grad = M1_grad.p;
        } else if (mode == 2) {
            p.A = A0.p; p.M_adj = M0_adj.p; p.A_adj = A0_adj.p;
        } else {
            M0.size_to((size_t)N * NLM() * K(), stream);
            if (mode == 0) M0_grad.size_to((size_t)N * NLM() * 16 * K(), stream);
            p.A = A0.p; p.M = M0.p; p.M_grad = mode == 0 ? M0_grad.p : nullptr;
        }
        p.packed = pp_packed.p + off; p.chunks = pp_chunks.p + off; p.coef = pp_coef.p + off; p.num_entries = pp_nent.p + off;
        p.table_slabs = (layer1 ? M1_tables : M0_tables) ? (layer1 ? M1_slabs.p : M0_slabs.p) : nullptr;
        p.num_cus = num_cus;
        need(t_perm.p, "species groups");
        p.perm = t_perm.p; p.tstart = t_start.p; p.T = hm.T;
        HIPCHK(launch_poly<F>(p, stream));
    }
    void st_H1(int N, bool reverse)
    {
        const int k = K(), nlm = NLM();
        if (reverse) M0_adj.size_to(M0.n, stream);
        else if (H1.n != M0.n) H1.resize(M0.n, stream);   // mace.cpp:400
        const F* src = reverse ? H1_adj.p : M0.p;
        F* dst = reverse ? M0_adj.p : H1.p;
        auto g = gemm_base<F, F, F>(N, false);
        g.nprob = hm.L_max + 1;
        for (int l = 0; l <= hm.L_max; ++l)
            g.prob[l] = gemm_prob<F, F, F>(src, (long)nlm * k, (long)l * l * k, k, dst, (long)nlm * k, (long)l * l * k, k,
                                           H1w.p, 0, (long)l * k * k, reverse ? 1 : 0, 0, k, k, 2 * l + 1);
        HIPCHK((launch_gemm<F, F, F>(g, stream)));
    }
    void st_agg1_fwd(int N)
    {
        need(xyz, "xyz (compute_Y)"); need(r, "r (compute_R1)"); need(neigh_indices, "neigh_indices");
        Phi1.size_to((size_t)N * NE() * K(), stream);
        if (slice_CH1) {
            auto sp = slice_params(1, N);
            sp.a.out = Phi1.p;
            HIPCHK(launch_slice_fwd<F>(sp, stream));
            return;
        }
        auto p = agg_params(1, N);
        p.out = Phi1.p;
        HIPCHK(launch_agg_fwd<F>(hm.L_max, p, stream));
    }
    void st_A1(int N, bool reverse, bool from_M1 = false)
    {
        const int k = K(), ne = NE();
        if (reverse) dPhi1.size_to(Phi1.n, stream); else A1.size_to((size_t)N * 16 * k, stream);
        long lme_off = 0;
        auto g = gemm_base<F, F, F>(N, false);
        g.nprob = 4;
        for (int l = 0; l < 4; ++l) {
            const int nel = hm.num_e[l];
            if (!reverse)
                g.prob[l] = gemm_prob<F, F, F>(Phi1.p, (long)ne * k, lme_off * k, (long)nel * k, A1.p, 16L * k,
                                               (long)l * l * k, k, A1w.p, 0, A1w_off[l], 0, 0, nel * k, k, 2 * l + 1);
            else
            {
                g.prob[l] = gemm_prob<F, F, F>(from_M1 ? M1_grad.p : A1_adj.p, 16L * k, (long)l * l * k, k, dPhi1.p, (long)ne * k,
                                               lme_off * k, (long)nel * k, A1w.p, 0, A1w_off[l], 1, 0, k, nel * k, 2 * l + 1);
                if (from_M1) { g.prob[l].Ascale = M1_adj.p; g.prob[l].ascale_node_stride = k; }
            }
            lme_off += (2 * l + 1) * nel;
        }
        HIPCHK((launch_gemm<F, F, F>(g, stream)));
    }
    // H2 = H1[l=0] . W_H1[type] + M1 . W_M1 in one launch (mace.cpp:820-845)
    void st_H2(int N)
    {
        const int k = K(), nlm = NLM();
        H2.size_to((size_t)N * k, stream);
        auto g = gemm_base<F, double, double>(N, true);
        g.nprob = 1;
        g.prob[0] = gemm_prob<F, double, double>(H1.p, (long)nlm * k, 0, 0, H2.p, k, 0, 0, H2w_H1.p, (long)k * k, 0, 0, 0,
                                                 k, k, 1);
        g.prob[0].A2 = M1.p; g.prob[0].a2_node_stride = k; g.prob[0].W2 = H2w_M1.p; g.prob[0].w2_type_stride = 0;
        g.prob[0].transW2 = 0; g.prob[0].Kd2 = k;
        HIPCHK((launch_gemm<F, double, double>(g, stream)));
    }
    // H1_adj[l=0] += H2_adj . W_H1[type]^T and M1_adj = H2_adj . W_M1^T in one launch
    void st_reverse_H2(int N, bool zero_H1_adj)
    {
        const int k = K(), nlm = NLM();
        H1_adj.resize(H1.n, stream); M1_adj.size_to(M1.n, stream);
        if (zero_H1_adj) HIPCHK(hipMemsetAsync(H1_adj.p, 0, H1_adj.n * sizeof(F), stream));
        auto g = gemm_base<double, F, double>(N, true);
        g.nprob = 2;
        g.prob[0] = gemm_prob<double, F, double>(H2_adj.p, k, 0, 0, H1_adj.p, (long)nlm * k, 0, 0, H2w_H1.p, (long)k * k,
                                                 0, 1, 1, k, k, 1);
        g.prob[1] = gemm_prob<double, F, double>(H2_adj.p, k, 0, 0, M1_adj.p, k, 0, 0, H2w_M1.p, 0, 0, 1, 0, k, k, 1);
        HIPCHK((launch_gemm<double, F, double>(g, stream)));
    }
    // H2, readouts and reverse_H2 of the full pipeline in one launch (they touch one atom's rows only)
    void st_tail(int N, bool zero_energies)
    {
        const int k = K(), nlm = NLM();
        need(t_perm.p, "species groups");
        H2.size_to((size_t)N * k, stream); H2_adj.size_to((size_t)N * k, stream);
        node_energies.resize((size_t)N, stream);
        H1_adj.size_to(H1.n, stream); M1_adj.size_to(M1.n, stream);
        const int rows = (int)(H1.n / ((size_t)nlm * k));
        if (rows < N || M1.n < (size_t)N * k) throw Error(SMX_EINVAL, "readouts called before H1 and M1 exist for these nodes");
        TailParams<F> p{};
        p.N = N; p.rows = rows; p.K = k; p.num_LM = nlm; p.T = hm.T;
        p.perm = t_perm.p; p.tstart = t_start.p;
        p.E0 = E0.p; p.w1 = ro1.p; p.W1 = ro2_w1.p; p.w2 = ro2_w2.p; p.scale = hm.readout_2_scale;
        p.H1 = H1.p; p.M1 = M1.p; p.W_H1 = H2w_H1.p; p.W_M1 = H2w_M1.p;
        p.H2 = H2.p; p.H2_adj = H2_adj.p; p.H1_adj = H1_adj.p; p.M1_adj = M1_adj.p;
        p.node_energies = node_energies.p; p.zero_energies = zero_energies ? 1 : 0; p.energies_copy = energies_copy;
        p.guard = guard_live(); p.guard_clear = guard_status;
        p.guard_forces = guard_status ? node_forces.p : nullptr; p.guard_forces_n = guard_status ? (long)node_forces.n : 0;
        HIPCHK(launch_tail_fused<F>(p, stream));
        if (guard_status && rows > 0) guard_clear_enqueued = true;
        energies_copy = nullptr;
    }
    void st_readouts(int N, bool zero_energies)
    {
        const int k = K(), nlm = NLM();
        node_energies.resize((size_t)N, stream);
        H1_adj.size_to(H1.n, stream);
        H2_adj.size_to(H2.n, stream);
        const int rows = (int)(H1.n / ((size_t)nlm * k));
        if (rows < N || H2.n < (size_t)N * k) throw Error(SMX_EINVAL, "readouts called before H1 and H2 exist for these nodes");
        HIPCHK(launch_readout_fused<F>(N, rows, k, nlm, node_types, E0.p, ro1.p, ro2_w1.p, ro2_w2.p, hm.readout_2_scale,
                                       H1.p, H2.p, H2_adj.p, H1_adj.p, node_energies.p, zero_energies ? 1 : 0,
                                       energies_copy, guard_live(), guard_status, guard_status ? node_forces.p : nullptr,
                                       guard_status ? (long)node_forces.n : 0, stream));
        if (guard_status && rows > 0) guard_clear_enqueued = true;
        energies_copy = nullptr;
    }
    // node counts for which compute() left A1_adj / A0_adj unwritten (-1: they are current)
    int pending_A1_adj = -1, pending_A0_adj = -1;
    int pending_M0_grad = -1;   // compute() kept no layer-0 gradients for this many nodes: formed when somebody asks
    void materialise_adjoints(bool gradients)
    {
        if (pending_A1_adj >= 0) { st_reverse_M1(pending_A1_adj); pending_A1_adj = -1; }
        if (pending_A0_adj >= 0) { st_reverse_M0(pending_A0_adj); pending_A0_adj = -1; }
        if (gradients && pending_M0_grad >= 0) {
            const int n = pending_M0_grad;
            pending_M0_grad = -1;
            // (the species groups of the evaluation are still in place: compute() leaves them built for all its nodes,
            // and every call that rebuilds them comes through here first; the caller's arrays are not read again)
            if (n > 0) st_poly(n, false, 0);
        }
    }
    void st_reverse_M1(int N)
    {
        A1_adj.size_to(A1.n, stream);
        HIPCHK(launch_poly_reverse<F>(N, 1, K(), M1_grad.p, M1_adj.p, A1_adj.p, stream));
    }
    void st_reverse_M0(int N)
    {
        A0_adj.size_to(A0.n, stream);
        if (A0.n > (size_t)N * 16 * K())
            HIPCHK(hipMemsetAsync(A0_adj.p, 0, A0_adj.n * sizeof(F), stream));  // mace.cpp:376-377
        if (pending_M0_grad >= 0) {
            need(t_perm.p, "species groups");
            st_poly(N, false, 2);
        } else {
            HIPCHK(launch_poly_reverse<F>(N, NLM(), K(), M0_grad.p, M0_adj.p, A0_adj.p, stream));
        }
    }
    void st_agg1_bwd(int N, bool zero_dxyz, bool zero_H1_adj)
    {
        need(xyz, "xyz"); need(r, "r"); need(neigh_indices, "neigh_indices");
        const int k = K(), nlm = NLM();
        node_forces.resize((size_t)3 * E, stream);
        H1_adj.resize(H1.n, stream);
        const int rows = (int)(H1.n / ((size_t)nlm * k));
        const size_t row_bytes = (size_t)nlm * k * sizeof(F);
        if (!slice_CH1 && (size_t)E1 * row_bytes > msg_limit_bytes) {
            agg1_bwd_chunked(N, rows, zero_dxyz, zero_H1_adj);
            return;
        }
        msg.size_to((size_t)E1 * nlm * k, stream);
        stage_begin(ST_AGG1B);
        if (slice_CH1) {
            auto sp = slice_params(1, N, true);
            const int S = (k + sp.CH - 1) / sp.CH;
            fpart.size_to((size_t)S * 3 * E, stream);
            sp.a.d_out = dPhi1.p; sp.a.msg = msg.p; sp.fpart = fpart.p;
            HIPCHK(launch_slice_bwd<F>(sp, stream));
            stage_end(ST_AGG1B);
            stage_begin(ST_FSUM1);
            if (carry_forces && sp.edge_lanes && slice_CH0 == slice_CH1) {
                // the layer-0 adjoint of the same call adds its share to these partial forces and sums once
                carried_edges = E1;
                carried_accumulate = zero_dxyz ? 0 : 1;
            } else {
                HIPCHK(launch_fpart_reduce(E1, E, S, fpart.p, node_forces.p, zero_dxyz ? 0 : 1, nullptr, stream, guard_live()));
            }
            stage_end(ST_FSUM1);
        } else {
            auto p = agg_params(1, N);
            p.d_out = dPhi1.p; p.forces = node_forces.p; p.accumulate_forces = zero_dxyz ? 0 : 1; p.msg = msg.p;
            agg_bwd_general(hm.L_max, p, E1, ST_AGG1B, ST_FSUM1);
        }
        stage_begin(ST_SRED);
        if (sender_rows != rows) build_sender_lists(rows);
        if (fuse_reverse_H1 && nlm == 1 && sender_reduce_linear_ok(k) && M0.n == (size_t)rows * k) {
            // scalar hidden features: reverse_H1 of the summed rows in the same launch
            M0_adj.size_to(M0.n, stream);
            HIPCHK(launch_sender_reduce_linear<F>(rows, k, s_start.p, s_list.p, msg.p, H1_adj.p, zero_H1_adj ? 1 : 0, H1w.p,
                                                  M0_adj.p, stream));
            reverse_H1_done = true;
        } else {
            HIPCHK(launch_sender_reduce<F>(rows, nlm * k, s_start.p, s_list.p, msg.p, H1_adj.p, zero_H1_adj ? 1 : 0, 0, E1, stream));
        }
        stage_end(ST_SRED);
    }
    bool carry_forces = false;      // compute() lets the layer-1 partial forces wait for the layer-0 adjoint
    long carried_edges = 0;         // ... and the stage left them in fpart for edges [0, carried_edges)
    int carried_accumulate = 1;
    bool fuse_reverse_H1 = false;   // compute() wants reverse_H1 folded into the sender-side sum
    bool reverse_H1_done = false;   // ... and the stage did it
    // The same stage for edge lists whose messages do not fit the staging buffer: receivers are taken in
    // chunks, each chunk's messages are added to the sender rows before the next chunk overwrites them.  Every
    // sender still receives its messages in ascending edge order, so the result does not depend on the chunking.
    void agg1_bwd_chunked(int N, int rows, bool zero_dxyz, bool zero_H1_adj)
    {
        const int k = K(), nlm = NLM();
        const size_t row_bytes = (size_t)nlm * k * sizeof(F);
        const long max_rows = (long)std::max<size_t>(msg_limit_bytes / row_bytes, 1);
        // receiver boundaries: equal receiver counts, then halved until every chunk's edges fit (read back from the CSR)
        int nchunks = (int)std::min<long>(N, (E1 + max_rows - 1) / max_rows + 1);
        std::vector<int> bnd, fe;
        for (;;) {
            bnd.assign((size_t)nchunks + 1, 0); fe.assign((size_t)nchunks + 1, 0);
            for (int c = 0; c <= nchunks; ++c) {
                bnd[c] = (int)((long)N * c / nchunks);
                HIPCHK(hipMemcpyAsync(&fe[c], first_neigh.p + bnd[c], sizeof(int), hipMemcpyDeviceToHost, stream));
            }
            HIPCHK(hipStreamSynchronize(stream));
            long worst = 0;
            for (int c = 0; c < nchunks; ++c) worst = std::max<long>(worst, (long)fe[c + 1] - fe[c]);
            if (worst <= max_rows || nchunks >= N) {
                if (worst > max_rows)
                    throw Error(SMX_ENOMEM, "one receiver's messages exceed the staging limit (smx_set_staging_limit)");
                msg.size_to((size_t)worst * nlm * k, stream);
                break;
            }
            nchunks = (int)std::min<long>(N, 2L * nchunks);
        }
        const int groups = agg_bwd_groups<F>(hm.L_max, k);
        if (groups > 1) fpart.size_to((size_t)groups * 3 * E, stream);
        if (sender_rows != rows) build_sender_lists(rows);
        stage_begin(ST_AGG1B);
        for (int c = 0; c < nchunks; ++c) {
            auto p = agg_params(1, bnd[c + 1]);
            p.node_begin = bnd[c]; p.msg_edge_begin = fe[c];
            p.d_out = dPhi1.p; p.forces = node_forces.p; p.accumulate_forces = zero_dxyz ? 0 : 1; p.msg = msg.p;
            p.fpart = groups > 1 ? fpart.p : nullptr;
            HIPCHK(launch_agg_bwd<F>(hm.L_max, p, stream));
            HIPCHK(launch_sender_reduce<F>(rows, nlm * k, s_start.p, s_list.p, msg.p, H1_adj.p,
                                           (c == 0 && zero_H1_adj) ? 1 : 0, fe[c], fe[c + 1], stream));
        }
        stage_end(ST_AGG1B);
        stage_begin(ST_FSUM1);
        if (groups > 1)
            HIPCHK(launch_fpart_reduce(E1, E, groups, fpart.p, node_forces.p, zero_dxyz ? 0 : 1, nullptr, stream, guard_live()));
        stage_end(ST_FSUM1);
        stage_begin(ST_SRED);
        stage_end(ST_SRED);
    }
    void st_agg0_bwd(int N)
    {
        need(xyz, "xyz"); need(r, "r");
        node_forces.resize((size_t)3 * E, stream);
        if (slice_CH0) {
            auto sp = slice_params(0, N, true);
            const int S = (K() + sp.CH - 1) / sp.CH;
            fpart.size_to((size_t)S * 3 * E, stream);
            sp.a.d_out = Phi0.p; sp.a.msg = nullptr; sp.fpart = fpart.p;
            int accumulate = 1;
            if (carried_edges > 0) {
                // With carried layer-1 partial forces, edges past them (ghost receivers) have only this stage's share:
                // the sum below overwrites, so the forces must not hold anything else for them.
                sp.fpart_carry = carried_edges;
                accumulate = carried_accumulate;
                carried_edges = 0;
            }
            stage_begin(ST_AGG0B);
            HIPCHK(launch_slice_bwd<F>(sp, stream));
            stage_end(ST_AGG0B);
            stage_begin(ST_FSUM0);
            HIPCHK(launch_fpart_reduce(E, E, S, fpart.p, node_forces.p, accumulate, forces_copy, stream, guard_live()));
            forces_copy = nullptr;
            stage_end(ST_FSUM0);
            return;
        }
        auto p = agg_params(0, N);
        p.d_out = Phi0.p; p.forces = node_forces.p; p.accumulate_forces = 1; p.msg = nullptr;
        agg_bwd_general(0, p, E, ST_AGG0B, ST_FSUM0);
    }
    // general adjoint kernel; wide models are cut into channel groups whose partial forces are added in order
    void agg_bwd_general(int L_max_H, AggParams<F>& p, long edges, int st_kernel, int st_sum)
    {
        const int groups = agg_bwd_groups<F>(L_max_H, K());
        if (groups > 1) {
            fpart.size_to((size_t)groups * 3 * E, stream);
            p.fpart = fpart.p;
        }
        stage_begin(st_kernel);
        HIPCHK(launch_agg_bwd<F>(L_max_H, p, stream));
        stage_end(st_kernel);
        if (groups > 1) {
            stage_begin(st_sum);
            HIPCHK(launch_fpart_reduce(edges, E, groups, fpart.p, node_forces.p, p.accumulate_forces, nullptr, stream, guard_live()));
            stage_end(st_sum);
        }
    }

    // ------------------------------------------------------------------
    void compute(int N, const int* nt, const int* nn, const int* ni, const int* nty, const double* x,
                 const double* rr, long E_, bool on_device, double* d_energies, double* d_forces, int N_local,
                 long E_local) override
    {
        try {
            compute_impl(N, nt, nn, ni, nty, x, rr, E_, on_device, d_energies, d_forces, N_local, E_local);
        } catch (...) {
            // whatever was half built is not trusted by the next call
            senders_counted = false; counters_clean = 0; sender_rows = -1;
            energies_copy = nullptr; forces_copy = nullptr;
            carried_edges = 0; carry_forces = false; fuse_reverse_H1 = false;
            // checks of the failed call may have raised the word that only its readout launch would have cleared
            if (guard_status && !guard_clear_enqueued) (void)launch_fill<int>(guard_status, 1, 0, stream);
            guard_status = nullptr;
            throw;
        }
        guard_status = nullptr;
    }
    void compute_impl(int N, const int* nt, const int* nn, const int* ni, const int* nty, const double* x,
                      const double* rr, long E_, bool on_device, double* d_energies, double* d_forces, int N_local,
                      long E_local)
    {
        if (N < 0 || E_ < 0) throw Error(SMX_EINVAL, "negative num_nodes or num_edges");
        if (E_ > 2147483647L) throw Error(SMX_EINVAL, "more than 2^31 - 1 edges: edge offsets are 32-bit");
        // ghost nodes (the last N - N1 nodes and their edges) go through layer 0 only: their H1 rows feed the
        // local receivers, their adjoint comes back through H1_adj (pair_symmetrix_mace.cpp:662-698)
        const int N1 = N_local < 0 ? N : N_local;
        if (N1 > N || E_local > E_) throw Error(SMX_EINVAL, "more local nodes or edges than nodes or edges");
        if (N1 < N && E_local < 0) {
            if (on_device) throw Error(SMX_EINVAL, "the number of local edges is needed with ghost nodes");
            E_local = 0;
            for (int i = 0; i < N1; ++i) E_local += nn[i];
        }
        if (!on_device) edges_from_counts_check(N, nn, E_);
        if (N == 0) {
            if (E_ != 0) throw Error(SMX_EINVAL, "edges without nodes");
            E = 0; N_geo = 0;
            node_energies.size_to(0, stream); node_forces.size_to(0, stream);
            return;
        }
        stage_begin(ST_PREP);
        set_geometry_ptrs(N, nt, nn, ni, nty, x, rr, E_, on_device);
        if (N1 < N) E1 = E_local;
        // range checks come before any kernel that uses these integers as indices: host arrays are checked with a
        // read-back below; device arrays inside the list preparation, whose last launch empties the lists when a
        // check failed (input_guard)
        guard_status = nullptr; guard_clear_enqueued = false;
        if (on_device) {
            guard_status = flags.p + 2;
            ++device_calls;
        }
        if (on_device && N <= 65536) {
            // one launch for first_neigh, degree order, species groups and the sender histogram
            hipStream_t s = stream;
            first_neigh.size_to((size_t)N + 1, s); recv_order.size_to((size_t)N, s);
            t_start.size_to((size_t)hm.T + 1, s); t_perm.size_to((size_t)N, s);
            const int* before = s_count.p;
            s_count.size_to((size_t)2 * N, s); s_start.size_to((size_t)N + 1, s);
            scan_tmp.size_to((size_t)N / 1024 + 2, s);
            if (s_count.p != before || counters_clean < 2L * N) HIPCHK(launch_fill<int>(s_count.p, 2L * N, 0, s));
            s_rank.size_to((size_t)E1, s);
            InputChecks chk;
            chk.status = guard_status; chk.neigh_types = neigh_types; chk.r = r; chk.r_cut = hm.r_cut; chk.num_edges = E;
            chk.num_local_nodes = N1;
            HIPCHK(launch_node_lists_count(num_neigh, N, first_neigh.p, recv_order.p, node_types, hm.T, t_start.p, t_perm.p,
                                           neigh_indices, E1, N, s_count.p, s_rank.p, chk, s));
            N_geo = N;
            senders_counted = true;
        } else {
            build_first_neigh(N);
            if (!on_device) validate(N, N);
            else {
                HIPCHK(launch_check_counts(num_neigh, N, first_neigh.p, N1, E, E1, guard_status, stream));
                HIPCHK(launch_check_range(node_types, N, hm.T, guard_status, stream));
                HIPCHK(launch_check_range(neigh_types, E, hm.T, guard_status, stream));
                HIPCHK(launch_check_range(neigh_indices, E1, N, guard_status, stream));
                HIPCHK(launch_check_r(r, E, hm.r_cut, guard_status, stream));
            }
            build_type_groups(N);
        }
        sender_rows = -1;
        build_sender_lists(N);
        stage_end(ST_PREP);

        node_energies.size_to((size_t)N1, stream);
        node_forces.size_to((size_t)3 * E, stream);
        if (N == 0) return;

        energies_copy = d_energies; forces_copy = d_forces;
        // Terms that add to the forces before the layer-1 adjoint writes them (mace.cpp:27-35, 56): with any of
        // them the force array starts at zero and every later stage accumulates.
        const bool early_forces = hm.has_zbl || hm.A1_scaled || N1 < N;
        if (early_forces) HIPCHK(launch_fill<double>(node_forces.p, 3 * E, 0.0, stream));
        if (hm.has_zbl) {
            HIPCHK(launch_fill<double>(node_energies.p, (long)N1, 0.0, stream));
            st_zbl(N1);
        }
        stage_begin(ST_AGG0F); st_agg0_fwd(N); stage_end(ST_AGG0F);
        stage_begin(ST_A0LIN); st_A0_lin(N, false); stage_end(ST_A0LIN);
        st_scale(0, N, false);
        pending_M0_grad = recompute_M0_grad() ? N : -1;
        stage_begin(ST_M0); st_poly(N, false, pending_M0_grad >= 0 ? 1 : 0); stage_end(ST_M0);
        stage_begin(ST_H1); st_H1(N, false); stage_end(ST_H1);
        // per-species node groups and the degree order of the receivers cover the nodes of the current stages
        auto node_lists_for = [&](int n) {
            build_type_groups(n);
            HIPCHK(launch_degree_order(n, first_neigh.p, recv_order.p, stream));
        };
        if (N1 < N) node_lists_for(N1);
        stage_begin(ST_AGG1F); st_agg1_fwd(N1); stage_end(ST_AGG1F);
        stage_begin(ST_A1); st_A1(N1, false); stage_end(ST_A1);
        st_scale(1, N1, false);
        stage_begin(ST_M1); st_poly(N1, true); stage_end(ST_M1);
        if (tail_fused_ok(K())) {
            stage_begin(ST_H2); st_tail(N1, !hm.has_zbl); stage_end(ST_H2);
            stage_begin(ST_READOUT); stage_end(ST_READOUT);
            stage_begin(ST_REVH2); stage_end(ST_REVH2);
        } else {
            stage_begin(ST_H2); st_H2(N1); stage_end(ST_H2);
            stage_begin(ST_READOUT); st_readouts(N1, !hm.has_zbl); stage_end(ST_READOUT);
            stage_begin(ST_REVH2); st_reverse_H2(N1, false); stage_end(ST_REVH2);
        }
        // Without density normalisation nothing between reverse_M and the adjoint linear reads A_adj: the
        // linear then forms M_grad . M_adj itself while loading its rows (one polynomial per channel) and
        // A_adj is only written if somebody asks for it (get_array).
        const bool fuse1 = !hm.A1_scaled && gemm_scaled_operand_ok(K(), K(), sizeof(F));
        const bool fuse0 = !hm.A0_scaled && NLM() == 1 && gemm_scaled_operand_ok(K(), K(), sizeof(F));
        stage_begin(ST_REVM1); if (!fuse1) st_reverse_M1(N1); stage_end(ST_REVM1);
        pending_A1_adj = fuse1 ? N1 : -1;
        st_scale(1, N1, true);
        stage_begin(ST_REVA1); st_A1(N1, true, fuse1); stage_end(ST_REVA1);
        fuse_reverse_H1 = N1 == N; reverse_H1_done = false;
        // (the density normalisation of layer 0 adds to the forces in between: then they must already hold the layer-1 sum)
        carry_forces = early_forces || !hm.A0_scaled; carried_edges = 0;
        st_agg1_bwd(N1, !early_forces, false);
        fuse_reverse_H1 = false; carry_forces = false;
        if (N1 < N) node_lists_for(N);
        stage_begin(ST_REVH1); if (!reverse_H1_done) st_H1(N, true); stage_end(ST_REVH1);
        stage_begin(ST_REVM0); if (!fuse0) st_reverse_M0(N); stage_end(ST_REVM0);
        pending_A0_adj = fuse0 ? N : -1;
        st_scale(0, N, true);
        stage_begin(ST_REVA0LIN); st_A0_lin(N, true, fuse0); stage_end(ST_REVA0LIN);
        st_agg0_bwd(N);
        // (a skipped evaluation: the readout launch has filled the forces with NaN, and every sum of partial forces
        // after it looks at the guard itself)
        if (guard_status && !guard_clear_enqueued) HIPCHK(launch_fill<int>(guard_status, 1, 0, stream));

        if (energies_copy) HIPCHK(hipMemcpyAsync(energies_copy, node_energies.p, (size_t)N1 * sizeof(double), hipMemcpyDeviceToDevice, stream));
        if (forces_copy && E) HIPCHK(hipMemcpyAsync(forces_copy, node_forces.p, (size_t)3 * E * sizeof(double), hipMemcpyDeviceToDevice, stream));
        energies_copy = nullptr; forces_copy = nullptr;
        // the reference throws from CubicSpline::evaluate for an edge beyond the normalisation spline
        // (cubic_spline.cpp:19-20); callers of the device-resident variant vouch for their edge lengths
        if (!on_device && (hm.A0_scaled || hm.A1_scaled)) check_spline_flag();
    }

    // stage-level entry points (host arrays)
    void stage(const char* name, int N, const int* nt, const int* nn, const int* ni, const int* nty,
               const double* x, const double* rr, long E_, int fa, int fb) override
    {
        const std::string s(name);
        energies_copy = nullptr; forces_copy = nullptr;
        carried_edges = 0; carry_forces = false; fuse_reverse_H1 = false; guard_status = nullptr;
        materialise_adjoints(true);
        if (N < 0) throw Error(SMX_EINVAL, "negative num_nodes");
        // A stage may cover the leading nodes of a longer edge list (the pair style runs layer 1 on its local
        // nodes with the arrays of local + ghost nodes, pair_symmetrix_mace.cpp:681-693): the edge arrays keep
        // their full length, the stage's own edges are the first sum(num_neigh[0..N)).
        long own_edges = -1;
        if (nn) {
            own_edges = 0;
            for (int i = 0; i < N; ++i) {
                if (nn[i] < 0) throw Error(SMX_EINVAL, "negative num_neigh entry");
                own_edges += nn[i];
            }
            const long have = E_ >= 0 ? E_ : E;
            if (own_edges > have) throw Error(SMX_EINVAL, "sum(num_neigh) exceeds the number of edges");
        }
        set_geometry_ptrs(N, nt, nn, ni, nty, x, rr, E_, false);
        if (nn) { build_first_neigh(N); E1 = own_edges; }
        validate_stage_inputs(N, nt != nullptr, ni != nullptr, nty != nullptr, rr != nullptr);
        if (s == "Y" || s == "R0" || s == "R1") return;  // geometry remembered; evaluated inside the fused kernels
        if (s == "A0") { build_type_groups(N); st_agg0_fwd(N); st_A0_lin(N, false); }
        else if (s == "reverse_A0") { build_type_groups(N); st_A0_lin(N, true); st_agg0_bwd(N); }
        else if (s == "A0_scaled") { st_scale(0, N, false); if (hm.A0_scaled) check_spline_flag(); }
        else if (s == "reverse_A0_scaled") { st_scale(0, N, true); if (hm.A0_scaled) check_spline_flag(); }
        else if (s == "A1_scaled") { st_scale(1, N, false); if (hm.A1_scaled) check_spline_flag(); }
        else if (s == "reverse_A1_scaled") {
            if (hm.A1_scaled) {
                node_forces.resize((size_t)3 * E, stream);
                if (fa) HIPCHK(launch_fill<double>(node_forces.p, 3 * E, 0.0, stream));
            }
            st_scale(1, N, true);
            if (hm.A1_scaled) check_spline_flag();
        }
        else if (s == "M0") { build_type_groups(N); st_poly(N, false); }
        else if (s == "reverse_M0") st_reverse_M0(N);
        else if (s == "H1") st_H1(N, false);
        else if (s == "reverse_H1") st_H1(N, true);
        else if (s == "Phi1") { need(node_types, "node_types (compute_R1)"); st_agg1_fwd(N); }
        else if (s == "reverse_Phi1") { sender_rows = -1; st_agg1_bwd(N, fa != 0, fb != 0); }
        else if (s == "A1") st_A1(N, false);
        else if (s == "reverse_A1") st_A1(N, true);
        else if (s == "M1") { build_type_groups(N); st_poly(N, true); }
        else if (s == "reverse_M1") st_reverse_M1(N);
        else if (s == "H2") { build_type_groups(N); st_H2(N); }
        else if (s == "reverse_H2") { build_type_groups(N); st_reverse_H2(N, fa != 0); }
        else if (s == "readouts") st_readouts(N, false);
        else if (s == "ZBL") {
            // zbl.cpp:96-125 adds to the caller's node_energies / node_forces: here to the engine's arrays, which
            // grow like std::vector::resize (new entries zero) when the edge list changed
            if (hm.has_zbl) {
                need(xyz, "xyz"); need(r, "r"); need(first_neigh.p, "num_neigh"); need(node_types, "node_types");
                need(neigh_types, "neigh_types");
                node_energies.resize((size_t)N, stream);
                node_forces.resize((size_t)3 * E, stream);
                st_zbl(N);
            }
        }
        else throw Error(SMX_EINVAL, "unknown stage " + s);
    }

    // ------------------------------------------------------------------
    struct Named { DVec<F>* f; DVec<double>* d; };
    Named find(const std::string& n)
    {
        if (n == "A0") return {&A0, nullptr};
        if (n == "A0_adj") return {&A0_adj, nullptr};
        if (n == "M0") return {&M0, nullptr};
        if (n == "M0_grad") return {&M0_grad, nullptr};
        if (n == "M0_adj") return {&M0_adj, nullptr};
        if (n == "H1") return {&H1, nullptr};
        if (n == "H1_adj") return {&H1_adj, nullptr};
        if (n == "Phi0") return {&Phi0, nullptr};
        if (n == "Phi1") return {&Phi1, nullptr};
        if (n == "Phi1_adj" || n == "dPhi1") return {&dPhi1, nullptr};
        if (n == "A1") return {&A1, nullptr};
        if (n == "A1_adj") return {&A1_adj, nullptr};
        if (n == "M1") return {&M1, nullptr};
        if (n == "M1_grad") return {&M1_grad, nullptr};
        if (n == "M1_adj") return {&M1_adj, nullptr};
        if (n == "H0_weights") return {&H0, nullptr};
        if (n == "H2") return {nullptr, &H2};
        if (n == "H2_adj") return {nullptr, &H2_adj};
        if (n == "node_energies") return {nullptr, &node_energies};
        if (n == "node_forces") return {nullptr, &node_forces};
        return {nullptr, nullptr};
    }
    void get_array(const char* name, double* out, long cap, long* n) override
    {
        const std::string s(name);
        hipStream_t st = stream;
        materialise_adjoints(s == "M0_grad");
        const double* src = nullptr;
        size_t len = 0;
        if (s == "Y" || s == "Y_grad") {
            need(xyz, "xyz (compute_Y)");
            scratch_d.size_to((size_t)E * 64, st);
            HIPCHK(launch_sph_harm(xyz, E, scratch_d.p, scratch_d.p + (size_t)E * 16, st));
            src = s == "Y" ? scratch_d.p : scratch_d.p + (size_t)E * 16;
            len = s == "Y" ? (size_t)E * 16 : (size_t)E * 48;
        } else if (s == "R0" || s == "R1") {
            need(r, "r (compute_R0/R1)"); need(first_neigh.p, "num_neigh"); need(node_types, "node_types");
            const bool l1 = s == "R1";
            const int nspl = l1 ? hm.nspl1 : hm.nspl0;
            scratch_d.size_to((size_t)E * nspl, st);
            HIPCHK(launch_radial<F>(N_geo, first_neigh.p, node_types, neigh_types, r, l1 ? tab1.p : tab0.p,
                                    l1 ? pair_table1.p : pair_table0.p, hm.T, hm.spl_nodes, hm.spl_h, nspl, scratch_d.p, st));
            src = scratch_d.p; len = (size_t)E * nspl;
        } else {
            Named v = find(s);
            if (!v.f && !v.d) throw Error(SMX_EINVAL, "unknown array '" + s + "'");
            if (v.d) { src = v.d->p; len = v.d->n; }
            else {
                len = v.f->n;
                if (std::is_same<F, double>::value) src = reinterpret_cast<const double*>(v.f->p);
                else {
                    scratch_d.size_to(len, st);
                    HIPCHK((launch_convert<F, double>(v.f->p, scratch_d.p, (long)len, st)));
                    src = scratch_d.p;
                }
            }
        }
        if (n) *n = (long)len;
        if (out && cap > 0 && len > 0) {
            const size_t m = std::min((size_t)cap, len);
            HIPCHK(hipMemcpyAsync(out, src, m * sizeof(double), hipMemcpyDeviceToHost, st));
        }
        HIPCHK(hipStreamSynchronize(st));
    }
    void set_array(const char* name, const double* in, long n) override
    {
        const std::string s(name);
        hipStream_t st = stream;
        if (n < 0) throw Error(SMX_EINVAL, "negative length");
        materialise_adjoints(true);
        Named v = find(s);
        if (s == "R0" || s == "R1")
            throw Error(SMX_EUNSUPPORTED, "unsupported: '" + s + "' is evaluated from r inside the edge kernels and never "
                        "stored; call compute_" + s + " with the edge lengths instead of assigning it");
        if ((!v.f && !v.d) || s == "M0_grad" || s == "M1_grad")
            throw Error(SMX_EINVAL, "array '" + s + "' cannot be set");
        if (s == "H0_weights" && (size_t)n != (size_t)hm.T * hm.K)
            throw Error(SMX_EINVAL, "H0_weights holds num_elements * num_channels values");
        if (v.d) { v.d->upload(in, (size_t)n, st); }
        else if (std::is_same<F, double>::value) { reinterpret_cast<DVec<double>*>(v.f)->upload(in, (size_t)n, st); }
        else {
            scratch_d.upload(in, (size_t)n, st);
            v.f->size_to((size_t)n, st);
            HIPCHK((launch_convert<double, F>(scratch_d.p, v.f->p, n, st)));
        }
        HIPCHK(hipStreamSynchronize(st));
    }

    void forces_view(ForcesView* v) override
    {
        v->node_forces = node_forces.p; v->forces_len = (long)node_forces.n; v->xyz = xyz; v->first_neigh = first_neigh.p;
        v->num_edges = E; v->num_receivers = N_geo; v->device = device;
    }
    // size a named array to n entries, all equal to `value`, without a host copy
    void fill_array(const char* name, long n, double value) override
    {
        const std::string s(name);
        if (n < 0) throw Error(SMX_EINVAL, "negative length");
        materialise_adjoints(true);
        Named v = find(s);
        if ((!v.f && !v.d) || s == "H0_weights" || s == "M0_grad" || s == "M1_grad")
            throw Error(SMX_EINVAL, "array '" + s + "' cannot be set");
        if (v.d) { v.d->size_to((size_t)n, stream); HIPCHK(launch_fill<double>(v.d->p, n, value, stream)); }
        else { v.f->size_to((size_t)n, stream); HIPCHK(launch_fill<F>(v.f->p, n, (F)value, stream)); }
    }

    // ------------------------------------------------------------------
    DVec<int> rf_send, rf_recv, rf_count, rf_sstart, rf_cursor, rf_slist, rf_rstart, rf_rlist;
    DVec<double> rf_out;
    void reduce_forces(int num_atoms, const int* sender_atom, const int* receiver_atom, double* atom_forces,
                       double* virial, bool sender_on_device) override
    {
        hipStream_t s = stream;
        need(node_forces.p, "node_forces");
        if (node_forces.n != (size_t)3 * E) throw Error(SMX_EINVAL, "node_forces does not match the current edge list");
        if (atom_forces) {
            if (num_atoms <= 0) throw Error(SMX_EINVAL, "num_atoms must be positive");
            if (!sender_atom) throw Error(SMX_EINVAL, "sender_atom is required");
            const int* send = sender_atom;
            if (!sender_on_device) { rf_send.upload(sender_atom, (size_t)E, s); send = rf_send.p; }
            rf_count.size_to(num_atoms, s); rf_cursor.size_to(num_atoms, s);
            rf_sstart.size_to((size_t)num_atoms + 1, s); rf_slist.size_to((size_t)E, s);
            scan_tmp.size_to((size_t)num_atoms / 1024 + 2, s);
            HIPCHK(hipMemsetAsync(flags.p, 0, sizeof(int), s));
            HIPCHK(launch_check_range(send, E, num_atoms, flags.p, s));
            {
                int f = 0;
                HIPCHK(hipMemcpyAsync(&f, flags.p, sizeof(int), hipMemcpyDeviceToHost, s));
                HIPCHK(hipStreamSynchronize(s));
                if (f) throw Error(SMX_EINVAL, "sender_atom out of range");
            }
            const int* rstart = nullptr;
            const int* rlist = nullptr;
            if (receiver_atom) {
                // receiver_atom[i] = atom row of receiver block i -> expand to edges
                std::vector<int> hn(N_geo), hr((size_t)E);
                HIPCHK(hipMemcpyAsync(hn.data(), num_neigh, (size_t)N_geo * sizeof(int), hipMemcpyDeviceToHost, s));
                HIPCHK(hipStreamSynchronize(s));
                size_t e = 0;
                for (int i = 0; i < N_geo; ++i) {
                    if (receiver_atom[i] < 0 || receiver_atom[i] >= num_atoms) throw Error(SMX_EINVAL, "receiver_atom out of range");
                    if (hn[i] < 0 || e + (size_t)hn[i] > (size_t)E) throw Error(SMX_EINVAL, "num_neigh does not match the number of edges");
                    for (int j = 0; j < hn[i]; ++j) hr[e++] = receiver_atom[i];
                }
                if (e != (size_t)E) throw Error(SMX_EINVAL, "num_neigh of the last call does not cover every edge");
                rf_recv.upload(hr.data(), hr.size(), s);
                HIPCHK(hipStreamSynchronize(s));
                rf_rstart.size_to((size_t)num_atoms + 1, s); rf_rlist.size_to((size_t)E, s);
                HIPCHK(launch_sender_lists(rf_recv.p, (int)E, num_atoms, rf_count.p, rf_rstart.p, rf_cursor.p, rf_rlist.p, scan_tmp.p, 0, nullptr, s));
                rstart = rf_rstart.p; rlist = rf_rlist.p;
            } else {
                if (num_atoms < N_geo) throw Error(SMX_EINVAL, "num_atoms is smaller than the number of receivers");
                // receiver block i is atom i: CSR offsets padded with E for atoms beyond the receivers
                std::vector<int> h((size_t)num_atoms + 1);
                HIPCHK(hipMemcpyAsync(h.data(), first_neigh.p, ((size_t)N_geo + 1) * sizeof(int), hipMemcpyDeviceToHost, s));
                HIPCHK(hipStreamSynchronize(s));
                for (int i = N_geo + 1; i <= num_atoms; ++i) h[i] = h[N_geo];
                rf_rstart.upload(h.data(), h.size(), s);
                HIPCHK(hipStreamSynchronize(s));
                rstart = rf_rstart.p;
            }
            HIPCHK(launch_sender_lists(send, (int)E, num_atoms, rf_count.p, rf_sstart.p, rf_cursor.p, rf_slist.p, scan_tmp.p, 0, nullptr, s));
            rf_out.size_to((size_t)3 * num_atoms, s);
            HIPCHK(launch_force_scatter(num_atoms, rstart, rlist, rf_sstart.p, rf_slist.p, node_forces.p, rf_out.p, s));
            HIPCHK(hipMemcpyAsync(atom_forces, rf_out.p, (size_t)3 * num_atoms * sizeof(double), hipMemcpyDeviceToHost, s));
            HIPCHK(hipStreamSynchronize(s));
        }
        if (virial) {
            const int nb = 64;
            scratch_d.size_to((size_t)nb * 6, s);
            HIPCHK(launch_virial(E, xyz, node_forces.p, scratch_d.p, nb, s));
            std::vector<double> part((size_t)nb * 6);
            HIPCHK(hipMemcpyAsync(part.data(), scratch_d.p, part.size() * sizeof(double), hipMemcpyDeviceToHost, s));
            HIPCHK(hipStreamSynchronize(s));
            for (int q = 0; q < 6; ++q) {
                double v = 0;
                for (int b = 0; b < nb; ++b) v += part[(size_t)b * 6 + q];
                virial[q] = v;
            }
        }
    }
};

void set_last_error(const std::string& msg) { g_last_error = msg; }

}  // namespace smx

// ===========================================================================
struct smx_model {
    std::unique_ptr<smx::EngineBase> eng;
};

namespace smx {
int engine_forces_view(smx_model* m, ForcesView* out, std::string* err)
{
    if (!m || !m->eng) { if (err) *err = "null model"; return SMX_EINVAL; }
    m->eng->forces_view(out);
    return SMX_OK;
}
}  // namespace smx

namespace {

template <typename Fn>
int guarded(Fn&& fn)
{
    try {
        fn();
        return SMX_OK;
    } catch (const smx::Error& e) {
        smx::g_last_error = e.what();
        return e.code;
    } catch (const smx::JsonError& e) {
        smx::g_last_error = e.what();
        return SMX_EFILE;
    } catch (const std::bad_alloc&) {
        smx::g_last_error = "out of host memory";
        return SMX_ENOMEM;
    } catch (const std::exception& e) {
        const std::string w = e.what();
        smx::g_last_error = w;
        return w.rfind("unsupported:", 0) == 0 ? SMX_EUNSUPPORTED : SMX_EINVAL;
    }
}

void require_device()
{
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0)
        throw smx::Error(SMX_ENODEVICE, "no HIP device available: this engine has no CPU path");
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) throw smx::Error(SMX_ENODEVICE, "hipGetDevice failed");
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) throw smx::Error(SMX_ENODEVICE, "hipGetDeviceProperties failed");
    if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0)
        throw smx::Error(SMX_ENODEVICE, std::string("kernels are built for gfx950 only; found ") + prop.gcnArchName);
}

smx::EngineBase& E(smx_model* m)
{
    if (!m || !m->eng) throw smx::Error(SMX_EINVAL, "null model");
    return *m->eng;
}

}  // namespace

// ---------------------------------------------------------------------------
// Device neighbour list (canonical order; see smx_kernels_nlist.hip)
namespace smx {
struct NeighborList {
    DVec<double> part, shift_vec, xyz, r;
    DVec<int> shift_int, atom_bin, bin_count, bin_start, bin_atoms, count, cfirst, first, num_neigh, neigh_indices,
        neigh_types, neigh_shift, scan_tmp;
    DVec<long long> keys, sorted;
    DVec<double> pos_dev;     // copies of host inputs (smx_nlist_build_host / smx_nlist_update_host)
    DVec<int> types_dev;
    int N = 0, num_shifts = 0;
    long E = 0, num_candidates = 0;
    double r_list = 0.0;

    // candidates: every (receiver, sender, image) closer than r_list, sorted per receiver
    void build(int N_, const double* d_pos, int num_shifts_, const int* h_shift_int, const double* h_shift_vec,
               double r_list_, hipStream_t s)
    {
        if (N_ < 0 || num_shifts_ <= 0 || !(r_list_ > 0.0) || !h_shift_int || !h_shift_vec || (N_ > 0 && !d_pos))
            throw Error(SMX_EINVAL, "neighbour list: bad arguments");
        int zero_shift = -1;
        for (int q = 0; q < num_shifts_; ++q)
            if (h_shift_int[3 * q] == 0 && h_shift_int[3 * q + 1] == 0 && h_shift_int[3 * q + 2] == 0) zero_shift = q;
        N = N_; num_shifts = num_shifts_; r_list = r_list_; E = 0; num_candidates = 0;
        cfirst.size_to((size_t)N + 1, s);
        if (N == 0) return;
        shift_int.upload(h_shift_int, (size_t)3 * num_shifts, s);
        shift_vec.upload(h_shift_vec, (size_t)3 * num_shifts, s);
        // bounding box (per-block partials, finished on the host)
        const int nblk = std::min(256, (N + 255) / 256);
        part.size_to((size_t)nblk * 6, s);
        HIPCHK(launch_nl_bbox(d_pos, N, part.p, nblk, s));
        std::vector<double> hp((size_t)nblk * 6);
        HIPCHK(hipMemcpyAsync(hp.data(), part.p, hp.size() * sizeof(double), hipMemcpyDeviceToHost, s));
        HIPCHK(hipStreamSynchronize(s));
        NlGrid g{};
        long nbins = 1;
        for (int k = 0; k < 3; ++k) {
            double lo = 1e300, hi = -1e300;
            for (int b = 0; b < nblk; ++b) { lo = std::min(lo, hp[(size_t)b * 6 + k]); hi = std::max(hi, hp[(size_t)b * 6 + 3 + k]); }
            if (!(lo <= hi) || !(hi - lo < 1e300)) throw Error(SMX_EINVAL, "neighbour list: positions are not finite");
            g.lo[k] = lo; g.hi[k] = hi;
            const double ext = hi - lo;
            int nb = (int)std::floor(std::min(ext / r_list, 1e6));
            nb = std::max(1, std::min(nb, 128));
            g.nb[k] = nb;
            g.inv_bs[k] = ext > 0.0 ? nb / ext : 0.0;
            nbins *= nb;
        }
        atom_bin.size_to((size_t)N, s); bin_count.size_to((size_t)2 * nbins, s); bin_start.size_to((size_t)nbins + 1, s);
        bin_atoms.size_to((size_t)N, s); scan_tmp.size_to((size_t)std::max<long>(nbins, N) / 1024 + 2, s);
        HIPCHK(hipMemsetAsync(bin_count.p, 0, (size_t)2 * nbins * sizeof(int), s));
        HIPCHK(launch_nl_bins(d_pos, N, g, atom_bin.p, bin_count.p, s));
        HIPCHK(launch_scan_exclusive(bin_count.p, bin_start.p, (int)nbins, scan_tmp.p, s));
        HIPCHK(launch_nl_bin_fill(N, atom_bin.p, bin_start.p, bin_count.p + nbins, bin_atoms.p, s));
        count.size_to((size_t)N, s);
        HIPCHK(launch_nl_search(false, d_pos, N, g, bin_start.p, bin_atoms.p, num_shifts, shift_vec.p, zero_shift, r_list,
                                count.p, nullptr, nullptr, s));
        HIPCHK(launch_scan_exclusive(count.p, cfirst.p, N, scan_tmp.p, s));
        int total = 0;
        HIPCHK(hipMemcpyAsync(&total, cfirst.p + N, sizeof(int), hipMemcpyDeviceToHost, s));
        HIPCHK(hipStreamSynchronize(s));
        if (total < 0) throw Error(SMX_EINVAL, "neighbour list: more than 2^31 candidate pairs");
        num_candidates = total;
        keys.size_to((size_t)num_candidates, s); sorted.size_to((size_t)num_candidates, s);
        HIPCHK(launch_nl_search(true, d_pos, N, g, bin_start.p, bin_atoms.p, num_shifts, shift_vec.p, zero_shift, r_list,
                                nullptr, cfirst.p, keys.p, s));
        HIPCHK(launch_nl_sort(N, cfirst.p, keys.p, sorted.p, s));
    }

    // edges: the candidates closer than r_cut at the given positions, in candidate order
    long update(const double* d_pos, const int* d_types, double r_cut, hipStream_t s)
    {
        if (!(r_cut > 0.0) || r_cut > r_list || (N > 0 && !d_pos))
            throw Error(SMX_EINVAL, "neighbour list: the cutoff must be positive and no larger than the radius of the last build");
        E = 0;
        first.size_to((size_t)N + 1, s); num_neigh.size_to((size_t)N, s);
        if (N == 0) {
            HIPCHK(hipMemsetAsync(first.p, 0, sizeof(int), s));
            return 0;
        }
        HIPCHK(launch_nl_filter(false, d_pos, d_types, N, cfirst.p, sorted.p, num_shifts, shift_vec.p, shift_int.p, r_cut,
                                num_neigh.p, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, s));
        HIPCHK(launch_scan_exclusive(num_neigh.p, first.p, N, scan_tmp.p, s));
        int total = 0;
        HIPCHK(hipMemcpyAsync(&total, first.p + N, sizeof(int), hipMemcpyDeviceToHost, s));
        HIPCHK(hipStreamSynchronize(s));
        E = total;
        neigh_indices.size_to((size_t)E, s); neigh_types.size_to((size_t)E, s); neigh_shift.size_to((size_t)3 * E, s);
        xyz.size_to((size_t)3 * E, s); r.size_to((size_t)E, s);
        HIPCHK(launch_nl_filter(true, d_pos, d_types, N, cfirst.p, sorted.p, num_shifts, shift_vec.p, shift_int.p, r_cut,
                                nullptr, first.p, neigh_indices.p, neigh_types.p, neigh_shift.p, xyz.p, r.p, s));
        return E;
    }
};
}  // namespace smx

extern "C" {

const char* smx_last_error(void) { return smx::g_last_error.c_str(); }

int smx_model_load(const char* json_path, int flags, smx_model** out)
{
    return guarded([&] {
        if (!json_path || !out) throw smx::Error(SMX_EINVAL, "null argument");
        if (flags != SMX_FP64 && flags != SMX_FP32_FEATURES) throw smx::Error(SMX_EINVAL, "unknown precision flag");
        *out = nullptr;
        smx::HostModel hm = smx::load_host_model(json_path);
        require_device();
        {
            // the scratch array of the entry point that does not allocate: its address on this device, once
            std::string err;
            const int rc = smx::noalloc_setup_current_device(&err);
            if (rc != SMX_OK) throw smx::Error(rc, err);
        }
        std::unique_ptr<smx_model> m(new smx_model());
        if (flags == SMX_FP64) m->eng.reset(new smx::Engine<double>(std::move(hm), flags));
        else m->eng.reset(new smx::Engine<float>(std::move(hm), flags));
        *out = m.release();
    });
}

void smx_model_free(smx_model* m)
{
    if (!m) return;
    (void)hipDeviceSynchronize();
    delete m;
}

int smx_model_get_int(const smx_model* m, const char* key, int* out)
{
    return guarded([&] {
        if (!m || !key || !out) throw smx::Error(SMX_EINVAL, "null argument");
        const smx::HostModel& h = m->eng->hm;
        const std::string k(key);
        if (k == "num_elements") *out = h.T;
        else if (k == "num_channels") *out = h.K;
        else if (k == "l_max") *out = h.l_max;
        else if (k == "num_lm") *out = h.num_lm;
        else if (k == "L_max") *out = h.L_max;
        else if (k == "num_LM") *out = h.num_LM;
        else if (k == "has_zbl") *out = h.has_zbl ? 1 : 0;
        else if (k == "num_lme") *out = h.num_lme;
        else if (k == "num_lelm1lm2") *out = h.num_lelm1lm2;
        else if (k == "precision") *out = m->eng->precision;
        else if (k == "num_radial_tables_0") *out = (int)h.tables0.size();
        else if (k == "num_radial_tables_1") *out = (int)h.tables1.size();
        else if (k == "contraction_tables") *out = m->eng->contraction_tables();
        else throw smx::Error(SMX_EINVAL, "unknown integer key '" + k + "'");
    });
}

int smx_model_get_double(const smx_model* m, const char* key, double* out)
{
    return guarded([&] {
        if (!m || !key || !out) throw smx::Error(SMX_EINVAL, "null argument");
        const std::string k(key);
        if (k == "r_cut") *out = m->eng->hm.r_cut;
        else throw smx::Error(SMX_EINVAL, "unknown double key '" + k + "'");
    });
}

int smx_model_get_atomic_numbers(const smx_model* m, int* out, int cap, int* n)
{
    return guarded([&] {
        if (!m) throw smx::Error(SMX_EINVAL, "null model");
        const auto& v = m->eng->hm.atomic_numbers;
        if (n) *n = (int)v.size();
        for (int i = 0; out && i < cap && i < (int)v.size(); ++i) out[i] = v[i];
    });
}
int smx_model_get_atomic_energies(const smx_model* m, double* out, int cap, int* n)
{
    return guarded([&] {
        if (!m) throw smx::Error(SMX_EINVAL, "null model");
        const auto& v = m->eng->hm.atomic_energies;
        if (n) *n = (int)v.size();
        for (int i = 0; out && i < cap && i < (int)v.size(); ++i) out[i] = v[i];
    });
}

int smx_compute_node_energies_forces(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                                     const int* neigh_indices, const int* neigh_types, const double* xyz,
                                     const double* r, long num_edges)
{
    return guarded([&] {
        auto& e = E(m);
        if (num_nodes > 0 && (!node_types || !num_neigh)) throw smx::Error(SMX_EINVAL, "null node array");
        if (num_edges > 0 && (!neigh_indices || !neigh_types || !xyz || !r)) throw smx::Error(SMX_EINVAL, "null edge array");
        e.stream = nullptr;
        e.compute(num_nodes, node_types, num_neigh, neigh_indices, neigh_types, xyz, r, num_edges, false, nullptr, nullptr, -1, -1);
        HIPCHK(hipStreamSynchronize(e.stream));
    });
}

int smx_compute_device(smx_model* m, int num_nodes, const int* d_node_types, const int* d_num_neigh,
                       const int* d_neigh_indices, const int* d_neigh_types, const double* d_xyz, const double* d_r,
                       long num_edges, double* d_node_energies, double* d_node_forces, void* stream)
{
    return guarded([&] {
        auto& e = E(m);
        if (num_nodes > 0 && (!d_node_types || !d_num_neigh)) throw smx::Error(SMX_EINVAL, "null node array");
        if (num_edges > 0 && (!d_neigh_indices || !d_neigh_types || !d_xyz || !d_r)) throw smx::Error(SMX_EINVAL, "null edge array");
        e.stream = static_cast<hipStream_t>(stream);
        e.compute(num_nodes, d_node_types, d_num_neigh, d_neigh_indices, d_neigh_types, d_xyz, d_r, num_edges, true,
                  d_node_energies, d_node_forces, -1, -1);
    });
}

int smx_compute_ghosted(smx_model* m, int num_local_nodes, int num_ghost_nodes, const int* node_types,
                        const int* num_neigh, const int* neigh_indices, const int* neigh_types, const double* xyz,
                        const double* r, long num_edges)
{
    return guarded([&] {
        auto& e = E(m);
        if (num_local_nodes < 0 || num_ghost_nodes < 0) throw smx::Error(SMX_EINVAL, "negative node count");
        const int n = num_local_nodes + num_ghost_nodes;
        if (n > 0 && (!node_types || !num_neigh)) throw smx::Error(SMX_EINVAL, "null node array");
        if (num_edges > 0 && (!neigh_indices || !neigh_types || !xyz || !r)) throw smx::Error(SMX_EINVAL, "null edge array");
        e.stream = nullptr;
        e.compute(n, node_types, num_neigh, neigh_indices, neigh_types, xyz, r, num_edges, false, nullptr, nullptr,
                  num_local_nodes, -1);
        HIPCHK(hipStreamSynchronize(e.stream));
    });
}

int smx_compute_ghosted_device(smx_model* m, int num_local_nodes, int num_ghost_nodes, const int* d_node_types,
                               const int* d_num_neigh, const int* d_neigh_indices, const int* d_neigh_types,
                               const double* d_xyz, const double* d_r, long num_edges, long num_local_edges,
                               double* d_node_energies, double* d_node_forces, void* stream)
{
    return guarded([&] {
        auto& e = E(m);
        if (num_local_nodes < 0 || num_ghost_nodes < 0 || num_local_edges < 0) throw smx::Error(SMX_EINVAL, "negative count");
        const int n = num_local_nodes + num_ghost_nodes;
        if (n > 0 && (!d_node_types || !d_num_neigh)) throw smx::Error(SMX_EINVAL, "null node array");
        if (num_edges > 0 && (!d_neigh_indices || !d_neigh_types || !d_xyz || !d_r)) throw smx::Error(SMX_EINVAL, "null edge array");
        e.stream = static_cast<hipStream_t>(stream);
        e.compute(n, d_node_types, d_num_neigh, d_neigh_indices, d_neigh_types, d_xyz, d_r, num_edges, true,
                  d_node_energies, d_node_forces, num_local_nodes, num_local_edges);
    });
}

int smx_set_num_H1_rows(smx_model* m, int rows)
{
    return guarded([&] { E(m).H1_rows_override = rows; });
}

#define SMX_STAGE(fn, name, NT, NN, NI, NTY, XYZ, R, EE, FA, FB) \
    return guarded([&] { auto& e = E(m); e.stream = nullptr; e.stage(name, num_nodes, NT, NN, NI, NTY, XYZ, R, EE, FA, FB); HIPCHK(hipStreamSynchronize(e.stream)); })

int smx_compute_Y(smx_model* m, const double* xyz, long n3)
{
    const int num_nodes = 0;
    if (n3 % 3) { smx::g_last_error = "xyz length is not a multiple of 3"; return SMX_EINVAL; }
    SMX_STAGE(smx_compute_Y, "Y", nullptr, nullptr, nullptr, nullptr, xyz, nullptr, n3 / 3, 0, 0);
}
int smx_compute_R0(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh, const int* neigh_types,
                   const double* r, long num_edges)
{
    SMX_STAGE(smx_compute_R0, "R0", node_types, num_neigh, nullptr, neigh_types, nullptr, r, num_edges, 0, 0);
}
int smx_compute_R1(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh, const int* neigh_types,
                   const double* r, long num_edges)
{
    SMX_STAGE(smx_compute_R1, "R1", node_types, num_neigh, nullptr, neigh_types, nullptr, r, num_edges, 0, 0);
}
int smx_compute_A0(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh, const int* neigh_types,
                   long num_edges)
{
    SMX_STAGE(smx_compute_A0, "A0", node_types, num_neigh, nullptr, neigh_types, nullptr, nullptr, num_edges, 0, 0);
}
int smx_reverse_A0(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh, const int* neigh_types,
                   const double* xyz, const double* r, long num_edges)
{
    SMX_STAGE(smx_reverse_A0, "reverse_A0", node_types, num_neigh, nullptr, neigh_types, xyz, r, num_edges, 0, 0);
}
int smx_compute_A0_scaled(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                          const int* neigh_types, const double* r, long num_edges)
{
    SMX_STAGE(smx_compute_A0_scaled, "A0_scaled", node_types, num_neigh, nullptr, neigh_types, nullptr, r, num_edges, 0, 0);
}
int smx_reverse_A0_scaled(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                          const int* neigh_types, const double* xyz, const double* r, long num_edges)
{
    SMX_STAGE(smx_reverse_A0_scaled, "reverse_A0_scaled", node_types, num_neigh, nullptr, neigh_types, xyz, r, num_edges, 0, 0);
}
int smx_compute_A1_scaled(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                          const int* neigh_types, const double* r, long num_edges)
{
    SMX_STAGE(smx_compute_A1_scaled, "A1_scaled", node_types, num_neigh, nullptr, neigh_types, nullptr, r, num_edges, 0, 0);
}
int smx_reverse_A1_scaled(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh,
                          const int* neigh_types, const double* xyz, const double* r, long num_edges, int zero_dxyz)
{
    SMX_STAGE(smx_reverse_A1_scaled, "reverse_A1_scaled", node_types, num_neigh, nullptr, neigh_types, xyz, r, num_edges,
              zero_dxyz, 0);
}
int smx_compute_M0(smx_model* m, int num_nodes, const int* node_types)
{
    SMX_STAGE(smx_compute_M0, "M0", node_types, nullptr, nullptr, nullptr, nullptr, nullptr, -1, 0, 0);
}
int smx_reverse_M0(smx_model* m, int num_nodes, const int* node_types)
{
    SMX_STAGE(smx_reverse_M0, "reverse_M0", node_types, nullptr, nullptr, nullptr, nullptr, nullptr, -1, 0, 0);
}
int smx_compute_H1(smx_model* m, int num_nodes)
{
    SMX_STAGE(smx_compute_H1, "H1", nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, -1, 0, 0);
}
int smx_reverse_H1(smx_model* m, int num_nodes)
{
    SMX_STAGE(smx_reverse_H1, "reverse_H1", nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, -1, 0, 0);
}
int smx_compute_Phi1(smx_model* m, int num_nodes, const int* num_neigh, const int* neigh_indices, long num_edges)
{
    SMX_STAGE(smx_compute_Phi1, "Phi1", nullptr, num_neigh, neigh_indices, nullptr, nullptr, nullptr, num_edges, 0, 0);
}
int smx_reverse_Phi1(smx_model* m, int num_nodes, const int* num_neigh, const int* neigh_indices, const double* xyz,
                     const double* r, long num_edges, int zero_dxyz, int zero_H1_adj)
{
    SMX_STAGE(smx_reverse_Phi1, "reverse_Phi1", nullptr, num_neigh, neigh_indices, nullptr, xyz, r, num_edges, zero_dxyz, zero_H1_adj);
}
int smx_compute_A1(smx_model* m, int num_nodes)
{
    SMX_STAGE(smx_compute_A1, "A1", nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, -1, 0, 0);
}
int smx_reverse_A1(smx_model* m, int num_nodes)
{
    SMX_STAGE(smx_reverse_A1, "reverse_A1", nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, -1, 0, 0);
}
int smx_compute_M1(smx_model* m, int num_nodes, const int* node_types)
{
    SMX_STAGE(smx_compute_M1, "M1", node_types, nullptr, nullptr, nullptr, nullptr, nullptr, -1, 0, 0);
}
int smx_reverse_M1(smx_model* m, int num_nodes, const int* node_types)
{
    SMX_STAGE(smx_reverse_M1, "reverse_M1", node_types, nullptr, nullptr, nullptr, nullptr, nullptr, -1, 0, 0);
}
int smx_compute_H2(smx_model* m, int num_nodes, const int* node_types)
{
    SMX_STAGE(smx_compute_H2, "H2", node_types, nullptr, nullptr, nullptr, nullptr, nullptr, -1, 0, 0);
}
int smx_reverse_H2(smx_model* m, int num_nodes, const int* node_types, int zero_H1_adj)
{
    SMX_STAGE(smx_reverse_H2, "reverse_H2", node_types, nullptr, nullptr, nullptr, nullptr, nullptr, -1, zero_H1_adj, 0);
}
int smx_compute_readouts(smx_model* m, int num_nodes, const int* node_types)
{
    SMX_STAGE(smx_compute_readouts, "readouts", node_types, nullptr, nullptr, nullptr, nullptr, nullptr, -1, 0, 0);
}

int smx_compute_ZBL(smx_model* m, int num_nodes, const int* node_types, const int* num_neigh, const int* neigh_types,
                    const double* r, const double* xyz, long num_edges)
{
    SMX_STAGE(smx_compute_ZBL, "ZBL", node_types, num_neigh, nullptr, neigh_types, xyz, r, num_edges, 0, 0);
}

int smx_get_array(smx_model* m, const char* name, double* out, long cap, long* n)
{
    return guarded([&] {
        if (!name) throw smx::Error(SMX_EINVAL, "null name");
        E(m).check_device_status();
        E(m).get_array(name, out, cap, n);
    });
}
int smx_set_array(smx_model* m, const char* name, const double* in, long n)
{
    return guarded([&] {
        if (!name || (!in && n > 0)) throw smx::Error(SMX_EINVAL, "null argument");
        E(m).set_array(name, in, n);
    });
}

int smx_fill_array(smx_model* m, const char* name, long n, double value)
{
    return guarded([&] {
        if (!name) throw smx::Error(SMX_EINVAL, "null name");
        auto& e = E(m);
        e.fill_array(name, n, value);
        HIPCHK(hipStreamSynchronize(e.stream));
    });
}

int smx_set_profiling(smx_model* m, int enabled)
{
    return guarded([&] {
        auto& e = E(m);
        e.profiling = enabled != 0;
        for (int i = 0; i < smx::ST_COUNT; ++i) e.ev_used[i] = false;
    });
}
int smx_set_staging_limit(smx_model* m, long bytes)
{
    return guarded([&] {
        if (bytes <= 0) throw smx::Error(SMX_EINVAL, "the staging limit must be positive");
        E(m).msg_limit_bytes = (size_t)bytes;
    });
}
const char* smx_stage_names(void) { return smx::kStageNames; }
int smx_get_stage_times(smx_model* m, float* ms, int cap, int* n)
{
    return guarded([&] {
        auto& e = E(m);
        HIPCHK(hipStreamSynchronize(e.stream));
        if (n) *n = smx::ST_COUNT;
        for (int i = 0; ms && i < cap && i < smx::ST_COUNT; ++i) {
            ms[i] = 0.f;
            if (e.ev_used[i]) HIPCHK(hipEventElapsedTime(&ms[i], e.ev0[i], e.ev1[i]));
        }
    });
}
int smx_synchronize(smx_model* m)
{
    return guarded([&] {
        auto& e = E(m);
        HIPCHK(hipStreamSynchronize(e.stream));
        e.check_device_status();
    });
}
int smx_reduce_forces(smx_model* m, int num_atoms, const int* sender_atom, const int* receiver_atom,
                      double* atom_forces, double* virial)
{
    return guarded([&] {
        E(m).reduce_forces(num_atoms, sender_atom, receiver_atom, atom_forces, virial, false);
        E(m).check_device_status();   // forces of a skipped device-resident evaluation are NaN: say why
    });
}
int smx_reduce_forces_device(smx_model* m, int num_atoms, const int* d_sender_atom, double* atom_forces, double* virial)
{
    return guarded([&] {
        E(m).reduce_forces(num_atoms, d_sender_atom, nullptr, atom_forces, virial, true);
        E(m).check_device_status();
    });
}

smx_nlist* smx_nlist_create(void)
{
    smx_nlist* out = nullptr;
    guarded([&] { out = reinterpret_cast<smx_nlist*>(new smx::NeighborList()); });
    return out;
}
void smx_nlist_free(smx_nlist* nl) { delete reinterpret_cast<smx::NeighborList*>(nl); }
int smx_nlist_build(smx_nlist* nl, int num_atoms, const double* d_positions, const int* d_types, int num_shifts,
                    const int* shift_int, const double* shift_vec, double r_list, double r_cut, void* stream,
                    long* num_edges)
{
    return guarded([&] {
        if (!nl || !shift_int || !shift_vec || (num_atoms > 0 && !d_positions)) throw smx::Error(SMX_EINVAL, "null argument");
        if (!(r_cut > 0.0) || r_cut > r_list) throw smx::Error(SMX_EINVAL, "neighbour list: need 0 < r_cut <= r_list");
        auto& n = *reinterpret_cast<smx::NeighborList*>(nl);
        n.build(num_atoms, d_positions, num_shifts, shift_int, shift_vec, r_list, (hipStream_t)stream);
        const long e = n.update(d_positions, d_types, r_cut, (hipStream_t)stream);
        if (num_edges) *num_edges = e;
    });
}
int smx_nlist_update(smx_nlist* nl, const double* d_positions, const int* d_types, double r_cut, void* stream,
                     long* num_edges)
{
    return guarded([&] {
        if (!nl) throw smx::Error(SMX_EINVAL, "null argument");
        const long e = reinterpret_cast<smx::NeighborList*>(nl)->update(d_positions, d_types, r_cut, (hipStream_t)stream);
        if (num_edges) *num_edges = e;
    });
}
int smx_nlist_build_host(smx_nlist* nl, int num_atoms, const double* positions, const int* types, int num_shifts,
                         const int* shift_int, const double* shift_vec, double r_list, double r_cut, long* num_edges)
{
    return guarded([&] {
        if (!nl || !shift_int || !shift_vec || num_atoms < 0 || (num_atoms > 0 && (!positions || !types)))
            throw smx::Error(SMX_EINVAL, "null argument");
        if (!(r_cut > 0.0) || r_cut > r_list) throw smx::Error(SMX_EINVAL, "neighbour list: need 0 < r_cut <= r_list");
        require_device();
        auto& n = *reinterpret_cast<smx::NeighborList*>(nl);
        n.pos_dev.upload(positions, (size_t)3 * num_atoms, nullptr);
        n.types_dev.upload(types, (size_t)num_atoms, nullptr);
        n.build(num_atoms, n.pos_dev.p, num_shifts, shift_int, shift_vec, r_list, nullptr);
        const long e = n.update(n.pos_dev.p, n.types_dev.p, r_cut, nullptr);
        HIPCHK(hipStreamSynchronize(nullptr));
        if (num_edges) *num_edges = e;
    });
}
int smx_nlist_update_host(smx_nlist* nl, const double* positions, double r_cut, long* num_edges)
{
    return guarded([&] {
        if (!nl) throw smx::Error(SMX_EINVAL, "null argument");
        auto& n = *reinterpret_cast<smx::NeighborList*>(nl);
        if (n.types_dev.n != (size_t)n.N || (n.N > 0 && !positions))
            throw smx::Error(SMX_EINVAL, "neighbour list: update from host positions needs a build from host positions first");
        n.pos_dev.upload(positions, (size_t)3 * n.N, nullptr);
        const long e = n.update(n.pos_dev.p, n.types_dev.p, r_cut, nullptr);
        HIPCHK(hipStreamSynchronize(nullptr));
        if (num_edges) *num_edges = e;
    });
}
int smx_nlist_inputs(smx_nlist* nl, const double** d_positions, const int** d_types)
{
    return guarded([&] {
        if (!nl) throw smx::Error(SMX_EINVAL, "null argument");
        auto& n = *reinterpret_cast<smx::NeighborList*>(nl);
        if (d_positions) *d_positions = n.pos_dev.p;
        if (d_types) *d_types = n.types_dev.p;
    });
}
int smx_nlist_arrays(smx_nlist* nl, const int** num_neigh, const int** first_neigh, const int** neigh_indices,
                     const int** neigh_types, const int** neigh_shift, const double** xyz, const double** r)
{
    return guarded([&] {
        if (!nl) throw smx::Error(SMX_EINVAL, "null argument");
        auto& n = *reinterpret_cast<smx::NeighborList*>(nl);
        if (num_neigh) *num_neigh = n.num_neigh.p;
        if (first_neigh) *first_neigh = n.first.p;
        if (neigh_indices) *neigh_indices = n.neigh_indices.p;
        if (neigh_types) *neigh_types = n.neigh_types.p;
        if (neigh_shift) *neigh_shift = n.neigh_shift.p;
        if (xyz) *xyz = n.xyz.p;
        if (r) *r = n.r.p;
    });
}
int smx_nlist_copy_to_host(smx_nlist* nl, int* num_neigh, int* neigh_indices, int* neigh_types, int* neigh_shift,
                           double* xyz, double* r)
{
    return guarded([&] {
        if (!nl) throw smx::Error(SMX_EINVAL, "null argument");
        auto& n = *reinterpret_cast<smx::NeighborList*>(nl);
        const size_t E = (size_t)n.E, N = (size_t)n.N;
        if (num_neigh && N) HIPCHK(hipMemcpy(num_neigh, n.num_neigh.p, N * sizeof(int), hipMemcpyDeviceToHost));
        if (neigh_indices && E) HIPCHK(hipMemcpy(neigh_indices, n.neigh_indices.p, E * sizeof(int), hipMemcpyDeviceToHost));
        if (neigh_types && E) HIPCHK(hipMemcpy(neigh_types, n.neigh_types.p, E * sizeof(int), hipMemcpyDeviceToHost));
        if (neigh_shift && E) HIPCHK(hipMemcpy(neigh_shift, n.neigh_shift.p, 3 * E * sizeof(int), hipMemcpyDeviceToHost));
        if (xyz && E) HIPCHK(hipMemcpy(xyz, n.xyz.p, 3 * E * sizeof(double), hipMemcpyDeviceToHost));
        if (r && E) HIPCHK(hipMemcpy(r, n.r.p, E * sizeof(double), hipMemcpyDeviceToHost));
    });
}

}  // extern "C"
