// Edge kernels for gfx950, general form: fused harmonics + radial splines +
// receiver-segmented aggregation, and the analytic edge-force adjoint, for any
// path list (scalar or l <= 1 hidden features) and any number of radial tables.
//
// Work decomposition.  The edge list is receiver-sorted (CSR).  One wavefront
// owns one receiver; lane j owns CPL consecutive channels, so every table or
// feature load of the wavefront is one contiguous run.  Accumulators (NE per
// channel) live in registers for the whole neighbour loop, so sums run in edge
// order with no atomics and are bit-reproducible.  Edges are taken in chunks of
// EC.  Per chunk, the first EC lanes evaluate direction, harmonics and spline
// interval of one edge each; then all 64 lanes share the EC x NB entries of the
// Clebsch-Gordan-contracted harmonics B (and their gradients in the adjoint);
// both go through LDS, from where the channel loop reads them as broadcasts.
// The four wavefronts of a block share nothing but the coupling list, so the
// only block-wide barrier is the one after that list is copied to LDS.
#include "smx_device.hpp"
#include "smx_kernels.hpp"
#include "smx_paths.hpp"

namespace smx {

namespace {

template <typename F, int LMAXH, bool BWD>
struct WaveLds {
    using PT = Paths<LMAXH>;
    static constexpr int NBP = (PT::NB + 3) / 4 * 4;          // B row padded for 16-byte reads
    static constexpr int NY = BWD ? 64 : 16;                  // Y (and dY/dx, dY/dy, dY/dz)
    static constexpr int NBT = BWD ? 4 * NBP : NBP;
    __host__ __device__ static constexpr size_t per_wave(int EC)
    {
        size_t b = (size_t)EC * (NY * sizeof(double) + (BWD ? 12 * sizeof(double) : 0) + NBT * sizeof(F));
        b += (size_t)EC * (sizeof(double) + 2 * sizeof(int));   // x (held as double-sized slot), rows, gather rows
        return (b + 15) / 16 * 16;
    }
    // Double-precision forward kernel with vector sender features: the coefficients of the first PRE paths of the
    // next edge wait in LDS, brought there by loads that bypass the registers (32 bytes per lane and path).
    static constexpr bool PREFETCH = !BWD && sizeof(F) == 8 && LMAXH == 1;
    static constexpr int PRE = PREFETCH ? PT::P / 2 : 0;
    __host__ __device__ static constexpr size_t prefetch_per_wave() { return (size_t)PRE * 64 * 32; }
    __host__ __device__ static constexpr size_t lists(int num_terms)
    {
        return ((size_t)num_terms * (sizeof(double) + sizeof(int)) + (PT::NB + 1) * sizeof(int) + 15) / 16 * 16;
    }
};

// The steps in which the adjoint kernel walks the coupling block B[path][m][m2] of an edge.  Wide steps (single
// precision): all rows m of a path with a scalar sender feature, three rows at a time of a path with a vector one
// (at most nine entries).  Narrow steps (double precision, where an entry takes eight registers): at most three
// entries, i.e. three rows of a scalar path or one row of a vector path.
template <int LMAXH, bool NARROW>
struct BwdSteps {
    using PT = Paths<LMAXH>;
    static constexpr int rows(int p) { return 2 * PT::l(p) + 1; }
    static constexpr int group(int p)
    {
        if (NARROW) return PT::l2(p) == 0 ? (rows(p) < 3 ? rows(p) : 3) : 1;
        return PT::l2(p) == 0 ? rows(p) : (PT::l2(p) == 1 ? 3 : 1);
    }
    static constexpr int groups(int p) { return (rows(p) + group(p) - 1) / group(p); }
    static constexpr int count()
    {
        int n = 0;
        for (int p = 0; p < PT::P; ++p) n += groups(p);
        return n;
    }
    static constexpr int path(int s)
    {
        for (int p = 0; p < PT::P; ++p) {
            if (s < groups(p)) return p;
            s -= groups(p);
        }
        return -1;
    }
    static constexpr int m0(int s)
    {
        for (int p = 0; p < PT::P; ++p) {
            if (s < groups(p)) return s * group(p);
            s -= groups(p);
        }
        return -1;
    }
    static constexpr int m1(int s)
    {
        const int p = path(s), e = m0(s) + group(p);
        return e < rows(p) ? e : rows(p);
    }
    static constexpr int len(int s) { return (m1(s) - m0(s)) * (2 * PT::l2(path(s)) + 1); }
    static constexpr int max_len()
    {
        int n = 0;
        for (int s = 0; s < count(); ++s) n = len(s) > n ? len(s) : n;
        return n;
    }
    static constexpr int MAXLEN = max_len();
};

// Everything addressed through boffs after this point is scheduled after the three sums are final.
template <typename F>
__device__ __forceinline__ void order_after(F& g1, F& g2, F& srad, int& boffs)
{
    asm volatile("" : "+v"(g1), "+v"(g2), "+v"(srad), "+v"(boffs));
}

// The value is final here: keeps an accumulation from drifting past the fences (its operands would stay live).
template <typename F>
__device__ __forceinline__ void pin(F& v)
{
    asm volatile("" : "+v"(v));
}

// v is final here, and what is addressed through off afterwards is not loaded before
template <typename F>
__device__ __forceinline__ void tie(F& v, int& off)
{
    asm volatile("" : "+v"(v), "+v"(off));
}

template <typename F, int CPL>
__device__ __forceinline__ Vec<F, CPL> ldv(const F* p)
{
    return *reinterpret_cast<const Vec<F, CPL>*>(p);
}

// Entry b of the coupling block, B[b] = sum_t c_t Y[lm1_t], as one lane holds it for the whole kernel: lane L owns the
// entries L and L + 64.  The first two terms sit in registers (most entries have one or two); further terms, if a
// model file has them, are read from the lists in LDS.
struct BlockEntry {
    double c0, c1;
    int l0, l1, t2, t_end;
};
__device__ __forceinline__ BlockEntry block_entry(int b, int NB, const int* cg_start, const double* cg_c, const int* cg_lm1)
{
    BlockEntry e{0.0, 0.0, 0, 0, 0, 0};
    if (b < NB) {
        const int s0 = cg_start[b], s1 = cg_start[b + 1];
        if (s1 > s0) { e.c0 = cg_c[s0]; e.l0 = cg_lm1[s0]; e.l1 = e.l0; }
        if (s1 > s0 + 1) { e.c1 = cg_c[s0 + 1]; e.l1 = cg_lm1[s0 + 1]; }
        e.t2 = s0 + 2 < s1 ? s0 + 2 : s1;
        e.t_end = s1;
    }
    return e;
}

// ---------------------------------------------------------------------------
// (Hidden features up to l = 2: 17 paths and 71 sums per channel.  Those instantiations take one block per CU, so
// that a wavefront has the whole register file of its SIMD.)
template <typename F, int LMAXH, int CPL, int EC>
__global__ __launch_bounds__(256, LMAXH >= 2 ? 1 : 2) void k_agg_fwd(const AggParams<F> a, const int num_terms)
{
    using PT = Paths<LMAXH>;
    using WL = WaveLds<F, LMAXH, false>;
    constexpr int NB = PT::NB, NBP = WL::NBP, NE = PT::NE, P = PT::P, NLM = PT::NLM;
    extern __shared__ __align__(16) unsigned char smem[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    double* cg_c = reinterpret_cast<double*>(smem);                               // [num_terms]
    int* cg_lm1 = reinterpret_cast<int*>(cg_c + num_terms);                       // [num_terms]
    int* cg_start = cg_lm1 + num_terms;                                           // [NB+1]
    unsigned char* base = smem + WL::lists(num_terms) + (size_t)wave * WL::per_wave(EC);
    double* Yt = reinterpret_cast<double*>(base);                                 // [EC][16]
    double* xs = Yt + EC * 16;                                                    // [EC]
    F* Bs = reinterpret_cast<F*>(xs + EC);                                        // [EC][NBP]
    int* rows = reinterpret_cast<int*>(Bs + EC * NBP);                            // [EC]
    int* grows = rows + EC;                                                       // [EC]

    for (int t = threadIdx.x; t < num_terms; t += 256) { cg_c[t] = a.B_c[t]; cg_lm1[t] = a.B_lm1[t]; }
    for (int t = threadIdx.x; t <= NB; t += 256) cg_start[t] = a.B_start[t];
    __syncthreads();
    // lane-owned entries of the coupling block: measured faster in double precision; in single precision their
    // registers cost a wavefront per SIMD and the kernel runs 15 % slower
    constexpr bool OWNED = sizeof(F) == 8;
    constexpr int NSLOT = OWNED ? (NB + 63) / 64 : 1;
    BlockEntry ent[NSLOT];
    if constexpr (OWNED) {
#pragma unroll
        for (int j = 0; j < NSLOT; ++j) ent[j] = block_entry(lane + 64 * j, NB, cg_start, cg_c, cg_lm1);
    }

    const int K = a.K;
    // One-dimensional grid, channel group fastest: consecutive blocks go to the dies in turn, so a die only ever
    // works on the channel groups congruent to its number and its L2 holds that share of the spline table alone
    // (half of it at two groups of 64 channels).
    const int groups = (K + 64 * CPL - 1) / (64 * CPL);
    const int cgroup = blockIdx.x % groups;
    const int i = (blockIdx.x / groups) * 4 + wave;
    if (i >= a.num_nodes) return;
    const int k0 = (cgroup * 64 + lane) * CPL;
    const bool active = k0 < K;
    const int e0 = a.first_neigh[i], e1 = a.first_neigh[i + 1], ti = a.node_types[i];

    F acc[CPL][NE];
#pragma unroll
    for (int c = 0; c < CPL; ++c)
#pragma unroll
        for (int q = 0; q < NE; ++q) acc[c][q] = F(0);

    for (int eb = e0; eb < e1; eb += EC) {
        const int nE = min(EC, e1 - eb);
        wave_lds_sync();
        if (lane < nE) {
            const int e = eb + lane;
            const double dx = a.xyz[3 * (size_t)e], dy = a.xyz[3 * (size_t)e + 1], dz = a.xyz[3 * (size_t)e + 2];
            const double inv = rsqrt_pos(dx * dx + dy * dy + dz * dz);
            double Y[16];
            sph_l3(dz * inv, dx * inv, dy * inv, Y);
#pragma unroll
            for (int q = 0; q < 16; ++q) Yt[lane * 16 + q] = Y[q];
            const double r = a.r[e];
            const int n = spline_interval(r, a.spl_inv_h, a.spl_nodes - 2);
            xs[lane] = r - a.spl_h * n;
            const int tbl = a.pair_table[pair_index(a.T, ti, a.neigh_types[e])];
            rows[lane] = tbl * (a.spl_nodes - 1) + n;
            grows[lane] = a.gather[e];
        }
        wave_lds_sync();
        if constexpr (OWNED) {
#pragma unroll
            for (int j = 0; j < NSLOT; ++j) {
                const int b = lane + 64 * j;
                if (b < NB) {
                    const BlockEntry& en = ent[j];
                    for (int le = 0; le < nE; ++le) {
                        const double* y = Yt + le * 16;
                        double s = en.c0 * y[en.l0] + en.c1 * y[en.l1];
                        for (int t = en.t2; t < en.t_end; ++t) s += cg_c[t] * y[cg_lm1[t]];
                        Bs[le * NBP + b] = (F)s;
                    }
                }
            }
        } else {
            for (int it = lane; it < nE * NB; it += 64) {
                const int le = it / NB, b = it - le * NB;
                double s = 0.0;
                for (int t = cg_start[b]; t < cg_start[b + 1]; ++t) s += cg_c[t] * Yt[le * 16 + cg_lm1[t]];
                Bs[le * NBP + b] = (F)s;
            }
        }
        wave_lds_sync();
        if (!active) continue;
        // Spline coefficients (P x CPL 16-byte loads, contiguous across the lanes for one path) and the sender
        // row of an edge.  In single precision those of the next edge are requested while the current edge is
        // worked on (AHEAD).  In double precision there are registers for half of that at most (HALF: the first
        // five paths and the sender row requested an edge ahead, the other five at the start of the edge).
        constexpr bool AHEAD = sizeof(F) == 4 && (CPL == 1 || LMAXH == 0) && LMAXH <= 1;
        constexpr bool HALF = false;   // measured slower than requesting all ten at the start of the edge (10.4 against 9.1 ms)
        constexpr int PA = HALF ? P / 2 : P;     // paths of the first part
        Vec<F, 4> cf[P][CPL];
        Vec<F, CPL> H[NLM];
        auto request = [&](int le_, auto first, auto last, bool sender) {
            constexpr int p0 = decltype(first)::value, p1 = decltype(last)::value;
            const int row = __builtin_amdgcn_readfirstlane(rows[le_]);
            const F* rowp = a.tabK + ((size_t)row * P * K + k0) * 4;
            if (sender) {
                const int grow = __builtin_amdgcn_readfirstlane(grows[le_]);
                const F* Hp = a.Hsrc + (size_t)grow * NLM * K + k0;
#pragma unroll
                for (int q = 0; q < NLM; ++q) H[q] = ldv<F, CPL>(Hp + q * K);
            }
#pragma unroll
            for (int q = p0; q < p1; ++q)
#pragma unroll
                for (int c = 0; c < CPL; ++c) cf[q][c] = ldv<F, 4>(rowp + ((size_t)q * K + c) * 4);
        };
        constexpr std::integral_constant<int, 0> c0{};
        constexpr std::integral_constant<int, PA> cA{};
        constexpr std::integral_constant<int, P> cP{};
        if ((AHEAD || HALF) && nE > 0) request(0, c0, cA, true);
        F w[P][CPL][2 * LMAXH + 1];   // radial value times sender feature per path and sender component
        auto products = [&](F x, auto first, auto last) {
            static_for<decltype(first)::value, decltype(last)::value>([&](auto qc) {
                constexpr int q = decltype(qc)::value, l2 = PT::l2(q);
#pragma unroll
                for (int c = 0; c < CPL; ++c) {
                    const Vec<F, 4> k4 = cf[q][c];
                    const F R = k4.v[0] + x * (k4.v[1] + x * (k4.v[2] + x * k4.v[3]));
#pragma unroll
                    for (int m2 = 0; m2 < 2 * l2 + 1; ++m2) w[q][c][m2] = R * H[l2 * l2 + m2].v[c];
                }
            });
        };
        // coefficient buffer of this wavefront: [PRE paths][2 halves][64 lanes] 16-byte words
        unsigned char* pre = smem + WL::lists(num_terms) + 4 * WL::per_wave(EC) + (size_t)wave * WL::prefetch_per_wave();
        constexpr int PRE = WL::PRE;
        Vec<F, CPL> Hn[NLM];
        auto request_lds = [&](int le_) {
            typedef const __attribute__((address_space(1))) void* GlobalPtr;
            typedef __attribute__((address_space(3))) void* LdsPtr;
            const int row = __builtin_amdgcn_readfirstlane(rows[le_]);
            const char* rowp = reinterpret_cast<const char*>(a.tabK + ((size_t)row * P * K + k0) * 4);
#pragma unroll
            for (int q = 0; q < PRE; ++q) {
                const char* src = rowp + (size_t)q * K * 4 * sizeof(F);
                __builtin_amdgcn_global_load_lds((GlobalPtr)src, (LdsPtr)(pre + (q * 2) * 1024), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((GlobalPtr)(src + 16), (LdsPtr)(pre + (q * 2 + 1) * 1024), 16, 0, 0);
            }
            const int grow = __builtin_amdgcn_readfirstlane(grows[le_]);
            const F* Hp = a.Hsrc + (size_t)grow * NLM * K + k0;
#pragma unroll
            for (int q = 0; q < NLM; ++q) Hn[q] = ldv<F, CPL>(Hp + q * K);
        };
        if constexpr (WL::PREFETCH) {
            if (nE > 0) { request_lds(0); request(0, std::integral_constant<int, PRE>{}, std::integral_constant<int, P>{}, false); }
        }
        for (int le = 0; le < nE; ++le) {
            const F x = (F)xs[le];
            const F* B = Bs + le * NBP;
            auto accumulate = [&](auto pc) {
                constexpr int p = decltype(pc)::value;
                constexpr int l = PT::l(p), l2 = PT::l2(p), bo = PT::boff(p);
                constexpr int lme0 = PT::lme(p, 0), es = PT::num_e(l), n2 = 2 * l2 + 1;
                F Bv[(2 * l + 1) * n2];
#pragma unroll
                for (int q = 0; q < (2 * l + 1) * n2; ++q) Bv[q] = B[bo + q];
#pragma unroll
                for (int c = 0; c < CPL; ++c) {
#pragma unroll
                    for (int m = 0; m < 2 * l + 1; ++m) {
                        F z = acc[c][lme0 + m * es];
#pragma unroll
                        for (int m2 = 0; m2 < n2; ++m2) z += Bv[m * n2 + m2] * w[p][c][m2];
                        acc[c][lme0 + m * es] = z;
                    }
                }
            };
            // requests for a following edge are unconditional (the last edge of a chunk asks for its own operands
            // again): a conditional request makes the values carried round the loop a merge of old and new registers,
            // which costs a register copy per value
            const int le_next = le + 1 < nE ? le + 1 : le;
            if constexpr (WL::PREFETCH) {
                constexpr std::integral_constant<int, PRE> cPre{};
                // first paths from the buffer (filled while the previous edge was worked on), sender row likewise
#pragma unroll
                for (int q = 0; q < NLM; ++q) H[q] = Hn[q];
#pragma unroll
                for (int q = 0; q < PRE; ++q) {
                    const Vec<F, 2> lo = *reinterpret_cast<const Vec<F, 2>*>(pre + (q * 2) * 1024 + lane * 16);
                    const Vec<F, 2> hi = *reinterpret_cast<const Vec<F, 2>*>(pre + (q * 2 + 1) * 1024 + lane * 16);
                    cf[q][0].v[0] = lo.v[0]; cf[q][0].v[1] = lo.v[1]; cf[q][0].v[2] = hi.v[0]; cf[q][0].v[3] = hi.v[1];
                }
                products(x, c0, cPre);
                static_for<0, PRE>(accumulate);
                products(x, cPre, cP);                    // the other paths came through registers, requested an edge ago
                // the next edge's operands: first paths into the buffer (these requests are the older ones, so the
                // wait for them at the top of the next edge leaves the register loads in flight), the rest into the
                // registers the products above have just freed
                request_lds(le_next);
                request(le_next, cPre, cP, false);
                static_for<PRE, P>(accumulate);
                continue;
            }
            if (!AHEAD && !HALF) request(le, c0, cP, true);
            if (HALF) request(le, cA, cP, false);
            products(x, c0, cA);
            if (AHEAD) request(le_next, c0, cP, true);
            static_for<0, PA>(accumulate);
            if constexpr (HALF) {
                products(x, cA, cP);
                request(le_next, c0, cA, true);
                static_for<PA, P>(accumulate);
            }
        }
    }
    if (active) {
#pragma unroll
        for (int q = 0; q < NE; ++q) {
            Vec<F, CPL> o;
#pragma unroll
            for (int c = 0; c < CPL; ++c) o.v[c] = acc[c][q];
            *reinterpret_cast<Vec<F, CPL>*>(a.out + ((size_t)i * NE + q) * K + k0) = o;
        }
    }
}

// ---------------------------------------------------------------------------
// Adjoint: per edge force -dE/dxyz_ij (MACE::reverse_A0, mace.cpp:238-269;
// MACE::reverse_Phi1, mace.cpp:531-574) and the adjoint message to the sender
// row (mace.cpp:579-604), staged per edge for the deterministic sender-side sum.
// With more than one channel group each group writes its share
// of the force to fpart[group][edge][3]; the caller adds the groups up.
template <typename F, int LMAXH, int CPL, int EC>
__global__ __launch_bounds__(256, LMAXH >= 2 ? 1 : 2) void k_agg_bwd(const AggParams<F> a, const int num_terms)
{
    using PT = Paths<LMAXH>;
    using WL = WaveLds<F, LMAXH, true>;
    constexpr int NB = PT::NB, NBP = WL::NBP, NE = PT::NE, P = PT::P, NLM = PT::NLM;
    extern __shared__ __align__(16) unsigned char smem[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    double* cg_c = reinterpret_cast<double*>(smem);
    int* cg_lm1 = reinterpret_cast<int*>(cg_c + num_terms);
    int* cg_start = cg_lm1 + num_terms;
    unsigned char* base = smem + WL::lists(num_terms) + (size_t)wave * WL::per_wave(EC);
    // the B block below is read with 4 * sizeof(F)-byte accesses: the doubles in front of it must keep that alignment
    static_assert((EC * (64 + 12 + 1) * sizeof(double)) % (4 * sizeof(F)) == 0, "chunk size breaks the alignment of the B block");
    double* Yt = reinterpret_cast<double*>(base);                                 // [EC][4][16]: Y, dY/dx, dY/dy, dY/dz
    double* us = Yt + EC * 64;                                                    // [EC][12]: xyz/r, -, tangent t1, tangent t2, -, -
    double* xs = us + EC * 12;                                                    // [EC]
    // The harmonics depend on the direction only, so their gradient is tangential: two components in a frame
    // (t1, t2) orthogonal to the direction carry it, and the contraction below costs three multiply-adds per
    // entry instead of four.
    F* Bs = reinterpret_cast<F*>(xs + EC);                                        // [EC][NBP][4]: B, dB.t1, dB.t2, -
    int* rows = reinterpret_cast<int*>(Bs + EC * 4 * NBP);
    int* grows = rows + EC;

    for (int t = threadIdx.x; t < num_terms; t += 256) { cg_c[t] = a.B_c[t]; cg_lm1[t] = a.B_lm1[t]; }
    for (int t = threadIdx.x; t <= NB; t += 256) cg_start[t] = a.B_start[t];
    __syncthreads();
    // lane-owned entries of the coupling block (registers for them exist in single precision only)
    constexpr bool OWNED = sizeof(F) == 4;
    constexpr int NSLOT = OWNED ? (NB + 63) / 64 : 1;
    BlockEntry ent[NSLOT];
    if constexpr (OWNED) {
#pragma unroll
        for (int j = 0; j < NSLOT; ++j) ent[j] = block_entry(lane + 64 * j, NB, cg_start, cg_c, cg_lm1);
    }

    const int K = a.K;
    // one-dimensional grid, channel group fastest (see k_agg_fwd)
    const int groups = (K + 64 * CPL - 1) / (64 * CPL);
    const int cgroup = blockIdx.x % groups;
    const int i = a.node_begin + (blockIdx.x / groups) * 4 + wave;
    if (i >= a.num_nodes) return;
    // Lanes beyond the last channel work on channel 0 with a zero adjoint (all their sums are zero) and skip the
    // message store: no branch on the lane's channel inside the edge loop, hence no merges of old and new registers.
    const bool active = (cgroup * 64 + lane) * CPL < K;
    const int k0 = active ? (cgroup * 64 + lane) * CPL : 0;
    const int e0 = a.first_neigh[i], e1 = a.first_neigh[i + 1], ti = a.node_types[i];
    double* fout = groups > 1 ? a.fpart + (size_t)cgroup * 3 * a.num_edges : a.forces;
    const bool add_forces = groups == 1 && a.accumulate_forces;

    F d[CPL][NE];
#pragma unroll
    for (int q = 0; q < NE; ++q) {
        const Vec<F, CPL> v = ldv<F, CPL>(a.d_out + ((size_t)i * NE + q) * K + k0);
#pragma unroll
        for (int c = 0; c < CPL; ++c) d[c][q] = active ? v.v[c] : F(0);
    }

    for (int eb = e0; eb < e1; eb += EC) {
        const int nE = min(EC, e1 - eb);
        wave_lds_sync();
        if (lane < nE) {
            const int e = eb + lane;
            const double dx = a.xyz[3 * (size_t)e], dy = a.xyz[3 * (size_t)e + 1], dz = a.xyz[3 * (size_t)e + 2];
            const double inv = rsqrt_pos(dx * dx + dy * dy + dz * dz);
            sph_l3_grad_store<16>(dz * inv, dx * inv, dy * inv, inv, Yt + lane * 64);
            const double r = a.r[e];
            // radial direction as the reference forms it: xyz / r with the caller's r
            const double ir = rcp_pos(r);
            us[lane * 12] = dx * ir; us[lane * 12 + 1] = dy * ir; us[lane * 12 + 2] = dz * ir;
            {
                // t1 = n x a / |n x a| with a the axis the direction n is least aligned with (|n x a|^2 >= 2/3), t2 = n x t1
                const double nx = dx * inv, ny = dy * inv, nz = dz * inv;
                const double ax = fabs(nx), ay = fabs(ny), az = fabs(nz);
                double t1x, t1y, t1z;
                if (ax <= ay && ax <= az) { t1x = 0.0; t1y = nz; t1z = -ny; }
                else if (ay <= az) { t1x = -nz; t1y = 0.0; t1z = nx; }
                else { t1x = ny; t1y = -nx; t1z = 0.0; }
                const double tn = rsqrt_pos(t1x * t1x + t1y * t1y + t1z * t1z);
                t1x *= tn; t1y *= tn; t1z *= tn;
                double* fr = us + lane * 12 + 4;
                fr[0] = t1x; fr[1] = t1y; fr[2] = t1z;
                fr[3] = ny * t1z - nz * t1y; fr[4] = nz * t1x - nx * t1z; fr[5] = nx * t1y - ny * t1x;
            }
            const int n = spline_interval(r, a.spl_inv_h, a.spl_nodes - 2);
            xs[lane] = r - a.spl_h * n;
            const int tbl = a.pair_table[pair_index(a.T, ti, a.neigh_types[e])];
            rows[lane] = tbl * (a.spl_nodes - 1) + n;
            grows[lane] = a.gather[e];
        }
        wave_lds_sync();
        if constexpr (OWNED) {
#pragma unroll
            for (int j = 0; j < NSLOT; ++j) {
                const int b = lane + 64 * j;
                if (b < NB) {
                    const BlockEntry& en = ent[j];
                    for (int le = 0; le < nE; ++le) {
                        const double* y0 = Yt + le * 64 + en.l0;
                        const double* y1 = Yt + le * 64 + en.l1;
                        double s = en.c0 * y0[0] + en.c1 * y1[0], sx = en.c0 * y0[16] + en.c1 * y1[16];
                        double sy = en.c0 * y0[32] + en.c1 * y1[32], sz = en.c0 * y0[48] + en.c1 * y1[48];
                        for (int t = en.t2; t < en.t_end; ++t) {
                            const double cc = cg_c[t];
                            const double* y = Yt + le * 64 + cg_lm1[t];
                            s += cc * y[0]; sx += cc * y[16]; sy += cc * y[32]; sz += cc * y[48];
                        }
                        const double* fr = us + le * 12 + 4;
                        Vec<F, 4> o;
                        o.v[0] = (F)s;
                        o.v[1] = (F)(sx * fr[0] + sy * fr[1] + sz * fr[2]);
                        o.v[2] = (F)(sx * fr[3] + sy * fr[4] + sz * fr[5]);
                        o.v[3] = F(0);
                        *reinterpret_cast<Vec<F, 4>*>(Bs + ((size_t)le * NBP + b) * 4) = o;
                    }
                }
            }
        } else {
        for (int it = lane; it < nE * NB; it += 64) {
            const int le = it / NB, b = it - le * NB;
            double s = 0.0, sx = 0.0, sy = 0.0, sz = 0.0;
            for (int t = cg_start[b]; t < cg_start[b + 1]; ++t) {
                const double cc = cg_c[t];
                const double* y = Yt + le * 64 + cg_lm1[t];
                s += cc * y[0]; sx += cc * y[16]; sy += cc * y[32]; sz += cc * y[48];
            }
            const double* fr = us + le * 12 + 4;
            Vec<F, 4> o;
            o.v[0] = (F)s;
            o.v[1] = (F)(sx * fr[0] + sy * fr[1] + sz * fr[2]);
            o.v[2] = (F)(sx * fr[3] + sy * fr[4] + sz * fr[5]);
            o.v[3] = F(0);
            *reinterpret_cast<Vec<F, 4>*>(Bs + ((size_t)le * NBP + b) * 4) = o;
        }
        }
        wave_lds_sync();
        // Spline coefficients of one edge: P x CPL 16-byte loads, contiguous across the lanes for one path.  In single
        // precision the next edge's coefficients are requested while the current edge is worked on (40
        // registers in flight); in double precision they are requested together at the start of the edge.
        constexpr bool AHEAD = sizeof(F) == 4 && LMAXH <= 1;
        Vec<F, 4> cf[P][CPL];
        auto load_cf = [&](int le_) {
            const int row = __builtin_amdgcn_readfirstlane(rows[le_]);
            const F* rowp = a.tabK + ((size_t)row * P * K + k0) * 4;
#pragma unroll
            for (int q = 0; q < P; ++q)
#pragma unroll
                for (int c = 0; c < CPL; ++c) cf[q][c] = ldv<F, 4>(rowp + ((size_t)q * K + c) * 4);
        };
        if (AHEAD && nE > 0) load_cf(0);
        // One edge.  The loop below runs it with the request for the next edge's coefficients for all edges but the
        // last of the chunk, which runs without: a request under a condition inside one loop body would make the
        // coefficients carried round the loop a merge of old and new registers (a register copy per value and edge).
        auto edge = [&](const int le, auto ahead) {
            F srad = F(0), g1 = F(0), g2 = F(0);
            {
                const F x = (F)xs[le];
                const int grow = __builtin_amdgcn_readfirstlane(grows[le]);
                // element offset of this edge's B block; it passes through the fences below, which keep the
                // LDS reads of a group behind the arithmetic of the group before it (all reads at once would
                // need several hundred registers)
                int boffs = le * 4 * NBP;
                const F* Hp = a.Hsrc + (size_t)grow * NLM * K + k0;
                Vec<F, CPL> H[NLM], mg[NLM];
#pragma unroll
                for (int q = 0; q < NLM; ++q) {
                    H[q] = ldv<F, CPL>(Hp + q * K);
#pragma unroll
                    for (int c = 0; c < CPL; ++c) mg[q].v[c] = F(0);
                }
                if (!AHEAD) load_cf(le);
                F Rv[P][CPL], Rdv[P][CPL];
#pragma unroll
                for (int q = 0; q < P; ++q)
#pragma unroll
                    for (int c = 0; c < CPL; ++c) {
                        const Vec<F, 4> k4 = cf[q][c];
                        Rv[q][c] = k4.v[0] + x * (k4.v[1] + x * (k4.v[2] + x * k4.v[3]));
                        Rdv[q][c] = k4.v[1] + x * (F(2) * k4.v[2] + F(3) * x * k4.v[3]);
                    }
                if constexpr (AHEAD && decltype(ahead)::value) load_cf(le + 1);
                // The B block of the edge is walked in steps (a few rows m of one path each).  Per path, the rows
                // are summed first, u[m2][comp] = sum_m d[m] * (B, dB.t1, dB.t2)[m][m2], then one product
                // with the sender feature per m2.  The LDS reads of the next step are issued before the
                // arithmetic of the current one (two register buffers); the fence after each step keeps
                // reads further ahead from being issued (all at once would need several hundred registers).
                using ST = BwdSteps<LMAXH, sizeof(F) == 8>;
                constexpr bool LOOKAHEAD = true;
                Vec<F, 4> buf[LOOKAHEAD ? 2 : 1][ST::MAXLEN];
                F u[CPL][2 * LMAXH + 1][3];
                auto load_step = [&](auto sc, Vec<F, 4>* dst) {
                    // (every table lookup lands in a constexpr variable: left to the optimizer, the path tables of the
                    // l = 2 instantiation stay behind as loops that run on the device)
                    constexpr int s = decltype(sc)::value, p = ST::path(s), n2 = 2 * PT::l2(p) + 1, len = ST::len(s);
                    constexpr int first = (PT::boff(p) + ST::m0(s) * n2) * 4;
                    const F* B4 = Bs + boffs + first;
#pragma unroll
                    for (int q = 0; q < len; ++q) dst[q] = ldv<F, 4>(B4 + 4 * q);
                };
                if constexpr (LOOKAHEAD) load_step(std::integral_constant<int, 0>{}, buf[0]);
                static_for<0, ST::count()>([&](auto sc) {
                    constexpr int s = decltype(sc)::value, p = ST::path(s), m0 = ST::m0(s), m1 = ST::m1(s);
                    constexpr int l = PT::l(p), l2 = PT::l2(p);
                    constexpr int lme0 = PT::lme(p, 0), es = PT::num_e(l), n2 = 2 * l2 + 1;
                    Vec<F, 4>* b4 = buf[LOOKAHEAD ? (s & 1) : 0];
                    if constexpr (!LOOKAHEAD) load_step(sc, b4);
                    else if constexpr (s + 1 < ST::count()) load_step(std::integral_constant<int, s + 1>{}, buf[(s + 1) & 1]);
#pragma unroll
                    for (int c = 0; c < CPL; ++c) {
#pragma unroll
                        for (int m = m0; m < m1; ++m) {
                            const F dd = d[c][lme0 + m * es];
#pragma unroll
                            for (int m2 = 0; m2 < n2; ++m2) {
                                const Vec<F, 4>& bb = b4[(m - m0) * n2 + m2];
                                // the unused fourth word counts as used where the others are: the read stays a 16-byte
                                // one (a 12-byte LDS read is slower) and is not waited for any earlier
                                asm volatile("" : : "v"(bb.v[3]));
#pragma unroll
                                for (int t = 0; t < 3; ++t)   // the first row of a path starts the sums
                                    u[c][m2][t] = m == 0 ? dd * bb.v[t] : u[c][m2][t] + dd * bb.v[t];
                            }
                        }
                    }
#pragma unroll
                    for (int c = 0; c < CPL; ++c)
#pragma unroll
                        for (int m2 = 0; m2 < n2; ++m2)
#pragma unroll
                            for (int t = 0; t < 3; ++t) tie(u[c][m2][t], boffs);
                    if constexpr (m1 == 2 * l + 1) {
#pragma unroll
                        for (int c = 0; c < CPL; ++c) {
                            const F R = Rv[p][c], Rd = Rdv[p][c];
                            F s0 = F(0), s1 = F(0), s2 = F(0);
#pragma unroll
                            for (int m2 = 0; m2 < n2; ++m2) {
                                const F h = H[l2 * l2 + m2].v[c];
                                s0 += u[c][m2][0] * h; s1 += u[c][m2][1] * h; s2 += u[c][m2][2] * h;
                                mg[l2 * l2 + m2].v[c] += R * u[c][m2][0];
                            }
                            srad += Rd * s0;
                            g1 += R * s1; g2 += R * s2;
                        }
                        order_after(g1, g2, srad, boffs);
#pragma unroll
                        for (int m2 = 0; m2 < n2; ++m2)
#pragma unroll
                            for (int c = 0; c < CPL; ++c) pin(mg[l2 * l2 + m2].v[c]);
                    }
                });
                if (a.msg && active) {
                    F* mrow = a.msg + (size_t)(eb + le - a.msg_edge_begin) * NLM * K + k0;
#pragma unroll
                    for (int q = 0; q < NLM; ++q) *reinterpret_cast<Vec<F, CPL>*>(mrow + q * K) = mg[q];
                }
            }
            // Sums over the channels of the wavefront (a fixed tree: bit-reproducible): the radial sum and the two
            // tangential ones, in the feature precision; the force is put together from them in double.
            const double sr = (double)wave_sum(srad), G1 = (double)wave_sum(g1), G2 = (double)wave_sum(g2);
            const double* uf = us + le * 12;
            const double fx = -(uf[0] * sr + uf[4] * G1 + uf[7] * G2);
            const double fy = -(uf[1] * sr + uf[5] * G1 + uf[8] * G2);
            const double fz = -(uf[2] * sr + uf[6] * G1 + uf[9] * G2);
            if (lane == 0) {
                double* f = fout + 3 * (size_t)(eb + le);
                if (add_forces) { f[0] += fx; f[1] += fy; f[2] += fz; }
                else { f[0] = fx; f[1] = fy; f[2] = fz; }
            }
        };
        if constexpr (AHEAD) {
            for (int le = 0; le + 1 < nE; ++le) edge(le, std::true_type{});
            if (nE > 0) edge(nE - 1, std::false_type{});
        } else {
            // one copy of the edge's code: the unrolled walk of the coupling block is tens of KB of instructions, and
            // a chunk's whole code path has to stay inside the instruction cache
            for (int le = 0; le < nE; ++le) edge(le, std::false_type{});
        }
    }
}

template <typename F, int LMAXH, int CPL, int EC, bool BWD>
hipError_t launch_agg_t(const AggParams<F>& p, hipStream_t s)
{
    using WL = WaveLds<F, LMAXH, BWD>;
    const int groups = (p.K + 64 * CPL - 1) / (64 * CPL);
    if (p.K % CPL != 0) return hipErrorInvalidValue;
    if (BWD && groups > 1 && !p.fpart) return hipErrorInvalidValue;
    const size_t lds = WL::lists(p.num_terms) + 4 * WL::per_wave(EC) + 4 * WL::prefetch_per_wave();
    if (!BWD && (p.node_begin != 0 || p.msg_edge_begin != 0)) return hipErrorInvalidValue;
    if (p.node_begin < 0 || p.node_begin > p.num_nodes) return hipErrorInvalidValue;
    const long blocks = (long)((p.num_nodes - p.node_begin + 3) / 4) * groups;
    if (blocks == 0) return hipSuccess;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    dim3 grid((unsigned)blocks);
    void (*kern)(const AggParams<F>, const int);
    if constexpr (BWD) kern = k_agg_bwd<F, LMAXH, CPL, EC>;
    else kern = k_agg_fwd<F, LMAXH, CPL, EC>;
    if (lds > 64 * 1024) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
    }
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, p, p.num_terms);
    return hipGetLastError();
}

// Channels per lane.  Two give paired loads and fewer broadcast reads per channel; the l <= 1 path list holds
// 40 accumulators per channel, which leaves room for two channels only in the single-precision forward kernel.
template <typename F, int LMAXH, bool BWD>
int agg_cpl(int K)
{
    const bool wide = LMAXH == 0;
    return (wide && K > 64 && K % 2 == 0) ? 2 : 1;
}

template <typename F, int LMAXH, bool BWD>
hipError_t launch_agg_sel(const AggParams<F>& p, hipStream_t s)
{
    // edges per chunk; the double-precision forward kernel of the ten-path list takes eight so that two blocks with
    // their coefficient buffers fit a CU
    // (l = 2 hidden features: the coupling block has 243 entries per edge, four edges of the adjoint fill the LDS share of a wavefront)
    constexpr int EC = LMAXH == 0 ? 16 : (BWD ? (sizeof(F) == 4 && LMAXH == 1 ? 8 : 4) : (sizeof(F) == 8 ? 8 : 16));
    // two channels per lane exist for the four-path list only (the ten-path kernels have no registers for them)
    if constexpr (LMAXH == 0) {
        if (agg_cpl<F, LMAXH, BWD>(p.K) == 2) return launch_agg_t<F, LMAXH, 2, EC, BWD>(p, s);
    }
    return launch_agg_t<F, LMAXH, 1, EC, BWD>(p, s);
}

}  // namespace

template <typename F>
hipError_t launch_agg_fwd(int L_max_H, const AggParams<F>& p, hipStream_t s)
{
    if (L_max_H == 0) return launch_agg_sel<F, 0, false>(p, s);
    if (L_max_H == 1) return launch_agg_sel<F, 1, false>(p, s);
    if (L_max_H == 2) return launch_agg_sel<F, 2, false>(p, s);
    return hipErrorInvalidValue;
}
template <typename F>
hipError_t launch_agg_bwd(int L_max_H, const AggParams<F>& p, hipStream_t s)
{
    if (L_max_H == 0) return launch_agg_sel<F, 0, true>(p, s);
    if (L_max_H == 1) return launch_agg_sel<F, 1, true>(p, s);
    if (L_max_H == 2) return launch_agg_sel<F, 2, true>(p, s);
    return hipErrorInvalidValue;
}
template <typename F>
int agg_bwd_groups(int L_max_H, int K)
{
    const int cpl = L_max_H == 0 ? agg_cpl<F, 0, true>(K) : 1;
    return (K + 64 * cpl - 1) / (64 * cpl);
}
// This file is compiled four times (SMX_EDGE_PART = 0..3), one object per
// precision and direction, so that the instantiations build in parallel.
#ifndef SMX_EDGE_PART
#error "define SMX_EDGE_PART (0: fwd double + helpers, 1: fwd float, 2: bwd double, 3: bwd float)"
#endif
#if SMX_EDGE_PART == 0
template hipError_t launch_agg_fwd<double>(int, const AggParams<double>&, hipStream_t);
#elif SMX_EDGE_PART == 1
template hipError_t launch_agg_fwd<float>(int, const AggParams<float>&, hipStream_t);
#elif SMX_EDGE_PART == 2
template hipError_t launch_agg_bwd<double>(int, const AggParams<double>&, hipStream_t);
template int agg_bwd_groups<double>(int, int);
#else
template hipError_t launch_agg_bwd<float>(int, const AggParams<float>&, hipStream_t);
template int agg_bwd_groups<float>(int, int);
#endif

#if SMX_EDGE_PART == 0

// ---------------------------------------------------------------------------
namespace {
// V consecutive elements per thread (16-byte accesses when the row width allows); four messages are requested
// before the first is added, the additions keep the ascending edge order
template <typename F, int V>
__global__ void k_sender_reduce(int rows, int width, const int* sstart, const int* slist, const F* msg,
                                F* H_adj, int zero_first, long e_lo, long e_hi)
{
    const int j = blockIdx.x;
    int s0 = sstart[j], s1 = sstart[j + 1];
    // the sender's edges are listed in ascending order: narrow to those inside [e_lo, e_hi)
    while (s0 < s1 && slist[s0] < e_lo) ++s0;
    while (s1 > s0 && slist[s1 - 1] >= e_hi) --s1;
    if (s0 == s1 && !zero_first) return;
    for (int q = threadIdx.x * V; q < width; q += blockDim.x * V) {
        Vec<F, V> acc;
        if (zero_first) {
#pragma unroll
            for (int c = 0; c < V; ++c) acc.v[c] = F(0);
        } else {
            acc = ldv<F, V>(H_adj + (size_t)j * width + q);
        }
        int t = s0;
        for (; t + 4 <= s1; t += 4) {
            Vec<F, V> m[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) m[i] = ldv<F, V>(msg + (size_t)(slist[t + i] - e_lo) * width + q);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int c = 0; c < V; ++c) acc.v[c] += m[i].v[c];
        }
        for (; t < s1; ++t) {
            const Vec<F, V> m = ldv<F, V>(msg + (size_t)(slist[t] - e_lo) * width + q);
#pragma unroll
            for (int c = 0; c < V; ++c) acc.v[c] += m.v[c];
        }
        *reinterpret_cast<Vec<F, V>*>(H_adj + (size_t)j * width + q) = acc;
    }
}
}  // namespace

template <typename F>
hipError_t launch_sender_reduce(int rows, int width, const int* sstart, const int* slist, const F* msg,
                                F* H_adj, int zero_first, long e_lo, long e_hi, hipStream_t s)
{
    if (rows <= 0) return hipSuccess;
    constexpr int V = 16 / (int)sizeof(F);
    if (width % V == 0) {
        const int lanes = width / V;
        const int bs = lanes <= 64 ? 64 : (lanes <= 128 ? 128 : 256);
        hipLaunchKernelGGL((k_sender_reduce<F, V>), dim3(rows), dim3(bs), 0, s, rows, width, sstart, slist, msg, H_adj,
                           zero_first, e_lo, e_hi);
    } else {
        const int bs = width <= 64 ? 64 : (width <= 128 ? 128 : 256);
        hipLaunchKernelGGL((k_sender_reduce<F, 1>), dim3(rows), dim3(bs), 0, s, rows, width, sstart, slist, msg, H_adj,
                           zero_first, e_lo, e_hi);
    }
    return hipGetLastError();
}
// ---------------------------------------------------------------------------
// The sender-side sum followed by reverse_H1 for scalar hidden features (mace.cpp:402-436 with one block of
// H1): a block of 16 wavefronts sums the messages of 16 consecutive sender rows (wavefront w takes row w, in
// ascending edge order as above), keeps the finished rows in LDS as doubles, and forms
// M0_adj = H1_adj . W^T for them on the matrix cores; wavefront w owns column tile w, its weight operands
// (32 contiguous bytes per lane, k permuted inside groups of 16 on both operands) are requested before the
// sums start.
namespace {
typedef double f64x4_t __attribute__((ext_vector_type(4)));
template <typename F, int KT>
__global__ __launch_bounds__(1024) void k_sender_reduce_linear(int rows, const int* sstart, const int* slist, const F* msg,
                                                              F* H_adj, int zero_first, const F* W, F* M_adj)
{
    constexpr int K = 16 * KT, ld = K + 1, V = 16 / (int)sizeof(F);
    __shared__ double X[16 * ld];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.x * 16;
    const bool owner = wave < KT;
    f64x4_t wv[KT];
    if (owner) {
#pragma unroll
        for (int j = 0; j < KT; ++j) {
            const Vec<F, 4> t = ldv<F, 4>(W + (size_t)(wave * 16 + r) * K + 16 * j + 4 * g);
#pragma unroll
            for (int c = 0; c < 4; ++c) wv[j][c] = (double)t.v[c];
        }
    }
    {
        const int rr = wave, j = row0 + rr;
        const int q = lane * V;
        if (q < K) {
            Vec<F, V> acc;
#pragma unroll
            for (int c = 0; c < V; ++c) acc.v[c] = F(0);
            if (j < rows) {
                const int s0 = sstart[j], s1 = sstart[j + 1];
                if (!zero_first) acc = ldv<F, V>(H_adj + (size_t)j * K + q);
                int t = s0;
                for (; t + 4 <= s1; t += 4) {
                    Vec<F, V> m[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) m[i] = ldv<F, V>(msg + (size_t)slist[t + i] * K + q);
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int c = 0; c < V; ++c) acc.v[c] += m[i].v[c];
                }
                for (; t < s1; ++t) {
                    const Vec<F, V> m = ldv<F, V>(msg + (size_t)slist[t] * K + q);
#pragma unroll
                    for (int c = 0; c < V; ++c) acc.v[c] += m.v[c];
                }
                *reinterpret_cast<Vec<F, V>*>(H_adj + (size_t)j * K + q) = acc;
            }
#pragma unroll
            for (int c = 0; c < V; ++c) X[rr * ld + q + c] = (double)acc.v[c];
        }
    }
    __syncthreads();
    if (owner) {
        f64x4_t acc = {0, 0, 0, 0};
        const double* a = X + r * ld + 4 * g;
#pragma unroll
        for (int j = 0; j < KT; ++j)
#pragma unroll
            for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f64_16x16x4f64(a[16 * j + t], wv[j][t], acc, 0, 0, 0);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int j = row0 + 4 * q + g;
            if (j < rows) M_adj[(size_t)j * K + wave * 16 + r] = (F)acc[q];
        }
    }
}
}  // namespace

bool sender_reduce_linear_ok(int K) { return K == 32 || K == 48 || K == 64 || K == 96 || K == 128; }

template <typename F>
hipError_t launch_sender_reduce_linear(int rows, int K, const int* sstart, const int* slist, const F* msg, F* H_adj,
                                       int zero_first, const F* W, F* M_adj, hipStream_t s)
{
    if (!sender_reduce_linear_ok(K)) return hipErrorInvalidValue;
    if (rows <= 0) return hipSuccess;
    const dim3 grid((unsigned)((rows + 15) / 16)), block(1024);
    switch (K / 16) {
    case 2: hipLaunchKernelGGL((k_sender_reduce_linear<F, 2>), grid, block, 0, s, rows, sstart, slist, msg, H_adj, zero_first, W, M_adj); break;
    case 3: hipLaunchKernelGGL((k_sender_reduce_linear<F, 3>), grid, block, 0, s, rows, sstart, slist, msg, H_adj, zero_first, W, M_adj); break;
    case 4: hipLaunchKernelGGL((k_sender_reduce_linear<F, 4>), grid, block, 0, s, rows, sstart, slist, msg, H_adj, zero_first, W, M_adj); break;
    case 6: hipLaunchKernelGGL((k_sender_reduce_linear<F, 6>), grid, block, 0, s, rows, sstart, slist, msg, H_adj, zero_first, W, M_adj); break;
    default: hipLaunchKernelGGL((k_sender_reduce_linear<F, 8>), grid, block, 0, s, rows, sstart, slist, msg, H_adj, zero_first, W, M_adj); break;
    }
    return hipGetLastError();
}
template hipError_t launch_sender_reduce_linear<double>(int, int, const int*, const int*, const double*, double*, int, const double*, double*, hipStream_t);
template hipError_t launch_sender_reduce_linear<float>(int, int, const int*, const int*, const float*, float*, int, const float*, float*, hipStream_t);

template hipError_t launch_sender_reduce<double>(int, int, const int*, const int*, const double*, double*, int, long, long, hipStream_t);
template hipError_t launch_sender_reduce<float>(int, int, const int*, const int*, const float*, float*, int, long, long, hipStream_t);

// ---------------------------------------------------------------------------
namespace {
__global__ void k_sph_harm(const double* xyz, long E, double* Y, double* Yg)
{
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    const double dx = xyz[3 * e], dy = xyz[3 * e + 1], dz = xyz[3 * e + 2];
    const double inv = rsqrt_pos(dx * dx + dy * dy + dz * dz);
    double y[16], G[3][16];
    sph_l3_grad(dz * inv, dx * inv, dy * inv, inv, y, G);
    for (int q = 0; q < 16; ++q) {
        Y[e * 16 + q] = y[q];
        Yg[e * 48 + q] = G[0][q];
        Yg[e * 48 + 16 + q] = G[1][q];
        Yg[e * 48 + 32 + q] = G[2][q];
    }
}

template <typename F>
__global__ void k_radial(int N, const int* first_neigh, const int* node_types, const int* neigh_types,
                         const double* r, const F* tab, const int* pair_table, int T, int nodes, double h,
                         int nspl, double* R)
{
    const int i = blockIdx.x;
    const int ti = node_types[i];
    for (int e = first_neigh[i]; e < first_neigh[i + 1]; ++e) {
        const double rr = r[e];
        int n = (int)(rr / h);
        n = min(max(n, 0), nodes - 2);
        const F x = (F)(rr - h * n);
        const F* row = tab + ((size_t)pair_table[pair_index(T, ti, neigh_types[e])] * (nodes - 1) + n) * 4 * nspl;
        for (int j = threadIdx.x; j < nspl; j += blockDim.x) {
            const F v = row[j] + x * (row[nspl + j] + x * (row[2 * nspl + j] + x * row[3 * nspl + j]));
            R[(size_t)e * nspl + j] = (double)v;
        }
    }
}
}  // namespace

hipError_t launch_sph_harm(const double* xyz, long E, double* Y, double* Y_grad, hipStream_t s)
{
    if (E <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_sph_harm, dim3((unsigned)((E + 127) / 128)), dim3(128), 0, s, xyz, E, Y, Y_grad);
    return hipGetLastError();
}

template <typename F>
hipError_t launch_radial(int N, const int* first_neigh, const int* node_types, const int* neigh_types,
                         const double* r, const F* tab, const int* pair_table, int T, int nodes, double h,
                         int nspl, double* R, hipStream_t s)
{
    if (N <= 0) return hipSuccess;
    hipLaunchKernelGGL(k_radial<F>, dim3(N), dim3(128), 0, s, N, first_neigh, node_types, neigh_types, r, tab,
                       pair_table, T, nodes, h, nspl, R);
    return hipGetLastError();
}
template hipError_t launch_radial<double>(int, const int*, const int*, const int*, const double*, const double*, const int*, int, int, double, int, double*, hipStream_t);
template hipError_t launch_radial<float>(int, const int*, const int*, const int*, const double*, const float*, const int*, int, int, double, int, double*, hipStream_t);

#endif  // SMX_EDGE_PART == 0

}  // namespace smx
