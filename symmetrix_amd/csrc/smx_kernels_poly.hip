// Symmetric contraction for the standard product basis on gfx950 (MACE::compute_M0 / compute_M1 and their
// adjoints, libsymmetrix/source/mace.cpp:349-395, 760-807, with the polynomial of
// multivariate_polynomial.cpp:10-101 walked from compile-time monomial lists).
// Compiled in two parts (SMX_POLY_PART = 0: double, 1: float) so that the parts build side by side.
#include "smx_device.hpp"
#include "smx_kernels.hpp"

#include <algorithm>
#include <type_traits>

namespace smx {

namespace {
// For harmonics up to l = 3 and correlation order 3 the monomials of output slot LM are a compile-time table
// (smx_poly_tables.inc), so the walk is straight-line code and the 16 variables of an atom stay in registers -- no
// index loads, no variables in LDS.  The LDS holds the coefficients instead: a block owns one species and one block
// of CB channels, copies that slab ([monomials of all polynomials][CB], laid out by the loader as 16-byte groups per
// channel, see poly_spec_shape) once and then takes a run of `chunk` atoms of the species, AG atoms at a time, one
// thread per (atom, channel).  Per monomial x_a x_b x_c the thread forms w x_a and x_b x_c once; three multiply-adds
// give the gradient terms (the product rule holds as written for repeated indices) and one more the value: six
// instructions.  Used when every polynomial of the launch maps onto its table (the loader checks); other files take
// the list-walking kernel of smx_kernels_node.hip.
template <typename F> __device__ __forceinline__ void pin_reg(F& v) { asm volatile("" : "+v"(v)); }
template <typename F> constexpr int spec_group() { return sizeof(F) == 8 ? 4 : 8; }   // coefficients per request
constexpr int SPEC_BT = 256;     // threads per block

// MODE 0: values and gradients (M, M_grad); 1: values only; 2: adjoint, A_adj = sum over the polynomials of
// M_adj[polynomial] * gradient, recomputed from the variables (the coefficient is scaled, the value dropped).
template <typename F, int LM, int MODE>
__device__ __forceinline__ void poly_spec_body(const unsigned char* slab_k, int row_stride_bytes, F (&x)[16], F (&g)[16], F& f,
                                               F madj)
{
    using TB = PolyTable<LM>;
    constexpr int V = 16 / (int)sizeof(F);
    typedef F V4 __attribute__((ext_vector_type(V)));
    constexpr int row0 = poly_spec_offset(LM) / V;   // first 16-byte group of this polynomial in the slab
    // Coefficients come in small groups: the next group is requested before the current one is used; compiler
    // and scheduling barriers keep all groups from being requested at once (the variables would spill).
    constexpr int G = spec_group<F>(), NG = (TB::N + G - 1) / G, RG = G / V;
    V4 wbuf[2][RG];
    auto request = [&](auto gc, V4 (&w)[RG]) {
        constexpr int r0 = decltype(gc)::value * RG;
#pragma unroll
        for (int j = 0; j < RG; ++j)
            if ((r0 + j) * V < poly_spec_padded(TB::N))
                w[j] = *reinterpret_cast<const V4*>(slab_k + (size_t)(row0 + r0 + j) * row_stride_bytes);
    };
    request(std::integral_constant<int, 0>{}, wbuf[0]);
    static_for<0, NG>([&](auto gc) {
        constexpr int gi = decltype(gc)::value;
        if constexpr (gi + 1 < NG) request(std::integral_constant<int, gi + 1>{}, wbuf[(gi + 1) & 1]);
        asm volatile("" ::: "memory");     // no read of a later group moves above this line
        __builtin_amdgcn_sched_barrier(0);
        static_for<gi * G, (gi * G + G < TB::N ? gi * G + G : TB::N)>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            constexpr int ia = TB::m[i][0], ib = TB::m[i][1], jc = TB::m[i][2];
            F w = wbuf[gi & 1][(i - gi * G) / V][(i - gi * G) % V];
            if constexpr (MODE == 2) w *= madj;
            if constexpr (ib == 16) {            // degree 1
                if constexpr (MODE != 1) g[jc] += w;
                if constexpr (MODE != 2) f += w * x[jc];
            } else if constexpr (ia == 16) {     // degree 2
                const F t = w * x[ib];
                if constexpr (MODE != 1) {
                    g[jc] += t;
                    g[ib] += w * x[jc];
                }
                if constexpr (MODE != 2) f += t * x[jc];
            } else {
                const F wa = w * x[ia], pbc = x[ib] * x[jc];
                if constexpr (MODE != 1) {
                    g[ia] += w * pbc;
                    g[ib] += wa * x[jc];
                    g[jc] += wa * x[ib];
                }
                if constexpr (MODE != 2) f += wa * pbc;
            }
        });
        // The sums are final here and the variables are new values for the next group: without this the arithmetic
        // of all groups sinks below the last request (the coefficients of the whole polynomial live at once) and the
        // pairwise products of the variables are hoisted above the first group (over a hundred more live values).
        if constexpr (MODE != 2) pin_reg(f);
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            if constexpr (MODE != 1) pin_reg(g[q]);
            pin_reg(x[q]);   // (x is not const for this: its values never change)
        }
        __builtin_amdgcn_sched_barrier(0);
    });
}

template <typename F, int COUNT, int MODE>
__global__ __launch_bounds__(SPEC_BT, sizeof(F) == 8 ? 4 : 5) void k_poly_spec(const PolyParams<F> a, const PolySpecShape sh, int chunk)
{
    extern __shared__ __align__(16) unsigned char spec_lds[];
    const int tid = threadIdx.x;
    const int kb = blockIdx.x % sh.kblocks;
    int type = -1, u = blockIdx.x / sh.kblocks, seg0 = 0, seg_n = 0;
    for (int t = 0; t < a.T; ++t) {
        const int n_t = a.tstart[t + 1] - a.tstart[t];
        const int units = (n_t + chunk - 1) / chunk;
        if (u < units) { type = t; seg0 = a.tstart[t]; seg_n = n_t; break; }
        u -= units;
    }
    if (type < 0) return;
    {   // the slab of (species, channel block): contiguous, a multiple of 16 bytes
        const uint4* src = reinterpret_cast<const uint4*>(reinterpret_cast<const unsigned char*>(a.table_slabs) +
                                                          ((size_t)type * sh.kblocks + kb) * sh.slab_bytes);
        uint4* dst = reinterpret_cast<uint4*>(spec_lds);
        const int n16 = (int)(sh.slab_bytes / 16);
        for (int i = tid; i < n16; i += SPEC_BT) dst[i] = src[i];
    }
    __syncthreads();
    const int ag = tid / sh.CB, kloc = tid - ag * sh.CB;
    const int k = kb * sh.CB + kloc;
    const bool klive = ag < sh.AG && k < a.K;
    const unsigned kk = k < a.K ? k : a.K - 1;
    const unsigned char* slab_k = spec_lds + (size_t)kloc * 16;
    const int row_stride = sh.CB * 16;
    const int j0 = u * chunk, j1 = j0 + chunk < seg_n ? j0 + chunk : seg_n;
    for (int jb = j0; jb < j1; jb += sh.AG) {
        const int j = jb + ag;
        const bool live = klive && j < j1;
        const int node = a.perm[seg0 + (j < seg_n ? j : seg_n - 1)];
        F x[16], g[16], madj = F(1);
#pragma unroll
        for (int q = 0; q < 16; ++q) x[q] = a.A[((size_t)node * 16 + q) * a.K + kk];
        if constexpr (MODE == 2) {
            madj = a.M_adj[(size_t)node * COUNT * a.K + kk];
#pragma unroll
            for (int q = 0; q < 16; ++q) g[q] = F(0);
        }
        // one polynomial after the other: the variables are read once
        static_for<0, COUNT>([&](auto pc) {
            constexpr int P = decltype(pc)::value;
            F f = F(0), madj_next = F(1);
            if constexpr (MODE == 2 && P + 1 < COUNT) madj_next = a.M_adj[((size_t)node * COUNT + P + 1) * a.K + kk];
            if constexpr (MODE == 0) {
#pragma unroll
                for (int q = 0; q < 16; ++q) g[q] = F(0);
            }
            poly_spec_body<F, P, MODE>(slab_k, row_stride, x, g, f, madj);
            madj = madj_next;
            if (live) {
                if constexpr (MODE == 0) {
#pragma unroll
                    for (int q = 0; q < 16; ++q) a.M_grad[(((size_t)node * COUNT + P) * 16 + q) * a.K + k] = g[q];
                }
                if constexpr (MODE != 2) a.M[((size_t)node * COUNT + P) * a.K + k] = f;
            }
        });
        if constexpr (MODE == 2) {
            if (live) {
#pragma unroll
                for (int q = 0; q < 16; ++q) a.A_adj[((size_t)node * 16 + q) * a.K + k] = g[q];
            }
        }
    }
}
}  // namespace

template <typename F>
hipError_t launch_poly_spec(const PolyParams<F>& p, hipStream_t s)
{
    if (p.num_nodes <= 0) return hipSuccess;
    // standard product basis: straight-line kernel, variables in registers, coefficients in LDS
    const PolySpecShape sh = poly_spec_shape((int)sizeof(F), p.K, p.NP);
    if (sh.CB <= 0 || !(p.NP == 1 || p.NP == 4 || p.NP == 9)) return hipErrorInvalidValue;   // the loader's checks
    // Runs of `chunk` atoms (whole passes of AG atoms): about as many units as the CUs hold blocks at once.  Every
    // species present adds at most one unit; a few slots are kept for them (a model may know many more species
    // than a system holds, so not one per species).
    const int slots = std::max(p.num_cus > 0 ? p.num_cus : 256, 1) * sh.blocks_per_cu;
    const int units_k = std::max(slots / sh.kblocks - std::min(p.T, 8), 1);
    int chunk = (p.num_nodes + units_k - 1) / units_k;
    chunk = (chunk + sh.AG - 1) / sh.AG * sh.AG;
    const unsigned units = (unsigned)((p.num_nodes + chunk - 1) / chunk + p.T);
    const dim3 grid(units * sh.kblocks), block(SPEC_BT);
    auto go = [&](auto cc, auto mc) -> hipError_t {
        constexpr int COUNT = decltype(cc)::value, MODE = decltype(mc)::value;
        static bool attr_done = false;   // per instantiation
        if (!attr_done) {
            hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(k_poly_spec<F, COUNT, MODE>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (err != hipSuccess) return err;
            attr_done = true;
        }
        hipLaunchKernelGGL((k_poly_spec<F, COUNT, MODE>), grid, block, sh.slab_bytes, s, p, sh, chunk);
        return hipGetLastError();
    };
    auto with_count = [&](auto mc) -> hipError_t {
        if (p.NP == 1) return go(std::integral_constant<int, 1>{}, mc);
        if (p.NP == 4) return go(std::integral_constant<int, 4>{}, mc);
        return go(std::integral_constant<int, 9>{}, mc);
    };
    if (p.mode == 1) return with_count(std::integral_constant<int, 1>{});
    if (p.mode == 2) return with_count(std::integral_constant<int, 2>{});
    return with_count(std::integral_constant<int, 0>{});
}

#if SMX_POLY_PART == 0
template hipError_t launch_poly_spec<double>(const PolyParams<double>&, hipStream_t);
#else
template hipError_t launch_poly_spec<float>(const PolyParams<float>&, hipStream_t);
#endif

}  // namespace smx
