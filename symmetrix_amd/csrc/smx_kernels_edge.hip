// Edge kernels for gfx950: fused harmonics + radial splines + receiver-segmented
// aggregation, and the analytic edge-force adjoint.
//
// Work decomposition.  The edge list is receiver-sorted (CSR).  A "team" of LPR
// lanes (half a wavefront or a whole one) owns one receiver; lane j of the team
// owns channels j, j+LPR, ... (CPL of them), so every table or feature load of a
// team is one contiguous run of LPR elements.  Accumulators (NE per channel)
// live in registers for the whole neighbour loop, so sums run in edge order with
// no atomics and are bit-reproducible.  Per chunk of EC edges the first EC lanes
// of the team evaluate the per-edge quantities that do not depend on the channel
// (direction, harmonics, Clebsch-Gordan-contracted harmonics B, spline interval)
// into LDS, from where the channel loop reads them as broadcasts.
#include "smx_kernels.hpp"
#include "smx_paths.hpp"

#include <type_traits>

namespace smx {

namespace {

// compile-time loop: f(std::integral_constant<int, I>) for I in [I0, N)
template <int I0, int N, typename Fn>
__device__ __forceinline__ void static_for(Fn&& f)
{
    if constexpr (I0 < N) {
        f(std::integral_constant<int, I0>{});
        static_for<I0 + 1, N>(f);
    }
}

// Real harmonics l<=3 in the engine convention (mace.cpp:118-148): orthonormal
// real harmonics of the direction, evaluated at the permuted vector
// (x',y',z') = (z,x,y) and multiplied by 2 sqrt(pi).  Arguments are the
// permuted unit vector.  Y[16].
__device__ __forceinline__ void sph_l3(double x, double y, double z, double* Y)
{
    const double s3 = 1.7320508075688772, s15 = 3.872983346207417, s5h = 1.118033988749895;
    const double s15h = 1.9364916731037085, c3a = 2.091650066335189, s105 = 10.246950765959598;
    const double c3c = 1.620185174601965, c3d = 1.3228756555322954, c3e = 5.123475382979799;
    const double xx = x * x, yy = y * y, zz = z * z;
    Y[0] = 1.0;
    Y[1] = s3 * y; Y[2] = s3 * z; Y[3] = s3 * x;
    Y[4] = s15 * x * y; Y[5] = s15 * y * z; Y[6] = s5h * (2 * zz - xx - yy);
    Y[7] = s15 * x * z; Y[8] = s15h * (xx - yy);
    Y[9] = c3a * y * (3 * xx - yy); Y[10] = s105 * x * y * z;
    Y[11] = c3c * y * (4 * zz - xx - yy); Y[12] = c3d * z * (2 * zz - 3 * xx - 3 * yy);
    Y[13] = c3c * x * (4 * zz - xx - yy); Y[14] = c3e * (xx - yy) * z; Y[15] = c3a * x * (xx - 3 * yy);
}

// Harmonics and their gradient with respect to the (unpermuted) edge vector.
// (x,y,z) is the permuted unit vector, inv_r = 1/|v|.  G[a][lm] with a = 0,1,2
// the derivative along the original x, y, z axes.
__device__ __forceinline__ void sph_l3_grad(double x, double y, double z, double inv_r, double* Y, double (*G)[16])
{
    const double s3 = 1.7320508075688772, s15 = 3.872983346207417, s5h = 1.118033988749895;
    const double s15h = 1.9364916731037085, c3a = 2.091650066335189, s105 = 10.246950765959598;
    const double c3c = 1.620185174601965, c3d = 1.3228756555322954, c3e = 5.123475382979799;
    const double xx = x * x, yy = y * y, zz = z * z;
    double g[3][16];  // derivative of the homogeneous forms along x', y', z'
    Y[0] = 1.0;                              g[0][0] = 0;               g[1][0] = 0;                g[2][0] = 0;
    Y[1] = s3 * y;                           g[0][1] = 0;               g[1][1] = s3;               g[2][1] = 0;
    Y[2] = s3 * z;                           g[0][2] = 0;               g[1][2] = 0;                g[2][2] = s3;
    Y[3] = s3 * x;                           g[0][3] = s3;              g[1][3] = 0;                g[2][3] = 0;
    Y[4] = s15 * x * y;                      g[0][4] = s15 * y;         g[1][4] = s15 * x;          g[2][4] = 0;
    Y[5] = s15 * y * z;                      g[0][5] = 0;               g[1][5] = s15 * z;          g[2][5] = s15 * y;
    Y[6] = s5h * (2 * zz - xx - yy);         g[0][6] = -2 * s5h * x;    g[1][6] = -2 * s5h * y;     g[2][6] = 4 * s5h * z;
    Y[7] = s15 * x * z;                      g[0][7] = s15 * z;         g[1][7] = 0;                g[2][7] = s15 * x;
    Y[8] = s15h * (xx - yy);                 g[0][8] = 2 * s15h * x;    g[1][8] = -2 * s15h * y;    g[2][8] = 0;
    Y[9] = c3a * y * (3 * xx - yy);          g[0][9] = 6 * c3a * x * y; g[1][9] = 3 * c3a * (xx - yy); g[2][9] = 0;
    Y[10] = s105 * x * y * z;                g[0][10] = s105 * y * z;   g[1][10] = s105 * x * z;    g[2][10] = s105 * x * y;
    Y[11] = c3c * y * (4 * zz - xx - yy);    g[0][11] = -2 * c3c * x * y; g[1][11] = c3c * (4 * zz - xx - 3 * yy); g[2][11] = 8 * c3c * y * z;
    Y[12] = c3d * z * (2 * zz - 3 * xx - 3 * yy); g[0][12] = -6 * c3d * x * z; g[1][12] = -6 * c3d * y * z; g[2][12] = 3 * c3d * (2 * zz - xx - yy);
    Y[13] = c3c * x * (4 * zz - xx - yy);    g[0][13] = c3c * (4 * zz - 3 * xx - yy); g[1][13] = -2 * c3c * x * y; g[2][13] = 8 * c3c * x * z;
    Y[14] = c3e * (xx - yy) * z;             g[0][14] = 2 * c3e * x * z; g[1][14] = -2 * c3e * y * z; g[2][14] = c3e * (xx - yy);
    Y[15] = c3a * x * (xx - 3 * yy);         g[0][15] = 3 * c3a * (xx - yy); g[1][15] = -6 * c3a * x * y; g[2][15] = 0;
    // chain rule through u = v/|v| (u.grad_u of a degree-l form is l times the form), then
    // undo the permutation: original x is x' index 1, y is index 2, z is index 0
    const double u[3] = {x, y, z};
#pragma unroll
    for (int lm = 0; lm < 16; ++lm) {
        const int l = lm < 1 ? 0 : (lm < 4 ? 1 : (lm < 9 ? 2 : 3));
        const double ly = l * Y[lm];
        G[0][lm] = (g[1][lm] - u[1] * ly) * inv_r;
        G[1][lm] = (g[2][lm] - u[2] * ly) * inv_r;
        G[2][lm] = (g[0][lm] - u[0] * ly) * inv_r;
    }
}

__device__ __forceinline__ int pair_index(int T, int a, int b)
{
    return (a <= b) ? a * (2 * T - a - 1) / 2 + b : b * (2 * T - b - 1) / 2 + a;
}

// sum over the LPR lanes of a team; every lane of the team gets the result
template <int LPR>
__device__ __forceinline__ double team_sum(double v)
{
#pragma unroll
    for (int off = LPR / 2; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <typename F, int NB, bool BWD>
struct TeamLds {
    static constexpr int NY = BWD ? 64 : 16;
    static constexpr int NBT = BWD ? 4 * NB : NB;
    __host__ __device__ static constexpr size_t bytes(int EC)
    {
        return (size_t)EC * (NY * sizeof(double) + NBT * sizeof(F) + sizeof(F) + (BWD ? 3 * sizeof(double) : 0) + 2 * sizeof(int)) + 16;
    }
};

// ---------------------------------------------------------------------------
template <typename F, int LMAXH, int LPR, int CPL, int EC>
__global__ __launch_bounds__(256) void k_agg_fwd(const AggParams<F> a)
{
    using PT = Paths<LMAXH>;
    constexpr int RPB = 256 / LPR, NB = PT::NB, NE = PT::NE, P = PT::P, NLM = PT::NLM;
    extern __shared__ __align__(16) unsigned char smem[];
    const int team = threadIdx.x / LPR, lane = threadIdx.x % LPR;
    unsigned char* base = smem + (size_t)team * ((TeamLds<F, NB, false>::bytes(EC) + 15) / 16 * 16);
    double* Yt = reinterpret_cast<double*>(base);                 // [EC][16]
    F* Bs = reinterpret_cast<F*>(Yt + EC * 16);                   // [EC][NB]
    F* xs = Bs + EC * NB;                                         // [EC]
    int* rows = reinterpret_cast<int*>(xs + EC + (EC & 1));       // [EC]
    int* grows = rows + EC;                                       // [EC]

    const int K = a.K, NSPL = P * K;
    const int i = blockIdx.x * RPB + team;
    const int kbase = blockIdx.y * (LPR * CPL);
    int e0 = 0, e1 = 0, ti = 0;
    if (i < a.num_nodes) { e0 = a.first_neigh[i]; e1 = a.first_neigh[i + 1]; ti = a.node_types[i]; }
    int maxdeg = 0;
#pragma unroll
    for (int t = 0; t < RPB; ++t) {
        const int ii = blockIdx.x * RPB + t;
        if (ii < a.num_nodes) maxdeg = max(maxdeg, a.first_neigh[ii + 1] - a.first_neigh[ii]);
    }
    const int nchunks = (maxdeg + EC - 1) / EC;

    F acc[CPL][NE];
#pragma unroll
    for (int c = 0; c < CPL; ++c)
#pragma unroll
        for (int q = 0; q < NE; ++q) acc[c][q] = F(0);

    for (int ch = 0; ch < nchunks; ++ch) {
        __syncthreads();
        const int eb = e0 + ch * EC;
        if (lane < EC && eb + lane < e1) {
            const int e = eb + lane;
            const double dx = a.xyz[3 * (size_t)e], dy = a.xyz[3 * (size_t)e + 1], dz = a.xyz[3 * (size_t)e + 2];
            const double inv = 1.0 / sqrt(dx * dx + dy * dy + dz * dz);
            double Y[16];
            sph_l3(dz * inv, dx * inv, dy * inv, Y);
#pragma unroll
            for (int q = 0; q < 16; ++q) Yt[lane * 16 + q] = Y[q];
            for (int b = 0; b < NB; ++b) {
                double s = 0.0;
                for (int t = a.B_start[b]; t < a.B_start[b + 1]; ++t) s += a.B_c[t] * Yt[lane * 16 + a.B_lm1[t]];
                Bs[lane * NB + b] = (F)s;
            }
            const double r = a.r[e];
            int n = (int)(r / a.spl_h);
            n = min(max(n, 0), a.spl_nodes - 2);
            xs[lane] = (F)(r - a.spl_h * n);
            const int tbl = a.pair_table[pair_index(a.T, ti, a.neigh_types[e])];
            rows[lane] = tbl * (a.spl_nodes - 1) + n;
            grows[lane] = a.gather[e];
        }
        __syncthreads();
        const int nE = min(EC, e1 - eb);
        for (int le = 0; le < nE; ++le) {
            const F x = xs[le];
            const F* row = a.tab + (size_t)rows[le] * 4 * NSPL;
            const F* Hrow = a.Hsrc + (size_t)grows[le] * NLM * K;
            const F* B = Bs + le * NB;
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                const int k = kbase + lane + c * LPR;
                if (k < K) {
                    F H[NLM];
#pragma unroll
                    for (int q = 0; q < NLM; ++q) H[q] = Hrow[q * K + k];
                    static_for<0, P>([&](auto pc) {
                        constexpr int p = decltype(pc)::value;
                        constexpr int l = PT::l(p), l2 = PT::l2(p), bo = PT::boff(p);
                        constexpr int lme0 = PT::lme(p, 0), es = PT::num_e(l);
                        const F c0 = row[p * K + k], c1 = row[NSPL + p * K + k];
                        const F c2 = row[2 * NSPL + p * K + k], c3 = row[3 * NSPL + p * K + k];
                        const F R = c0 + x * (c1 + x * (c2 + x * c3));
#pragma unroll
                        for (int m = 0; m < 2 * l + 1; ++m) {
                            F z = F(0);
#pragma unroll
                            for (int m2 = 0; m2 < 2 * l2 + 1; ++m2)
                                z += B[bo + m * (2 * l2 + 1) + m2] * H[l2 * l2 + m2];
                            acc[c][lme0 + m * es] += R * z;
                        }
                    });
                }
            }
        }
    }
    if (i < a.num_nodes) {
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            const int k = kbase + lane + c * LPR;
            if (k < K) {
#pragma unroll
                for (int q = 0; q < NE; ++q) a.out[((size_t)i * NE + q) * K + k] = acc[c][q];
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Adjoint: per edge force -dE/dxyz_ij (MACE::reverse_A0, mace.cpp:238-269;
// MACE::reverse_Phi1, mace.cpp:531-574) and the adjoint message to the sender
// row (mace.cpp:579-604), staged per edge for the deterministic sender-side sum.
template <typename F, int LMAXH, int LPR, int CPL, int EC>
__global__ __launch_bounds__(256) void k_agg_bwd(const AggParams<F> a)
{
    using PT = Paths<LMAXH>;
    constexpr int RPB = 256 / LPR, NB = PT::NB, NE = PT::NE, P = PT::P, NLM = PT::NLM;
    extern __shared__ __align__(16) unsigned char smem[];
    const int team = threadIdx.x / LPR, lane = threadIdx.x % LPR;
    unsigned char* base = smem + (size_t)team * ((TeamLds<F, NB, true>::bytes(EC) + 15) / 16 * 16);
    double* Yt = reinterpret_cast<double*>(base);                 // [EC][4][16]: Y, dY/dx, dY/dy, dY/dz
    double* us = Yt + EC * 64;                                    // [EC][3] unit vector xyz/r
    F* Bs = reinterpret_cast<F*>(us + EC * 3);                    // [EC][4][NB]
    F* xs = Bs + EC * 4 * NB;                                     // [EC]
    int* rows = reinterpret_cast<int*>(xs + EC + (EC & 1));
    int* grows = rows + EC;

    const int K = a.K, NSPL = P * K;
    const int i = blockIdx.x * RPB + team;
    const int kbase = blockIdx.y * (LPR * CPL);
    int e0 = 0, e1 = 0, ti = 0;
    if (i < a.num_nodes) { e0 = a.first_neigh[i]; e1 = a.first_neigh[i + 1]; ti = a.node_types[i]; }
    int maxdeg = 0;
#pragma unroll
    for (int t = 0; t < RPB; ++t) {
        const int ii = blockIdx.x * RPB + t;
        if (ii < a.num_nodes) maxdeg = max(maxdeg, a.first_neigh[ii + 1] - a.first_neigh[ii]);
    }
    const int nchunks = (maxdeg + EC - 1) / EC;

    F d[CPL][NE];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        const int k = kbase + lane + c * LPR;
#pragma unroll
        for (int q = 0; q < NE; ++q)
            d[c][q] = (i < a.num_nodes && k < K) ? a.d_out[((size_t)i * NE + q) * K + k] : F(0);
    }

    for (int ch = 0; ch < nchunks; ++ch) {
        __syncthreads();
        const int eb = e0 + ch * EC;
        if (lane < EC && eb + lane < e1) {
            const int e = eb + lane;
            const double dx = a.xyz[3 * (size_t)e], dy = a.xyz[3 * (size_t)e + 1], dz = a.xyz[3 * (size_t)e + 2];
            const double inv = 1.0 / sqrt(dx * dx + dy * dy + dz * dz);
            double Y[16], G[3][16];
            sph_l3_grad(dz * inv, dx * inv, dy * inv, inv, Y, G);
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                Yt[lane * 64 + q] = Y[q];
                Yt[lane * 64 + 16 + q] = G[0][q];
                Yt[lane * 64 + 32 + q] = G[1][q];
                Yt[lane * 64 + 48 + q] = G[2][q];
            }
            for (int b = 0; b < NB; ++b) {
                double s = 0.0, sx = 0.0, sy = 0.0, sz = 0.0;
                for (int t = a.B_start[b]; t < a.B_start[b + 1]; ++t) {
                    const double cc = a.B_c[t];
                    const int lm1 = a.B_lm1[t];
                    s += cc * Yt[lane * 64 + lm1];
                    sx += cc * Yt[lane * 64 + 16 + lm1];
                    sy += cc * Yt[lane * 64 + 32 + lm1];
                    sz += cc * Yt[lane * 64 + 48 + lm1];
                }
                Bs[(lane * 4 + 0) * NB + b] = (F)s;
                Bs[(lane * 4 + 1) * NB + b] = (F)sx;
                Bs[(lane * 4 + 2) * NB + b] = (F)sy;
                Bs[(lane * 4 + 3) * NB + b] = (F)sz;
            }
            const double r = a.r[e];
            // radial direction as the reference forms it: xyz / r with the caller's r
            us[lane * 3] = dx / r; us[lane * 3 + 1] = dy / r; us[lane * 3 + 2] = dz / r;
            int n = (int)(r / a.spl_h);
            n = min(max(n, 0), a.spl_nodes - 2);
            xs[lane] = (F)(r - a.spl_h * n);
            const int tbl = a.pair_table[pair_index(a.T, ti, a.neigh_types[e])];
            rows[lane] = tbl * (a.spl_nodes - 1) + n;
            grows[lane] = a.gather[e];
        }
        __syncthreads();
        const int nE = min(EC, e1 - eb);
        for (int le = 0; le < nE; ++le) {
            const F x = xs[le];
            const F* row = a.tab + (size_t)rows[le] * 4 * NSPL;
            const F* Hrow = a.Hsrc + (size_t)grows[le] * NLM * K;
            const F* B = Bs + (le * 4) * NB;
            const F* Bx = B + NB;
            const F* By = B + 2 * NB;
            const F* Bz = B + 3 * NB;
            double srad = 0.0, gx = 0.0, gy = 0.0, gz = 0.0;
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                const int k = kbase + lane + c * LPR;
                if (k < K) {
                    F H[NLM], mg[NLM];
#pragma unroll
                    for (int q = 0; q < NLM; ++q) { H[q] = Hrow[q * K + k]; mg[q] = F(0); }
                    F s_c = F(0), gx_c = F(0), gy_c = F(0), gz_c = F(0);
                    static_for<0, P>([&](auto pc) {
                        constexpr int p = decltype(pc)::value;
                        constexpr int l = PT::l(p), l2 = PT::l2(p), bo = PT::boff(p);
                        constexpr int lme0 = PT::lme(p, 0), es = PT::num_e(l);
                        const F c0 = row[p * K + k], c1 = row[NSPL + p * K + k];
                        const F c2 = row[2 * NSPL + p * K + k], c3 = row[3 * NSPL + p * K + k];
                        const F R = c0 + x * (c1 + x * (c2 + x * c3));
                        const F Rd = c1 + x * (F(2) * c2 + F(3) * x * c3);
#pragma unroll
                        for (int m = 0; m < 2 * l + 1; ++m) {
                            const F dd = d[c][lme0 + m * es];
                            const F t = dd * R;
                            F z = F(0), zx = F(0), zy = F(0), zz = F(0);
#pragma unroll
                            for (int m2 = 0; m2 < 2 * l2 + 1; ++m2) {
                                const int b = bo + m * (2 * l2 + 1) + m2;
                                const F h = H[l2 * l2 + m2];
                                z += B[b] * h; zx += Bx[b] * h; zy += By[b] * h; zz += Bz[b] * h;
                                mg[l2 * l2 + m2] += t * B[b];
                            }
                            s_c += dd * Rd * z;
                            gx_c += t * zx; gy_c += t * zy; gz_c += t * zz;
                        }
                    });
                    srad += (double)s_c; gx += (double)gx_c; gy += (double)gy_c; gz += (double)gz_c;
                    if (a.msg) {
                        F* mrow = a.msg + (size_t)(eb + le) * NLM * K;
#pragma unroll
                        for (int q = 0; q < NLM; ++q) mrow[q * K + k] = mg[q];
                    }
                }
            }
            double fx = -(us[le * 3] * srad + gx);
            double fy = -(us[le * 3 + 1] * srad + gy);
            double fz = -(us[le * 3 + 2] * srad + gz);
            fx = team_sum<LPR>(fx); fy = team_sum<LPR>(fy); fz = team_sum<LPR>(fz);
            if (lane == 0 && gridDim.y == 1) {
                double* f = a.forces + 3 * (size_t)(eb + le);
                if (a.accumulate_forces) { f[0] += fx; f[1] += fy; f[2] += fz; }
                else { f[0] = fx; f[1] = fy; f[2] = fz; }
            }
        }
    }
}

template <typename F, int LMAXH, int LPR, int CPL, int EC, bool BWD>
hipError_t launch_agg_t(const AggParams<F>& p, hipStream_t s)
{
    using PT = Paths<LMAXH>;
    constexpr int RPB = 256 / LPR;
    const size_t per_team = (TeamLds<F, PT::NB, BWD>::bytes(EC) + 15) / 16 * 16;
    const size_t lds = per_team * RPB;
    dim3 grid((p.num_nodes + RPB - 1) / RPB, (p.K + LPR * CPL - 1) / (LPR * CPL));
    if (grid.x == 0) return hipSuccess;
    if (BWD && grid.y != 1) return hipErrorInvalidValue;
    void (*kern)(const AggParams<F>);
    if constexpr (BWD) kern = k_agg_bwd<F, LMAXH, LPR, CPL, EC>;
    else kern = k_agg_fwd<F, LMAXH, LPR, CPL, EC>;
    if (lds > 64 * 1024) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
    }
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, s, p);
    return hipGetLastError();
}

template <typename F, int LMAXH, bool BWD>
hipError_t launch_agg_sel(const AggParams<F>& p, hipStream_t s)
{
    const int K = p.K;
    if (LMAXH == 0) {
        constexpr int EC = BWD ? 8 : 16;
        if (K <= 32) return launch_agg_t<F, LMAXH, 32, 1, EC, BWD>(p, s);
        if (K <= 64) return launch_agg_t<F, LMAXH, 32, 2, EC, BWD>(p, s);
        if (K <= 96) return launch_agg_t<F, LMAXH, 32, 3, EC, BWD>(p, s);
        if (K <= 128) return launch_agg_t<F, LMAXH, 32, 4, EC, BWD>(p, s);
        if (K <= 256) return launch_agg_t<F, LMAXH, 64, 4, EC, BWD>(p, s);
        return hipErrorInvalidValue;
    } else {
        constexpr int EC = BWD ? 4 : 8;
        if (K <= 32) return launch_agg_t<F, LMAXH, 32, 1, EC, BWD>(p, s);
        if (K <= 64) return launch_agg_t<F, LMAXH, 32, 2, EC, BWD>(p, s);
        if (K <= 128) return launch_agg_t<F, LMAXH, 64, 2, EC, BWD>(p, s);
        return hipErrorInvalidValue;
    }
}

}  // namespace

template <typename F>
hipError_t launch_agg_fwd(int L_max_H, const AggParams<F>& p, hipStream_t s)
{
    if (L_max_H == 0) return launch_agg_sel<F, 0, false>(p, s);
    if (L_max_H == 1) return launch_agg_sel<F, 1, false>(p, s);
    return hipErrorInvalidValue;
}
template <typename F>
hipError_t launch_agg_bwd(int L_max_H, const AggParams<F>& p, hipStream_t s)
{
    if (L_max_H == 0) return launch_agg_sel<F, 0, true>(p, s);
    if (L_max_H == 1) return launch_agg_sel<F, 1, true>(p, s);
    return hipErrorInvalidValue;
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
#else
template hipError_t launch_agg_bwd<float>(int, const AggParams<float>&, hipStream_t);
#endif

#if SMX_EDGE_PART == 0

// ---------------------------------------------------------------------------
namespace {
template <typename F>
__global__ void k_sender_reduce(int rows, int width, const int* sstart, const int* slist, const F* msg,
                                F* H_adj, int zero_first)
{
    const int j = blockIdx.x;
    const int s0 = sstart[j], s1 = sstart[j + 1];
    for (int q = threadIdx.x; q < width; q += blockDim.x) {
        F acc = zero_first ? F(0) : H_adj[(size_t)j * width + q];
        for (int t = s0; t < s1; ++t) acc += msg[(size_t)slist[t] * width + q];
        H_adj[(size_t)j * width + q] = acc;
    }
}
}  // namespace

template <typename F>
hipError_t launch_sender_reduce(int rows, int width, const int* sstart, const int* slist, const F* msg,
                                F* H_adj, int zero_first, hipStream_t s)
{
    if (rows <= 0) return hipSuccess;
    const int bs = width <= 64 ? 64 : (width <= 128 ? 128 : 256);
    hipLaunchKernelGGL(k_sender_reduce<F>, dim3(rows), dim3(bs), 0, s, rows, width, sstart, slist, msg, H_adj, zero_first);
    return hipGetLastError();
}
template hipError_t launch_sender_reduce<double>(int, int, const int*, const int*, const double*, double*, int, hipStream_t);
template hipError_t launch_sender_reduce<float>(int, int, const int*, const int*, const float*, float*, int, hipStream_t);

// ---------------------------------------------------------------------------
namespace {
__global__ void k_sph_harm(const double* xyz, long E, double* Y, double* Yg)
{
    const long e = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    const double dx = xyz[3 * e], dy = xyz[3 * e + 1], dz = xyz[3 * e + 2];
    const double inv = 1.0 / sqrt(dx * dx + dy * dy + dz * dz);
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
