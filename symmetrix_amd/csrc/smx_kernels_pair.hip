// Pair terms that depend on the edge length only: the ZBL repulsion
// (libsymmetrix/source/zbl.cpp:22-125) and the density normalisation of the
// A-basis (MACE::compute_A0_scaled / reverse_A0_scaled, mace.cpp:273-346, and
// their layer-1 twins, mace.cpp:681-757).  One wavefront per receiver: lanes
// take the receiver's edges in turn, per-receiver sums are formed with a fixed
// lane-to-edge assignment and a fixed reduction tree (bit-reproducible, no
// atomics); the per-edge force terms are added to the edge's own force entry.
#include "smx_device.hpp"
#include "smx_kernels.hpp"

namespace smx {

namespace {

// cubic_spline.cpp:29-41: value and derivative of one spline; intervals outside the table raise bit 4 of *flags
__device__ __forceinline__ void spline_eval(const PairSpline& sp, int pair, double r, double& f, double& d, int* flags)
{
    int i = (int)(r / sp.h);
    if (i < 0 || i >= sp.nodes - 1) {
        atomicOr(flags, 4);
        i = min(max(i, 0), sp.nodes - 2);
    }
    const double x = r - sp.h * i;
    const double* c = sp.c + ((size_t)pair * (sp.nodes - 1) + i) * 4;
    f = c[0] + c[1] * x + c[2] * x * x + c[3] * x * x * x;
    d = c[1] + 2 * c[2] * x + 3 * c[3] * x * x;
}

__device__ __forceinline__ double ipow(double x, int n)
{
    double p = 1.0;
    for (int q = 0; q < n; ++q) p *= x;
    return p;
}

// zbl.cpp:96-125 with the pair constants (screening length, envelope radius, Z_i Z_j) tabulated per species pair
__global__ __launch_bounds__(256) void k_zbl(int N, const int* first_neigh, const int* node_types, const int* neigh_types,
                                             const double* xyz, const double* r, ZblParams z, double* energies,
                                             double* forces)
{
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (i >= N) return;
    const int ti = node_types[i];
    double esum = 0.0;
    for (int e = first_neigh[i] + lane; e < first_neigh[i + 1]; e += 64) {
        const int pr = ti * z.T + neigh_types[e];
        const double a = z.a_pair[pr], r_max = z.rmax_pair[pr], zz = z.zz_pair[pr];
        const double rr = r[e], ra = rr / a;
        // zbl.cpp:22-71
        const double k0 = -3.2, k1 = -0.9423, k2 = -0.4028, k3 = -0.2016;
        const double e0 = z.c[0] * exp(k0 * ra), e1 = z.c[1] * exp(k1 * ra);
        const double e2 = z.c[2] * exp(k2 * ra), e3 = z.c[3] * exp(k3 * ra);
        const double phi = e0 + e1 + e2 + e3;
        const double dphi = (k0 * e0 + k1 * e1 + k2 * e2 + k3 * e3) / a;
        const double v = 14.3996 * zz / rr * phi;
        const double dv = 14.3996 * zz * (rr * dphi - phi) / (rr * rr);
        // zbl.cpp:73-94: polynomial envelope of order p and its derivative
        double env = 0.0, denv = 0.0;
        if (rr < r_max) {
            const double x = rr / r_max, p = z.p;
            const double xp1 = ipow(x, z.p - 1), xp = xp1 * x, xq = xp * x, xs = xq * x;
            env = 1.0 - ((p + 1.0) * (p + 2.0) / 2.0) * xp + p * (p + 2.0) * xq - (p * (p + 1.0) / 2.0) * xs;
            denv = (-((p + 1.0) * (p + 2.0) / 2.0) * p * xp1 + p * (p + 2.0) * (p + 1.0) * xp -
                    (p * (p + 1.0) / 2.0) * (p + 2.0) * xq) / r_max;
        }
        esum += v * (0.5 * env);
        const double g = 0.5 * (v * denv + dv * env) / rr;
        forces[3 * (size_t)e] -= xyz[3 * (size_t)e] * g;
        forces[3 * (size_t)e + 1] -= xyz[3 * (size_t)e + 1] * g;
        forces[3 * (size_t)e + 2] -= xyz[3 * (size_t)e + 2] * g;
    }
    esum = wave_sum(esum);
    if (lane == 0) energies[i] += esum;
}

// A[i, :] /= 1 + sum_j s_pair(r_ij); the divisor is kept for the adjoint
template <typename F>
__global__ __launch_bounds__(256) void k_scale_fwd(int N, const int* first_neigh, const int* node_types,
                                                   const int* neigh_types, const double* r, PairSpline sp, int T,
                                                   F* A, int width, double* divisor, int* flags)
{
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (i >= N) return;
    const int ti = node_types[i];
    double s = 0.0;
    for (int e = first_neigh[i] + lane; e < first_neigh[i + 1]; e += 64) {
        double f, d;
        spline_eval(sp, pair_index(T, ti, neigh_types[e]), r[e], f, d, flags);
        s += f;
    }
    s = 1.0 + wave_sum(s);
    if (lane == 0) divisor[i] = s;
    F* Ai = A + (size_t)i * width;
    for (int q = lane; q < width; q += 64) Ai[q] = (F)((double)Ai[q] / s);
}

// mace.cpp:299-346: dot = A_adj . A (A already divided); force_ij += dot / s * s'(r_ij) * xyz_ij / r_ij; A_adj /= s
template <typename F>
__global__ __launch_bounds__(256) void k_scale_bwd(int N, const int* first_neigh, const int* node_types,
                                                   const int* neigh_types, const double* xyz, const double* r,
                                                   PairSpline sp, int T, const F* A, F* A_adj, int width,
                                                   const double* divisor, double* forces, int* flags)
{
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (i >= N) return;
    const int ti = node_types[i];
    const double s = divisor[i];
    const F* Ai = A + (size_t)i * width;
    F* Aa = A_adj + (size_t)i * width;
    double dot = 0.0;
    for (int q = lane; q < width; q += 64) dot += (double)Aa[q] * (double)Ai[q];
    dot = wave_sum(dot);
    for (int e = first_neigh[i] + lane; e < first_neigh[i + 1]; e += 64) {
        double f, d;
        spline_eval(sp, pair_index(T, ti, neigh_types[e]), r[e], f, d, flags);
        const double g = dot / s * d / r[e];
        forces[3 * (size_t)e] += g * xyz[3 * (size_t)e];
        forces[3 * (size_t)e + 1] += g * xyz[3 * (size_t)e + 1];
        forces[3 * (size_t)e + 2] += g * xyz[3 * (size_t)e + 2];
    }
    for (int q = lane; q < width; q += 64) Aa[q] = (F)((double)Aa[q] / s);
}

}  // namespace

hipError_t launch_zbl(int N, const int* first_neigh, const int* node_types, const int* neigh_types, const double* xyz,
                      const double* r, const ZblParams& z, double* energies, double* forces, hipStream_t s)
{
    if (N > 0)
        hipLaunchKernelGGL(k_zbl, dim3((N + 3) / 4), dim3(256), 0, s, N, first_neigh, node_types, neigh_types, xyz, r, z,
                           energies, forces);
    return hipGetLastError();
}

template <typename F>
hipError_t launch_scale_fwd(int N, const int* first_neigh, const int* node_types, const int* neigh_types, const double* r,
                            const PairSpline& sp, int T, F* A, int width, double* divisor, int* flags, hipStream_t s)
{
    if (N > 0)
        hipLaunchKernelGGL(k_scale_fwd<F>, dim3((N + 3) / 4), dim3(256), 0, s, N, first_neigh, node_types, neigh_types, r,
                           sp, T, A, width, divisor, flags);
    return hipGetLastError();
}
template <typename F>
hipError_t launch_scale_bwd(int N, const int* first_neigh, const int* node_types, const int* neigh_types,
                            const double* xyz, const double* r, const PairSpline& sp, int T, const F* A, F* A_adj,
                            int width, const double* divisor, double* forces, int* flags, hipStream_t s)
{
    if (N > 0)
        hipLaunchKernelGGL(k_scale_bwd<F>, dim3((N + 3) / 4), dim3(256), 0, s, N, first_neigh, node_types, neigh_types,
                           xyz, r, sp, T, A, A_adj, width, divisor, forces, flags);
    return hipGetLastError();
}
template hipError_t launch_scale_fwd<double>(int, const int*, const int*, const int*, const double*, const PairSpline&, int, double*, int, double*, int*, hipStream_t);
template hipError_t launch_scale_fwd<float>(int, const int*, const int*, const int*, const double*, const PairSpline&, int, float*, int, double*, int*, hipStream_t);
template hipError_t launch_scale_bwd<double>(int, const int*, const int*, const int*, const double*, const double*, const PairSpline&, int, const double*, double*, int, const double*, double*, int*, hipStream_t);
template hipError_t launch_scale_bwd<float>(int, const int*, const int*, const int*, const double*, const double*, const PairSpline&, int, const float*, float*, int, const double*, double*, int*, hipStream_t);

}  // namespace smx
