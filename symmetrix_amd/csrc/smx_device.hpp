// Device helpers shared by the edge kernels: real harmonics up to l = 3, DPP
// lane moves, wave-level sums, compile-time loops.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

namespace smx {

// compile-time loop: f(std::integral_constant<int, I>) for I in [I0, N)
template <int I0, int N, typename Fn>
__device__ __forceinline__ void static_for(Fn&& f)
{
    if constexpr (I0 < N) {
        f(std::integral_constant<int, I0>{});
        static_for<I0 + 1, N>(f);
    }
}

constexpr int lm_l(int lm) { return lm < 1 ? 0 : (lm < 4 ? 1 : (lm < 9 ? 2 : 3)); }

// Real harmonics l<=3 in the engine convention (mace.cpp:118-148): orthonormal
// real harmonics of the direction, evaluated at the permuted vector
// (x',y',z') = (z,x,y) and multiplied by 2 sqrt(pi).  Arguments are the
// permuted unit vector.  ylm_g<LM> gives harmonic LM and the derivative of its
// homogeneous form along the permuted axes.
template <int LM>
__device__ __forceinline__ void ylm_g(double x, double y, double z, double& Y, double& g0, double& g1, double& g2)
{
    constexpr double s3 = 1.7320508075688772, s15 = 3.872983346207417, s5h = 1.118033988749895;
    constexpr double s15h = 1.9364916731037085, c3a = 2.091650066335189, s105 = 10.246950765959598;
    constexpr double c3c = 1.620185174601965, c3d = 1.3228756555322954, c3e = 5.123475382979799;
    const double xx = x * x, yy = y * y, zz = z * z;
    if constexpr (LM == 0) { Y = 1.0; g0 = 0; g1 = 0; g2 = 0; }
    if constexpr (LM == 1) { Y = s3 * y; g0 = 0; g1 = s3; g2 = 0; }
    if constexpr (LM == 2) { Y = s3 * z; g0 = 0; g1 = 0; g2 = s3; }
    if constexpr (LM == 3) { Y = s3 * x; g0 = s3; g1 = 0; g2 = 0; }
    if constexpr (LM == 4) { Y = s15 * x * y; g0 = s15 * y; g1 = s15 * x; g2 = 0; }
    if constexpr (LM == 5) { Y = s15 * y * z; g0 = 0; g1 = s15 * z; g2 = s15 * y; }
    if constexpr (LM == 6) { Y = s5h * (2 * zz - xx - yy); g0 = -2 * s5h * x; g1 = -2 * s5h * y; g2 = 4 * s5h * z; }
    if constexpr (LM == 7) { Y = s15 * x * z; g0 = s15 * z; g1 = 0; g2 = s15 * x; }
    if constexpr (LM == 8) { Y = s15h * (xx - yy); g0 = 2 * s15h * x; g1 = -2 * s15h * y; g2 = 0; }
    if constexpr (LM == 9) { Y = c3a * y * (3 * xx - yy); g0 = 6 * c3a * x * y; g1 = 3 * c3a * (xx - yy); g2 = 0; }
    if constexpr (LM == 10) { Y = s105 * x * y * z; g0 = s105 * y * z; g1 = s105 * x * z; g2 = s105 * x * y; }
    if constexpr (LM == 11) { Y = c3c * y * (4 * zz - xx - yy); g0 = -2 * c3c * x * y; g1 = c3c * (4 * zz - xx - 3 * yy); g2 = 8 * c3c * y * z; }
    if constexpr (LM == 12) { Y = c3d * z * (2 * zz - 3 * xx - 3 * yy); g0 = -6 * c3d * x * z; g1 = -6 * c3d * y * z; g2 = 3 * c3d * (2 * zz - xx - yy); }
    if constexpr (LM == 13) { Y = c3c * x * (4 * zz - xx - yy); g0 = c3c * (4 * zz - 3 * xx - yy); g1 = -2 * c3c * x * y; g2 = 8 * c3c * x * z; }
    if constexpr (LM == 14) { Y = c3e * (xx - yy) * z; g0 = 2 * c3e * x * z; g1 = -2 * c3e * y * z; g2 = c3e * (xx - yy); }
    if constexpr (LM == 15) { Y = c3a * x * (xx - 3 * yy); g0 = 3 * c3a * (xx - yy); g1 = -6 * c3a * x * y; g2 = 0; }
}

// Y[16]
__device__ __forceinline__ void sph_l3(double x, double y, double z, double* Y)
{
    static_for<0, 16>([&](auto lc) {
        constexpr int lm = decltype(lc)::value;
        double g0, g1, g2;
        ylm_g<lm>(x, y, z, Y[lm], g0, g1, g2);
    });
}

// harmonics Y[16] and the derivative of their homogeneous forms along the permuted axes, g[3][16]
__device__ __forceinline__ void sph_l3_g(double x, double y, double z, double* Y, double (*g)[16])
{
    static_for<0, 16>([&](auto lc) {
        constexpr int lm = decltype(lc)::value;
        ylm_g<lm>(x, y, z, Y[lm], g[0][lm], g[1][lm], g[2][lm]);
    });
}

// Harmonics and their gradient with respect to the (unpermuted) edge vector,
// written as they are formed: out[lm] = Y, out[stride*(1+a) + lm] = dY/d(axis a)
// with a = 0,1,2 the original x, y, z axes.  (x,y,z) is the permuted unit
// vector, inv_r = 1/|v|.  Chain rule through u = v/|v|: u.grad_u of a degree-l
// form is l times the form; original x is permuted axis 1, y axis 2, z axis 0.
template <int STRIDE>
__device__ __forceinline__ void sph_l3_grad_store(double x, double y, double z, double inv_r, double* out)
{
    static_for<0, 16>([&](auto lc) {
        constexpr int lm = decltype(lc)::value;
        double Y, g0, g1, g2;
        ylm_g<lm>(x, y, z, Y, g0, g1, g2);
        const double ly = lm_l(lm) * Y;
        out[lm] = Y;
        out[STRIDE + lm] = (g1 - y * ly) * inv_r;
        out[2 * STRIDE + lm] = (g2 - z * ly) * inv_r;
        out[3 * STRIDE + lm] = (g0 - x * ly) * inv_r;
        // keep the live range of each harmonic short: the callers hold many accumulators
        if constexpr (lm % 4 == 3) __builtin_amdgcn_sched_barrier(0);
    });
}
__device__ __forceinline__ void sph_l3_grad(double x, double y, double z, double inv_r, double* Y, double (*G)[16])
{
    double g[3][16];
    sph_l3_g(x, y, z, Y, g);
    const double u[3] = {x, y, z};
#pragma unroll
    for (int lm = 0; lm < 16; ++lm) {
        const double ly = lm_l(lm) * Y[lm];
        G[0][lm] = (g[1][lm] - u[1] * ly) * inv_r;
        G[1][lm] = (g[2][lm] - u[2] * ly) * inv_r;
        G[2][lm] = (g[0][lm] - u[0] * ly) * inv_r;
    }
}

// 1/sqrt(a) and 1/a for positive normal a: hardware estimate (about 23 bits) and two Newton steps, good to
// the last bit or two.  The library forms (sqrt then divide, IEEE divide) cost four to five times as many
// instructions, and the edge kernels evaluate them per (edge, channel slice).
__device__ __forceinline__ double rsqrt_pos(double a)
{
    double y = __builtin_amdgcn_rsq(a);
    const double h = 0.5 * a;
    y = fma(y, fma(-h * y, y, 0.5), y);
    y = fma(y, fma(-h * y, y, 0.5), y);
    return y;
}
__device__ __forceinline__ double rcp_pos(double a)
{
    double y = __builtin_amdgcn_rcp(a);
    y = fma(y, fma(-a, y, 1.0), y);
    y = fma(y, fma(-a, y, 1.0), y);
    return y;
}
// spline interval of r: floor(r / h) computed with the reciprocal spacing, clamped to the table
__device__ __forceinline__ int spline_interval(double r, double inv_h, int last)
{
    return min(max((int)(r * inv_h), 0), last);
}

__device__ __forceinline__ int pair_index(int T, int a, int b)
{
    return (a <= b) ? a * (2 * T - a - 1) / 2 + b : b * (2 * T - b - 1) / 2 + a;
}

// DPP lane moves inside a 16-lane row (VALU moves, no LDS traffic).  Every lane of a row has a
// source lane, so no previous value of the destination is needed (mov_dpp leaves it undefined, which
// spares the register copy that update_dpp would make).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v)
{
    const int b = __float_as_int(v);
    return __int_as_float(__builtin_amdgcn_mov_dpp(b, CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ double dpp_move(double v)
{
    const long long b = __double_as_longlong(v);
    const int l = (int)(b & 0xffffffffll), h = (int)(b >> 32);
    const int lo = __builtin_amdgcn_mov_dpp(l, CTRL, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_mov_dpp(h, CTRL, 0xf, 0xf, false);
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
// value of the lane ROT places further round its 16-lane row (row_ror)
template <int ROT, typename T>
__device__ __forceinline__ T row_rotate(T v) { return dpp_move<0x120 + ROT>(v); }
// value of the neighbouring lane (lane ^ 1): quad_perm [1,0,3,2]
template <typename T>
__device__ __forceinline__ T lane_xor1(T v) { return dpp_move<0xB1>(v); }
// value of lane ^ 2: quad_perm [2,3,0,1]
template <typename T>
__device__ __forceinline__ T lane_xor2(T v) { return dpp_move<0x4E>(v); }
// value of the lane mirrored inside its group of eight (lane i <-> 7 - i): row_half_mirror
template <typename T>
__device__ __forceinline__ T half_mirror(T v) { return dpp_move<0x141>(v); }
// sum over the lanes of a 16-lane row whose index agrees modulo CL (CL = 1, 2, 4 or 8)
template <int CL, typename T>
__device__ __forceinline__ T row_sum_strided(T v)
{
    if constexpr (CL <= 8) v += row_rotate<8>(v);
    if constexpr (CL <= 4) v += row_rotate<4>(v);
    if constexpr (CL <= 2) v += row_rotate<2>(v);
    if constexpr (CL <= 1) v += row_rotate<1>(v);
    return v;
}

__device__ __forceinline__ double read_lane(double v, int lane)
{
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_readlane((int)(b & 0xffffffffll), lane);
    const int hi = __builtin_amdgcn_readlane((int)(b >> 32), lane);
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
__device__ __forceinline__ float read_lane(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ float wave_sum(float v)
{
    v = row_sum_strided<1>(v);
    return (read_lane(v, 0) + read_lane(v, 16)) + (read_lane(v, 32) + read_lane(v, 48));
}
// sum over the 64 lanes of the wavefront, the same value (and the same order of additions) in every lane
__device__ __forceinline__ double wave_sum(double v)
{
    v = row_sum_strided<1>(v);
    return (read_lane(v, 0) + read_lane(v, 16)) + (read_lane(v, 32) + read_lane(v, 48));
}

// Orders the LDS traffic of one wavefront: what its lanes wrote before is
// visible to all its lanes after.  No other wavefront is involved.
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// CPL consecutive elements moved with one load or store
template <typename F, int N>
struct alignas(sizeof(F) * N) Vec {
    F v[N];
};

}  // namespace smx
