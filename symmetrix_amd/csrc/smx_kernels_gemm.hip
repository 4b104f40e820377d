// Channel-mixing linears on the gfx950 matrix cores.
//
// Block tile: 64 rows x GN columns (GN = 16*NT, chosen per launch from the
// output width so that K = 96 or 128 channels fill whole tiles), four
// wavefronts, wavefront w owns rows 16w..16w+15 and all NT 16-column tiles.
// The inner dimension is consumed in slabs of 32 staged through LDS in k-major
// order (a 16-lane group then reads 16 consecutive elements: no bank
// conflicts); the global loads of slab s+1 are issued into registers before the
// MFMAs of slab s, so their latency hides behind the matrix work.
// v_mfma_f64_16x16x4_f64 / v_mfma_f32_16x16x4_f32 operand layout: lane L
// supplies A[L%16][L/16] and B[L/16][L%16] of a 16x4 by 4x16 product;
// accumulator register r holds column L%16 of row 4*(L/16)+r (f32) or of row
// 4*r+L/16 (f64).
#include "smx_kernels.hpp"

namespace smx {

namespace {
constexpr int GM = 64, GK = 32;

template <typename CT> struct Mfma;
template <> struct Mfma<double> {
    typedef double acc_t __attribute__((ext_vector_type(4)));
    __device__ static int out_row(int lane, int r) { return 4 * r + (lane >> 4); }
    __device__ static acc_t run(double a, double b, acc_t c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
};
template <> struct Mfma<float> {
    typedef float acc_t __attribute__((ext_vector_type(4)));
    __device__ static int out_row(int lane, int r) { return 4 * (lane >> 4) + r; }
    __device__ static acc_t run(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
};

template <typename T>
struct alignas(sizeof(T) * 4) Vec4 {
    T v[4];
};

// row stride of the k-major LDS tiles: 64 bytes past a multiple of 128, so that the four
// 16-lane groups of a wavefront (k, k+1, k+2, k+3) fall on alternating halves of the banks
template <typename CT>
__host__ __device__ constexpr int lds_stride(int n)
{
    constexpr int half = 64 / (int)sizeof(CT), full = 128 / (int)sizeof(CT);
    return n + ((half - n % full) + full) % full;
}

// four consecutive elements of a row, zero beyond `limit`; one vector load when the caller vouches for alignment
template <typename TS, typename CT>
__device__ __forceinline__ Vec4<CT> load4(const TS* p, int first, int limit, bool vec)
{
    Vec4<CT> o;
    if (vec && first + 3 < limit) {
        const Vec4<TS> t = *reinterpret_cast<const Vec4<TS>*>(p + first);
#pragma unroll
        for (int j = 0; j < 4; ++j) o.v[j] = (CT)t.v[j];
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) o.v[j] = (first + j < limit) ? (CT)p[first + j] : CT(0);
    }
    return o;
}

template <typename TA, typename TC, typename CT, int NT>
__global__ __launch_bounds__(256) void k_gemm(const GemmParams<TA, TC, CT> g)
{
    constexpr int GN = 16 * NT;
    constexpr int SA = lds_stride<CT>(GM), SW = lds_stride<CT>(GN);
    constexpr int WV = (8 * GN + 255) / 256;          // 4-element groups of the W slab per thread
    __shared__ __align__(32) CT As[GK * SA];
    __shared__ __align__(32) CT Ws[GK * SW];
    __shared__ long a_row_off[GM];
    __shared__ long a2_row_off[GM];
    __shared__ long c_row_off[GM];
    const GemmProb<TA, TC, CT>& pr = g.prob[blockIdx.z];
    const int Nn = pr.Nn, sub = pr.sub;
    const int col0 = blockIdx.y * GN;
    if (col0 >= Nn) return;
    // locate this block's species segment and row tile
    int type = 0, tile = blockIdx.x, nrows_seg = g.num_nodes * sub, seg_node0 = 0;
    if (g.perm) {
        bool found = false;
        for (int t = 0; t < g.T; ++t) {
            const int n_t = g.tstart[t + 1] - g.tstart[t];
            const int tiles = (n_t * sub + GM - 1) / GM;
            if (tile < tiles) { type = t; nrows_seg = n_t * sub; seg_node0 = g.tstart[t]; found = true; break; }
            tile -= tiles;
        }
        if (!found) return;
    } else if (tile * GM >= nrows_seg) {
        return;
    }
    const int row0 = tile * GM;
    const int tid = threadIdx.x;
    if (tid < GM) {
        const int rr = row0 + tid;
        long ao = -1, a2o = -1, co = -1;
        if (rr < nrows_seg) {
            const int ns = rr / sub, sb = rr % sub;
            const int node = g.perm ? g.perm[seg_node0 + ns] : ns;
            ao = (long)node * pr.a_node_stride + pr.a_off + (long)sb * pr.a_sub_stride;
            a2o = (long)node * pr.a2_node_stride;
            co = (long)node * pr.c_node_stride + pr.c_off + (long)sb * pr.c_sub_stride;
        }
        a_row_off[tid] = ao; a2_row_off[tid] = a2o; c_row_off[tid] = co;
    }
    __syncthreads();
    const int wave = tid >> 6, lane = tid & 63;
    typename Mfma<CT>::acc_t acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = {0, 0, 0, 0};

    const int slabs1 = (pr.Kd + GK - 1) / GK;
    const int slabs2 = pr.A2 ? (pr.Kd2 + GK - 1) / GK : 0;
    const bool vec = g.vec_ok != 0;

    // registers of the slab in flight
    Vec4<CT> ra[2], rw[WV];
    const int a_row = tid & 63, a_kc = (tid >> 6) * 8;
    auto fetch = [&](int s) {
        const bool second = s >= slabs1;
        const int k0 = (second ? s - slabs1 : s) * GK;
        const int Kd = second ? pr.Kd2 : pr.Kd;
        const TA* A = second ? pr.A2 : pr.A;
        const long ao = second ? a2_row_off[a_row] : a_row_off[a_row];
        if (ao >= 0) {
            ra[0] = load4<TA, CT>(A + ao, k0 + a_kc, Kd, vec);
            ra[1] = load4<TA, CT>(A + ao, k0 + a_kc + 4, Kd, vec);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) { ra[0].v[j] = CT(0); ra[1].v[j] = CT(0); }
        }
        const CT* W = second ? pr.W2 + (size_t)type * pr.w2_type_stride
                             : pr.W + (size_t)type * pr.w_type_stride + pr.w_off;
        const int trans = second ? pr.transW2 : pr.transW;
#pragma unroll
        for (int q = 0; q < WV; ++q) {
            const int v = tid + q * 256;
#pragma unroll
            for (int j = 0; j < 4; ++j) rw[q].v[j] = CT(0);
            if (v < 8 * GN) {
                if (!trans) {
                    // W block is [Kd][Nn]: four consecutive columns of one k
                    const int k = k0 + v / (GN / 4), n = col0 + (v % (GN / 4)) * 4;
                    if (k < Kd) rw[q] = load4<CT, CT>(W + (size_t)k * Nn, n, Nn, vec);
                } else {
                    // W block is [Nn][Kd]: four consecutive k of one column
                    const int n = col0 + v % GN, k = k0 + (v / GN) * 4;
                    if (n < Nn) rw[q] = load4<CT, CT>(W + (size_t)n * Kd, k, Kd, vec);
                }
            }
        }
    };
    auto stage = [&](int s) {
        const bool second = s >= slabs1;
        const int trans = second ? pr.transW2 : pr.transW;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            As[(a_kc + j) * SA + a_row] = ra[0].v[j];
            As[(a_kc + 4 + j) * SA + a_row] = ra[1].v[j];
        }
#pragma unroll
        for (int q = 0; q < WV; ++q) {
            const int v = tid + q * 256;
            if (v < 8 * GN) {
                if (!trans) {
                    const int k = v / (GN / 4), n = (v % (GN / 4)) * 4;
                    *reinterpret_cast<Vec4<CT>*>(&Ws[k * SW + n]) = rw[q];
                } else {
                    const int n = v % GN, k = (v / GN) * 4;
#pragma unroll
                    for (int j = 0; j < 4; ++j) Ws[(k + j) * SW + n] = rw[q].v[j];
                }
            }
        }
    };

    const int slabs = slabs1 + slabs2;
    fetch(0);
    for (int s = 0; s < slabs; ++s) {
        stage(s);
        __syncthreads();
        if (s + 1 < slabs) fetch(s + 1);
#pragma unroll
        for (int kk = 0; kk < GK; kk += 4) {
            const CT av = As[(kk + (lane >> 4)) * SA + wave * 16 + (lane & 15)];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const CT bv = Ws[(kk + (lane >> 4)) * SW + t * 16 + (lane & 15)];
                acc[t] = Mfma<CT>::run(av, bv, acc[t]);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int nn = col0 + t * 16 + (lane & 15);
        if (nn >= Nn) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const long co = c_row_off[wave * 16 + Mfma<CT>::out_row(lane, r)];
            if (co < 0) continue;
            const CT v = acc[t][r];
            if (pr.accumulate) pr.C[co + nn] = (TC)((CT)pr.C[co + nn] + v);
            else pr.C[co + nn] = (TC)v;
        }
    }
}

template <typename TA, typename TC, typename CT, int NT>
hipError_t launch_gemm_t(const GemmParams<TA, TC, CT>& p, int max_sub, int max_n, hipStream_t s)
{
    constexpr int GN = 16 * NT;
    const long rows = (long)p.num_nodes * max_sub;
    const unsigned gx = (unsigned)((rows + GM - 1) / GM + (p.perm ? p.T : 0));
    const unsigned gy = (unsigned)((max_n + GN - 1) / GN);
    hipLaunchKernelGGL((k_gemm<TA, TC, CT, NT>), dim3(gx, gy, p.nprob), dim3(256), 0, s, p);
    return hipGetLastError();
}
}  // namespace

template <typename TA, typename TC, typename CT>
hipError_t launch_gemm(const GemmParams<TA, TC, CT>& p_in, hipStream_t s)
{
    if (p_in.num_nodes <= 0 || p_in.nprob <= 0) return hipSuccess;
    GemmParams<TA, TC, CT> p = p_in;
    int max_sub = 0, max_n = 0;
    bool vec = true;
    auto mult4 = [](long v) { return v % 4 == 0; };
    for (int z = 0; z < p.nprob; ++z) {
        const auto& q = p.prob[z];
        if (q.A2 && q.sub != 1) return hipErrorInvalidValue;
        max_sub = max_sub > q.sub ? max_sub : q.sub;
        max_n = max_n > q.Nn ? max_n : q.Nn;
        vec = vec && mult4(q.Kd) && mult4(q.Nn) && mult4(q.a_node_stride) && mult4(q.a_off) && mult4(q.a_sub_stride) &&
              mult4(q.w_type_stride) && mult4(q.w_off);
        if (q.A2) vec = vec && mult4(q.Kd2) && mult4(q.a2_node_stride) && mult4(q.w2_type_stride);
    }
    p.vec_ok = vec ? 1 : 0;
    // tile width: the narrowest of 16, 32, 64, 96, 128 that covers the output, else the least padded of 64, 96, 128
    int nt = 8;
    if (max_n <= 16) nt = 1;
    else if (max_n <= 32) nt = 2;
    else if (max_n <= 64) nt = 4;
    else if (max_n <= 96) nt = 6;
    else if (max_n <= 128) nt = 8;
    else {
        long best = -1;
        for (int c : {8, 6, 4}) {
            const long padded = (long)((max_n + 16 * c - 1) / (16 * c)) * 16 * c;
            if (best < 0 || padded < best) { best = padded; nt = c; }
        }
    }
    switch (nt) {
    case 1: return launch_gemm_t<TA, TC, CT, 1>(p, max_sub, max_n, s);
    case 2: return launch_gemm_t<TA, TC, CT, 2>(p, max_sub, max_n, s);
    case 4: return launch_gemm_t<TA, TC, CT, 4>(p, max_sub, max_n, s);
    case 6: return launch_gemm_t<TA, TC, CT, 6>(p, max_sub, max_n, s);
    default: return launch_gemm_t<TA, TC, CT, 8>(p, max_sub, max_n, s);
    }
}
template hipError_t launch_gemm<double, double, double>(const GemmParams<double, double, double>&, hipStream_t);
template hipError_t launch_gemm<float, float, float>(const GemmParams<float, float, float>&, hipStream_t);
template hipError_t launch_gemm<float, double, double>(const GemmParams<float, double, double>&, hipStream_t);
template hipError_t launch_gemm<double, float, double>(const GemmParams<double, float, double>&, hipStream_t);

}  // namespace smx
