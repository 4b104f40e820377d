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

#include <algorithm>
#include <type_traits>

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

// ---------------------------------------------------------------------------
// Row-streaming variant for inner sizes up to 128 (every channel mixing of a K <= 128 model except the
// concatenated ones).  The whole weight block [Kd][GN] sits in LDS for the life of the block, so after
// one barrier the eight wavefronts never synchronise again: wavefront (s, h) streams 16-row tiles
// s, s+4, ... of the block's row range straight from global memory into the A-operand registers (a lane
// loads 32 contiguous bytes per row, i.e. whole 128-byte lines per 16-lane group; the matrix cores see the
// k index permuted inside groups of KG, which a sum over k allows), keeps the next tile's rows in flight
// while it multiplies, and owns the column tiles of half h.  The two wavefronts that share a SIMD thus
// do the same number of matrix instructions.
template <typename T, int N>
struct alignas(16) VecN {
    T v[N];
};
template <typename CT> constexpr int rows_vl() { return 32 / (int)sizeof(CT); }   // k values per lane and group
template <typename CT, int NTW> constexpr int rows_sw() { return 32 * NTW + (sizeof(CT) == 4 ? 2 : 0); }
constexpr int ROWS_KMAX = 128;
constexpr int ROWS_MMAX = 8;                     // 16-row tiles per wavefront at most
constexpr size_t ROWS_OFFS_BYTES = 8 * ROWS_MMAX * 16 * sizeof(int2);

// KQ: the inner sizes the instantiation takes, in quarters of ROWS_KMAX (3: up to 96, 4: up to 128).  Rows are held
// whole in registers (this tile's, the next one's, with SCALED the next one's factors), so K = 96 in the 128-wide
// instantiation pays a quarter more loads and registers than it needs (256 registers with SCALED in fp64).
template <typename TA, typename TC, typename CT, int NTW, bool SCALED, int KQ>
__global__ __launch_bounds__(512) void k_gemm_rows(const GemmParams<TA, TC, CT> g, const int m)
{
    constexpr int VL = rows_vl<CT>(), KG = 4 * VL, KMAXT = ROWS_KMAX * KQ / 4, KJ = KMAXT / KG;
    static_assert(KMAXT % KG == 0, "whole groups of k");
    constexpr int GN = 32 * NTW, SW = rows_sw<CT, NTW>();
    extern __shared__ __align__(16) unsigned char smem_raw[];
    CT* Wl = reinterpret_cast<CT*>(smem_raw);          // [Kp][SW], rows Kd..Kp-1 zero
    const int chunk_rows = 64 * m;
    // Products whose weights do not depend on the species come as a one-dimensional grid of exactly the blocks
    // that have rows, numbered problem by problem: consecutive blocks go to the dies in turn, so the dies get
    // equal shares.  (With species segments the host cannot count the blocks: three-dimensional grid, blocks
    // without rows leave at once.)
    int z = blockIdx.z, chunk = blockIdx.x, cb = blockIdx.y;
    if (!g.perm) {
        int b = blockIdx.x;
        for (z = 0; z < g.nprob; ++z) {
            const int chunks = (g.num_nodes * g.prob[z].sub + chunk_rows - 1) / chunk_rows;
            const int cols = (g.prob[z].Nn + GN - 1) / GN;
            if (b < chunks * cols) { chunk = b / cols; cb = b - chunk * cols; break; }
            b -= chunks * cols;
        }
        if (z == g.nprob) return;
    }
    const GemmProb<TA, TC, CT>& pr = g.prob[z];
    const int Nn = pr.Nn, Kd = pr.Kd, sub = pr.sub;
    const int col0 = cb * GN;
    if (col0 >= Nn) return;
    int type = 0, nrows_seg = g.num_nodes * sub, seg_node0 = 0;
    if (g.perm) {
        bool found = false;
        for (int t = 0; t < g.T; ++t) {
            const int n_t = g.tstart[t + 1] - g.tstart[t];
            const int chunks = (n_t * sub + chunk_rows - 1) / chunk_rows;
            if (chunk < chunks) { type = t; nrows_seg = n_t * sub; seg_node0 = g.tstart[t]; found = true; break; }
            chunk -= chunks;
        }
        if (!found) return;
    } else if ((long)chunk * chunk_rows >= nrows_seg) {
        return;
    }
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int srow = wave & 3, t0 = (wave >> 2) * NTW;
    const int r = lane & 15, gq = lane >> 4;
    const int row_base = chunk * chunk_rows;

    // Row `rr` of the segment as (node, sub-row); beyond the segment the last row with a flag: its A row is
    // still loaded (so that every load below is unconditional straight-line code the matrix instructions
    // need not wait for), what it produces is never stored.
    constexpr int OUTSIDE = 1 << 30;
    auto row_of = [&](int rr) {
        const bool inside = rr < nrows_seg;
        const int rc = inside ? rr : nrows_seg - 1;
        const int ns = rc / sub, sb = rc - ns * sub;
        const int node = g.perm ? g.perm[seg_node0 + ns] : ns;
        return make_int2(node, inside ? sb : sb | OUTSIDE);
    };
    auto a_offset = [&](int2 o) { return (long)o.x * pr.a_node_stride + pr.a_off + (long)(o.y & ~OUTSIDE) * pr.a_sub_stride; };
    auto c_offset = [&](int2 o) {
        return (o.y & OUTSIDE) ? -1L : (long)o.x * pr.c_node_stride + pr.c_off + (long)o.y * pr.c_sub_stride;
    };
    // a run beyond Kx (a multiple of VL) is read from the last run instead: it meets zero rows of the weights
    auto fetch = [&](const TA* A, long ao, int Kx, VecN<CT, VL> (&dst)[KJ]) {
#pragma unroll
        for (int jj = 0; jj < KJ; ++jj) {
            const int k0 = min(jj * KG + gq * VL, Kx - VL);
            const TA* src = A + ao + k0;
#pragma unroll
            for (int q = 0; q < VL; q += 4) {
                const Vec4<TA> t = *reinterpret_cast<const Vec4<TA>*>(src + q);
#pragma unroll
                for (int u = 0; u < 4; ++u) dst[jj].v[q + u] = (CT)t.v[u];
            }
        }
    };

    // A problem with a second product (sub = 1) walks every tile twice: first A with W, then A2 with W2
    // into the same accumulators; both weight blocks are resident.
    const int S = pr.A2 ? 2 : 1;
    const int Kp1 = (Kd + KG - 1) / KG * KG, Kp2 = pr.A2 ? (pr.Kd2 + KG - 1) / KG * KG : 0;
    CT* Wl2 = Wl + (size_t)Kp1 * SW;
    // A weight block goes to LDS in two steps: all loads (four-element groups, WQ per thread at most), later
    // the writes.  The first block's loads are issued before anything else: they are answered from L2 while
    // the species permutation, on which the first rows' addresses depend, is still on its way.
    constexpr int WQ = (KMAXT * (GN / 4) + 511) / 512;
    auto w_issue = [&](const CT* W, int trans, int Kw, int Kp, Vec4<CT> (&w)[WQ]) {
        const int groups = Kp * (GN / 4);
#pragma unroll
        for (int q = 0; q < WQ; ++q) {
            const int v = tid + q * 512;
#pragma unroll
            for (int j = 0; j < 4; ++j) w[q].v[j] = CT(0);
            if (v < groups) {
                if (!trans) {
                    // W block is [Kw][Nn]: four consecutive columns of one k
                    const int k = v / (GN / 4), n = (v % (GN / 4)) * 4;
                    if (k < Kw) w[q] = load4<CT, CT>(W + (size_t)k * Nn, col0 + n, Nn, true);
                } else {
                    // W block is [Nn][Kw]: four consecutive k of one column
                    const int k = (v % (Kp / 4)) * 4, n = v / (Kp / 4);
                    if (col0 + n < Nn) w[q] = load4<CT, CT>(W + (size_t)(col0 + n) * Kw, k, Kw, true);
                }
            }
        }
    };
    auto w_store = [&](CT* dst, int trans, int Kp, const Vec4<CT> (&w)[WQ]) {
        const int groups = Kp * (GN / 4);
#pragma unroll
        for (int q = 0; q < WQ; ++q) {
            const int v = tid + q * 512;
            if (v < groups) {
                if (!trans) {
                    const int k = v / (GN / 4), n = (v % (GN / 4)) * 4;
#pragma unroll
                    for (int j = 0; j < 4; ++j) dst[k * SW + n + j] = w[q].v[j];
                } else {
                    const int k = (v % (Kp / 4)) * 4, n = v / (Kp / 4);
#pragma unroll
                    for (int j = 0; j < 4; ++j) dst[(k + j) * SW + n] = w[q].v[j];
                }
            }
        }
    };
    Vec4<CT> wreg[WQ];
    w_issue(pr.W + (size_t)type * pr.w_type_stride + pr.w_off, pr.transW, Kd, Kp1, wreg);

    // The rows of all tiles of this wavefront go through a private LDS table first (lane group gq fills
    // tiles gq and gq + 4): inside the tile loop the only vector-memory operations are then the row loads
    // and the stores, and no small dependent load has to be waited for behind a tile's stores.
    int2* rows_of = reinterpret_cast<int2*>(smem_raw + (size_t)(Kp1 + Kp2) * SW * sizeof(CT)) + wave * (ROWS_MMAX * 16);
    for (int jt = gq; jt < m; jt += 4) rows_of[jt * 16 + r] = row_of(row_base + (srow + 4 * jt) * 16 + r);
    int2 o_cur = rows_of[r];
    // step u = tile u / S, source u % S
    auto fetch_step = [&](int2 o, int src, VecN<CT, VL> (&dst)[KJ]) {
        if (src == 0) fetch(pr.A, a_offset(o), Kd, dst);
        else fetch(pr.A2, (long)o.x * pr.a2_node_stride, pr.Kd2, dst);
    };
    VecN<CT, VL> a[KJ];
    fetch_step(o_cur, 0, a);
    if constexpr (SCALED) {
        VecN<CT, VL> sc[KJ];
        fetch(pr.Ascale, (long)o_cur.x * pr.ascale_node_stride, Kd, sc);
#pragma unroll
        for (int jj = 0; jj < KJ; ++jj)
#pragma unroll
            for (int q = 0; q < VL; ++q) a[jj].v[q] *= sc[jj].v[q];
    }
    w_store(Wl, pr.transW, Kp1, wreg);
    if (pr.A2) {
        w_issue(pr.W2 + (size_t)type * pr.w2_type_stride, pr.transW2, pr.Kd2, Kp2, wreg);
        w_store(Wl2, pr.transW2, Kp2, wreg);
    }
    __syncthreads();
    if (col0 + t0 * 16 >= Nn) return;                   // this half has no live column
    const int lane_w = gq * VL * SW + t0 * 16 + r;
    typename Mfma<CT>::acc_t acc[NTW];
    const int steps = m * S;
    for (int u = 0; u < steps; ++u) {
        const int j = u / S, src = u - j * S;
        if (row_base + (srow + 4 * j) * 16 >= nrows_seg) break;
        // rows of the next step (past the last one: the last one again, unused)
        const int un = min(u + 1, steps - 1), jn = un / S;
        const int2 o_n = rows_of[jn * 16 + r];
        VecN<CT, VL> an[KJ], sn[SCALED ? KJ : 1];
        fetch_step(o_n, un - jn * S, an);
        // the factor rows stay apart until the hand-over: a product here would wait for both loads
        if constexpr (SCALED) fetch(pr.Ascale, (long)o_n.x * pr.ascale_node_stride, Kd, sn);

        if (src == 0) {
#pragma unroll
            for (int t = 0; t < NTW; ++t) acc[t] = {0, 0, 0, 0};
        }
        const CT* wl = (src ? Wl2 : Wl) + lane_w;
        const int Ks = src ? pr.Kd2 : Kd;
#pragma unroll
        for (int jj = 0; jj < KJ; ++jj) {
            if (jj * KG < Ks) {
#pragma unroll
                for (int q = 0; q < VL; ++q) {
#pragma unroll
                    for (int t = 0; t < NTW; ++t) {
                        const CT bv = wl[(jj * KG + q) * SW + t * 16];
                        acc[t] = Mfma<CT>::run(a[jj].v[q], bv, acc[t]);
                    }
                }
            }
        }
        // The next step's rows become the current ones before this tile's results are stored: waiting for
        // them here waits for loads issued a step ago, after the stores it would wait for the stores too.
#pragma unroll
        for (int jj = 0; jj < KJ; ++jj) {
#pragma unroll
            for (int q = 0; q < VL; ++q) {
                if constexpr (SCALED) a[jj].v[q] = an[jj].v[q] * sn[jj].v[q];
                else a[jj].v[q] = an[jj].v[q];
                asm volatile("" : "+v"(a[jj].v[q]));
            }
        }
        if (src == S - 1) {
            // the offset of output row q is held by lane q
            const long co = c_offset(o_cur);
            long crow[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int from = Mfma<CT>::out_row(lane, q);
                const int lo = __shfl((int)(co & 0xffffffff), from), hi = __shfl((int)(co >> 32), from);
                crow[q] = ((long)hi << 32) | (unsigned)lo;
            }
#pragma unroll
            for (int t = 0; t < NTW; ++t) {
                const int nn = col0 + (t0 + t) * 16 + r;
                if (nn >= Nn) continue;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if (crow[q] < 0) continue;
                    const CT v = acc[t][q];
                    if (pr.accumulate) pr.C[crow[q] + nn] = (TC)((CT)pr.C[crow[q] + nn] + v);
                    else pr.C[crow[q] + nn] = (TC)v;
                }
            }
        }
        o_cur = o_n;
    }
}

template <typename TA, typename TC, typename CT, int NTW, bool SCALED, int KQ>
hipError_t launch_gemm_rows_q(const GemmParams<TA, TC, CT>& p, int max_sub, int max_n, size_t lds, long total_rows,
                              hipStream_t s)
{
    constexpr int GN = 32 * NTW;
    static bool attr_done = false;   // per instantiation
    if (!attr_done) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(k_gemm_rows<TA, TC, CT, NTW, SCALED, KQ>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (err != hipSuccess) return err;
        attr_done = true;
    }
    const unsigned gy = (unsigned)((max_n + GN - 1) / GN);
    // 16-row tiles per SIMD of a block (at most eight): the smallest number with which all blocks that find
    // rows are resident at once.  Blocks go to the eight dies in turn, whatever they find there, so the
    // count leaves an eighth of the block slots free for an uneven split.
    int per_cu = 1;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k_gemm_rows<TA, TC, CT, NTW, SCALED, KQ>, 512, lds) != hipSuccess || per_cu < 1)
        per_cu = 1;
    if (!p.perm) {
        // exact block count: every slot can be used
        auto blocks_for = [&](long mm) {
            long b = 0;
            for (int z = 0; z < p.nprob; ++z)
                b += ((long)p.num_nodes * p.prob[z].sub + 64 * mm - 1) / (64 * mm) * ((p.prob[z].Nn + GN - 1) / GN);
            return b;
        };
        long m = 1;
        while (m < ROWS_MMAX && blocks_for(m) > 256L * per_cu) ++m;
        hipLaunchKernelGGL((k_gemm_rows<TA, TC, CT, NTW, SCALED, KQ>), dim3((unsigned)blocks_for(m)), dim3(512), lds, s, p, (int)m);
        return hipGetLastError();
    }
    const long slots = 224L * per_cu;
    const long slack = std::min<long>((long)p.nprob * p.T, 64);
    long m = 1;
    while (m < ROWS_MMAX && (total_rows + 64 * m - 1) / (64 * m) * gy + slack > slots) ++m;
    const long rows = (long)p.num_nodes * max_sub;
    const unsigned gx = (unsigned)((rows + 64 * m - 1) / (64 * m) + p.T);
    hipLaunchKernelGGL((k_gemm_rows<TA, TC, CT, NTW, SCALED, KQ>), dim3(gx, gy, p.nprob), dim3(512), lds, s, p, (int)m);
    return hipGetLastError();
}

template <typename TA, typename TC, typename CT, int NTW, bool SCALED>
hipError_t launch_gemm_rows_t(const GemmParams<TA, TC, CT>& p, int max_sub, int max_n, size_t lds, long total_rows,
                              hipStream_t s)
{
    // the narrower instantiation for the working precisions (the mixed ones serve inspection calls only)
    if constexpr (std::is_same<TA, CT>::value && std::is_same<TC, CT>::value) {
        int kmax = 0;
        for (int z = 0; z < p.nprob; ++z) kmax = std::max(kmax, std::max(p.prob[z].Kd, p.prob[z].A2 ? p.prob[z].Kd2 : 0));
        if (kmax <= ROWS_KMAX * 3 / 4) return launch_gemm_rows_q<TA, TC, CT, NTW, SCALED, 3>(p, max_sub, max_n, lds, total_rows, s);
    }
    return launch_gemm_rows_q<TA, TC, CT, NTW, SCALED, 4>(p, max_sub, max_n, lds, total_rows, s);
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
    bool scaled = false;
    for (int z = 0; z < p.nprob; ++z) scaled = scaled || p.prob[z].Ascale != nullptr;
    // row-streaming kernel: weights of one block resident in LDS
    {
        constexpr int VL = rows_vl<CT>(), KG = 4 * VL;
        bool rows_ok = vec && max_n >= 32;
        long kp_sum = 0, total_rows = 0;   // padded inner sizes of the widest problem (both products)
        for (int z = 0; z < p.nprob; ++z) {
            const auto& q = p.prob[z];
            if (scaled) rows_ok = rows_ok && q.Ascale && !q.A2 && mult4(q.ascale_node_stride);
            rows_ok = rows_ok && q.Kd <= ROWS_KMAX && q.Kd % VL == 0;
            long kp = (q.Kd + KG - 1) / KG * KG;
            if (q.A2) {
                rows_ok = rows_ok && q.Kd2 <= ROWS_KMAX && q.Kd2 % VL == 0;
                kp += (q.Kd2 + KG - 1) / KG * KG;
            }
            kp_sum = kp_sum > kp ? kp_sum : kp;
            total_rows += (long)p.num_nodes * q.sub;
        }
        if (rows_ok) {
            auto lds_for = [&](int ntw) {
                return (size_t)kp_sum * (32 * ntw + (sizeof(CT) == 4 ? 2 : 0)) * sizeof(CT) + ROWS_OFFS_BYTES;
            };
            // preferred width of a column block: narrow for few rows (more compute units share the work),
            // else the one that tiles the output; narrower when the weight blocks would not fit
            int ntw = (total_rows <= 128 * 64 && max_n % 32 == 0) ? 1 : max_n % 96 == 0 ? 3 : max_n <= 64 ? 2 : 4;
            while (ntw > 1 && lds_for(ntw) > 160 * 1024) --ntw;
            if (ntw == 3 && max_n % 96 != 0) ntw = 2;
            // the factor rows of the next tile take as many registers as the rows themselves: with them the
            // widest column block does not fit the register file
            if (scaled && ntw == 4) ntw = 2;
            const size_t lds = lds_for(ntw);
            if (lds <= 160 * 1024 && !scaled) {
                switch (ntw) {
                case 1: return launch_gemm_rows_t<TA, TC, CT, 1, false>(p, max_sub, max_n, lds, total_rows, s);
                case 2: return launch_gemm_rows_t<TA, TC, CT, 2, false>(p, max_sub, max_n, lds, total_rows, s);
                case 3: return launch_gemm_rows_t<TA, TC, CT, 3, false>(p, max_sub, max_n, lds, total_rows, s);
                default: return launch_gemm_rows_t<TA, TC, CT, 4, false>(p, max_sub, max_n, lds, total_rows, s);
                }
            }
            if constexpr (std::is_same<TA, CT>::value && std::is_same<TC, CT>::value) {
                if (lds <= 160 * 1024 && scaled) {
                    switch (ntw) {
                    case 1: return launch_gemm_rows_t<TA, TC, CT, 1, true>(p, max_sub, max_n, lds, total_rows, s);
                    case 2: return launch_gemm_rows_t<TA, TC, CT, 2, true>(p, max_sub, max_n, lds, total_rows, s);
                    default: return launch_gemm_rows_t<TA, TC, CT, 3, true>(p, max_sub, max_n, lds, total_rows, s);
                    }
                }
            }
        }
    }
    if (scaled) return hipErrorInvalidValue;   // callers check gemm_scaled_operand_ok first
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
bool gemm_scaled_operand_ok(int Kd, int Nn, size_t elem)
{
    const int vl = 32 / (int)elem;
    return Kd <= ROWS_KMAX && Kd % vl == 0 && Nn >= 32 && Nn % 4 == 0;
}
template hipError_t launch_gemm<double, double, double>(const GemmParams<double, double, double>&, hipStream_t);
template hipError_t launch_gemm<float, float, float>(const GemmParams<float, float, float>&, hipStream_t);
template hipError_t launch_gemm<float, double, double>(const GemmParams<float, double, double>&, hipStream_t);
template hipError_t launch_gemm<double, float, double>(const GemmParams<double, float, double>&, hipStream_t);

}  // namespace smx
