// Channel-slice edge kernels for gfx950 (scalar hidden features, P = 4 paths).
//
// The radial spline table is the hot operand of the edge stages: every edge
// needs 4 coefficient rows x 4 paths x K channels (12 KB at K = 96 in double),
// far more than its geometry or its sender row.  These kernels cut the channel
// axis into slices of CH channels, small enough that the whole table slice
// ([intervals][4][4][CH], about 130 KB) stays resident in the 160 KB LDS of a
// CU.  A block owns one slice; its lanes own receivers (SPLIT lanes share one
// receiver and take alternate edges) and walk the receiver's edge list, so that
//   - spline coefficients come from LDS, never from L2/HBM, after one
//     contiguous copy of the slice per block,
//   - harmonics are evaluated by the lane that uses them (no staging),
//   - accumulators (16 x CH per lane) stay in registers, sums run in edge
//     order, no atomics: results are bit-reproducible.
// The adjoint kernel writes, per slice, a partial force per edge; a last kernel
// adds the partials over slices in a fixed order.
#include "smx_device.hpp"
#include "smx_kernels.hpp"

#include <algorithm>

namespace smx {

namespace {

// The table slice of a block, global memory -> LDS (both sides 16-byte aligned, size a multiple of 16).  Whole
// kilobytes go through loads that write straight into LDS (16 bytes per lane, the 64 lanes of a wavefront side by
// side, no registers in between), so that a wavefront has all its pieces in flight at once; the caller's barrier
// follows the wait for them.
__device__ __forceinline__ void copy_slice_to_lds(const void* src, void* dst, size_t bytes)
{
    typedef const __attribute__((address_space(1))) void* GlobalPtr;
    typedef __attribute__((address_space(3))) void* LdsPtr;
    const char* s = reinterpret_cast<const char*>(src);
    char* d = reinterpret_cast<char*>(dst);
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
    const int waves = blockDim.x >> 6;
    const int chunks = (int)(bytes / 1024);
    for (int q = wave; q < chunks; q += waves)
        __builtin_amdgcn_global_load_lds((GlobalPtr)(s + (size_t)q * 1024 + lane * 16), (LdsPtr)(d + (size_t)q * 1024), 16, 0, 0);
    const size_t tail = (size_t)chunks * 1024;
    for (size_t q = tail + threadIdx.x * 16; q < bytes; q += (size_t)blockDim.x * 16)
        *reinterpret_cast<uint4*>(d + q) = *reinterpret_cast<const uint4*>(s + q);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the direct loads have written the LDS
}

// Which slice and which receiver group a block works on.  Blocks go to the eight dies in turn (block b to die
// b % 8), and every die has its own L2.  A slice's share of a feature row is 32 bytes, so four consecutive slices
// share a 128-byte cache line.  The unit that must stay on one die is therefore (line of four slices, receiver
// group): its four blocks read and write whole lines of the rows of their receivers (adjoint rows, messages, sums)
// in one L2, where the partial writes merge.  Units are numbered receiver group first, then line, and each die
// takes a contiguous eighth of them: a die's blocks mostly share their receivers, hence the edge arrays they read.
struct BlockSlot { int slice, group; };
__device__ __forceinline__ BlockSlot block_slot(int units_per_die, int lines, int num_units)
{
    const int die = blockIdx.x % 8, j = blockIdx.x / 8;
    const int unit = die * units_per_die + j / 4;
    if (j >= 4 * units_per_die || unit >= num_units) return {1 << 28, 0};   // no work: a slice past the last
    return {4 * (unit % lines) + j % 4, unit / lines};
}
// receiver groups of a launch over S slices: one block per CU, and no die with more blocks than it has CUs (an eighth
// of them; four blocks per unit)
template <typename P>
static inline void place_blocks(P& q, int S, int& RG, unsigned& blocks)
{
    const int lines = (S + 3) / 4;
    const int max_units = q.num_cus / 4 > 0 ? q.num_cus / 4 : 1;
    if (RG * lines > max_units) RG = max_units / lines > 0 ? max_units / lines : 1;
    q.slot_lines = lines;
    q.num_units = lines * RG;
    q.units_per_die = (q.num_units + 7) / 8;
    q.receiver_groups = RG;
    blocks = 8u * 4u * (unsigned)q.units_per_die;
}

// The tasks of a block (groups of receivers, largest first) are handed to its wavefronts as they become free: an
// integer counter in LDS, so that the wavefronts of a block finish together whatever the degrees.  Which wavefront
// takes a task has no influence on any result (a task's sums are its own).
__device__ __forceinline__ int next_block_task(int* counter)
{
    int j = 0;
    if ((threadIdx.x & 63) == 0) j = atomicAdd(counter, 1);
    return __builtin_amdgcn_readfirstlane(j);
}

struct EdgeGeo {
    double dx, dy, dz, r;
    int g;
};
template <typename F>
__device__ __forceinline__ EdgeGeo load_edge(const AggParams<F>& a, int e)
{
    EdgeGeo q;
    q.dx = a.xyz[3 * (size_t)e]; q.dy = a.xyz[3 * (size_t)e + 1]; q.dz = a.xyz[3 * (size_t)e + 2];
    q.r = a.r[e];
    q.g = a.gather[e];
    return q;
}

// cu <- nx with moves the compiler cannot postpone: where this stands, the wait for nx stands
__device__ __forceinline__ void take_edge(EdgeGeo& cu, const EdgeGeo& nx)
{
    asm volatile("v_mov_b64 %0, %4\n\tv_mov_b64 %1, %5\n\tv_mov_b64 %2, %6\n\tv_mov_b64 %3, %7"
                 : "=&v"(cu.dx), "=&v"(cu.dy), "=&v"(cu.dz), "=&v"(cu.r) : "v"(nx.dx), "v"(nx.dy), "v"(nx.dz), "v"(nx.r));
    asm volatile("v_mov_b32 %0, %1" : "=v"(cu.g) : "v"(nx.g));
}

// Scheduling fences without instructions: what is computed from vx, vy, vz after order_l cannot start
// before the five sums are final; pin_value ends the live range of an accumulation's operands here.
template <typename F>
__device__ __forceinline__ void order_l(F& s0, F& s1, F& s2, F& s3, F& s4, double& vx, double& vy, double& vz)
{
    asm volatile("" : "+v"(s0), "+v"(s1), "+v"(s2), "+v"(s3), "+v"(s4), "+v"(vx), "+v"(vy), "+v"(vz));
}
template <typename F>
__device__ __forceinline__ void pin_value(F& v)
{
    asm volatile("" : "+v"(v));
}

// Single precision: the kernels wait on the LDS, and reading the paths in an order rotated by the lane's edge
// slot removes the bank conflicts between the edges served in one LDS cycle (rows are multiples of 128 bytes
// there, the four paths of a coefficient lie 32 bytes apart).  Double precision: the kernels wait on vector
// issue, the selects that undo the rotation cost more than the conflicts; rows are padded to an odd number of
// 16-byte words instead.  The host lays the table out accordingly (slice_row_elements).
template <typename F> __host__ __device__ constexpr bool slice_rotates() { return sizeof(F) == 4; }

// v[l] <- v[(l - rot) & 3] for rot = 0..3, as two conditional rotations by one and by two
template <typename F>
__device__ __forceinline__ void unrotate4(F* v, int rot)
{
    const bool r1 = rot & 1, r2 = rot & 2;
    const F a0 = r1 ? v[3] : v[0], a1 = r1 ? v[0] : v[1], a2 = r1 ? v[1] : v[2], a3 = r1 ? v[2] : v[3];
    v[0] = r2 ? a2 : a0; v[1] = r2 ? a3 : a1; v[2] = r2 ? a0 : a2; v[3] = r2 ? a1 : a3;
}

// ---------------------------------------------------------------------------
// Lane mapping of both kernels.  A wavefront works on four receivers at a time,
// one per 16-lane row.  Inside a row, CL lanes share an edge and split the CH
// channels of the slice between them (CPLN = CH/CL consecutive channels per
// lane, one 16-byte LDS read per coefficient), and 16/CL edges are in flight.
// The LDS unit serves a 16-byte read 8 lanes per cycle, i.e. 8/CL edges whose
// lanes read adjacent bytes: far fewer distinct rows per cycle than with one
// edge per lane, hence far fewer bank conflicts.
template <typename F, int CH, int CL, int BT>
__global__ __launch_bounds__(BT) void k_slice_fwd(const SliceParams<F> p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const F* lds = reinterpret_cast<const F*>(smem);
    const AggParams<F>& a = p.a;
    constexpr int CPLN = CH / CL, EPR = 16 / CL;
    const BlockSlot slot_of_block = block_slot(p.units_per_die, p.slot_lines, p.num_units);
    const int slice = slot_of_block.slice, K = a.K;
    if ((long)slice * CH >= K) return;                      // a block without a slot
    const int W = p.W, R = a.spl_nodes - 1;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int sub = lane & 15, e_sub = sub / CL, cs = sub % CL;
    const int kc = slice * CH + cs * CPLN;                 // first channel of this lane
    const int rot = slice_rotates<F>() ? (e_sub & 3) : 0;
    int poff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) poff[i] = ((i + rot) & 3) * CH;
    const int wave_tasks = (a.num_nodes + 3) / 4;
    __shared__ int task_counter;

    if (threadIdx.x == 0) task_counter = 0;
    copy_slice_to_lds(p.tabS + (size_t)slice * R * W, smem, (size_t)R * W * sizeof(F));
    __syncthreads();
    for (int task = slot_of_block.group + p.receiver_groups * next_block_task(&task_counter); task < wave_tasks;
         task = slot_of_block.group + p.receiver_groups * next_block_task(&task_counter)) {
        const int slot = task * 4 + (lane >> 4);
        const bool live = slot < a.num_nodes;
        const int i = live ? p.order[slot] : 0;
        int e0 = 0, e1 = 0;
        if (live) { e0 = a.first_neigh[i]; e1 = a.first_neigh[i + 1]; }
        F acc[16][CPLN];
#pragma unroll
        for (int q = 0; q < 16; ++q)
#pragma unroll
            for (int c = 0; c < CPLN; ++c) acc[q][c] = F(0);
        // the geometry of the next edge of this lane is loaded while the current one is processed
        EdgeGeo nx = {1.0, 0.0, 0.0, 1.0, 0};
        {
            const int ef = e0 + e_sub;
            if (ef < e1) nx = load_edge(a, ef);
        }
        for (int e = e0 + e_sub; e < e1; e += EPR) {
            const EdgeGeo cu = nx;
            nx = load_edge(a, min(e + EPR, e1 - 1));   // unconditional: a conditional load costs a register copy per value
            const double dx = cu.dx, dy = cu.dy, dz = cu.dz;
            const double r = cu.r;
            const int g = cu.g;
            const double inv = rsqrt_pos(dx * dx + dy * dy + dz * dz);
            double Yd[16];
            sph_l3(dz * inv, dx * inv, dy * inv, Yd);
            const int n = spline_interval(r, a.spl_inv_h, R - 1);
            const F x = (F)(r - a.spl_h * n);
            const F* row = lds + (size_t)n * W + cs * CPLN;
            // step i reads path (i + rot) & 3, rot = this lane's edge slot in single precision, else 0
            F t[CPLN][4];
#pragma unroll
            for (int c = 0; c < CPLN; ++c) {
                const F h = a.Hsrc[(size_t)g * K + min(kc + c, K - 1)];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const F* rp = row + poff[i] + c;
                    const F c0 = rp[0], c1 = rp[4 * CH], c2 = rp[8 * CH], c3 = rp[12 * CH];
                    t[c][i] = (c0 + x * (c1 + x * (c2 + x * c3))) * h;
                }
                if constexpr (slice_rotates<F>()) unrotate4(t[c], rot);
            }
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const F y = (F)Yd[q];
#pragma unroll
                for (int c = 0; c < CPLN; ++c) acc[q][c] += t[c][lm_l(q)] * y;
            }
        }
        // add up the lanes of the row that hold the same channels (they took alternate edges)
#pragma unroll
        for (int q = 0; q < 16; ++q)
#pragma unroll
            for (int c = 0; c < CPLN; ++c) acc[q][c] = row_sum_strided<CL>(acc[q][c]);
        if (live && e_sub == 0) {
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const F cd = (F)p.cdiag[q];
#pragma unroll
                for (int c = 0; c < CPLN; ++c)
                    if (kc + c < K) {
                        F* o = a.out + ((size_t)i * 16 + q) * K + kc + c;
                        *o = acc[q][c] * cd;
                    }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Forward kernel for slices of 32 bytes of channels (four lanes per edge, CH / 4 channels each) with a table layout
// made for the LDS banks.  A row is [4 paths][2 halves][4 lanes][16 bytes]: the 16 bytes hold, for the lane's
// channels, the coefficient pair (c0, c1) in half 0 and (c2, c3) in half 1, so that the four lanes of an edge read 64
// contiguous bytes per instruction.  Rows are 512 bytes, so every edge's 64 bytes would fall on the same half of the
// banks; edges in odd slots therefore read the halves in the opposite order, an even and an odd edge fill one 128-byte
// bank row per cycle, and no read conflicts with another whatever the rows.  The cubic is evaluated as
// (c0 + c1 x) + x^2 (c2 + c3 x): the two brackets are formed from whichever half arrived first and second, and
// the lane's factors (1, x^2) or (x^2, 1), already multiplied with the sender feature, put them together.
template <typename F, int BT>
__global__ __launch_bounds__(BT) void k_slice_fwd_halves(const SliceParams<F> p)
{
    constexpr int CH = 32 / (int)sizeof(F), CL = 4, CPLN = CH / CL, EPR = 16 / CL;
    using V = Vec<F, 2 * CPLN>;                            // 16 bytes
    extern __shared__ __align__(16) unsigned char smem[];
    const F* lds = reinterpret_cast<const F*>(smem);
    const AggParams<F>& a = p.a;
    const BlockSlot slot_of_block = block_slot(p.units_per_die, p.slot_lines, p.num_units);
    const int slice = slot_of_block.slice, K = a.K;
    if ((long)slice * CH >= K) return;                      // a block without a slot
    constexpr int WF = 512 / (int)sizeof(F);               // row length in elements
    const int R = a.spl_nodes - 1;
    const int lane = threadIdx.x & 63;
    const int sub = lane & 15, e_sub = sub / CL, cs = sub % CL;
    const int kc = slice * CH + cs * CPLN;                 // first channel of this lane
    const int par = e_sub & 1;
    const int off_first = (par * 4 + cs) * 2 * CPLN, off_second = ((par ^ 1) * 4 + cs) * 2 * CPLN;
    const int wave_tasks = (a.num_nodes + 3) / 4;
    __shared__ int task_counter;

    if (threadIdx.x == 0) task_counter = 0;
    copy_slice_to_lds(p.tabF + (size_t)slice * R * WF, smem, (size_t)R * 512);
    __syncthreads();
    for (int task = slot_of_block.group + p.receiver_groups * next_block_task(&task_counter); task < wave_tasks;
         task = slot_of_block.group + p.receiver_groups * next_block_task(&task_counter)) {
        const int slot = task * 4 + (lane >> 4);
        const bool live = slot < a.num_nodes;
        const int i = live ? p.order[slot] : 0;
        int e0 = 0, e1 = 0;
        if (live) { e0 = a.first_neigh[i]; e1 = a.first_neigh[i + 1]; }
        F acc[16][CPLN];
#pragma unroll
        for (int q = 0; q < 16; ++q)
#pragma unroll
            for (int c = 0; c < CPLN; ++c) acc[q][c] = F(0);
        // the geometry of the next edge of this lane is loaded while the current one is processed
        EdgeGeo nx = {1.0, 0.0, 0.0, 1.0, 0};
        {
            const int ef = e0 + e_sub;
            if (ef < e1) nx = load_edge(a, ef);
        }
        for (int e = e0 + e_sub; e < e1; e += EPR) {
            const EdgeGeo cu = nx;
            nx = load_edge(a, min(e + EPR, e1 - 1));   // unconditional: a conditional load costs a register copy per value
            const int g = cu.g;
            const double dx = cu.dx, dy = cu.dy, dz = cu.dz;
            const double r = cu.r;
            const double inv = rsqrt_pos(dx * dx + dy * dy + dz * dz);
            double Yd[16];
            sph_l3(dz * inv, dx * inv, dy * inv, Yd);
            const int n = spline_interval(r, a.spl_inv_h, R - 1);
            const F x = (F)(r - a.spl_h * n);
            const F x2 = x * x;
            const F* row = lds + (size_t)n * WF;
            F s_first[CPLN], s_second[CPLN];
#pragma unroll
            for (int c = 0; c < CPLN; ++c) {
                const F h = a.Hsrc[(size_t)g * K + min(kc + c, K - 1)];
                const F hx = h * x2;
                s_first[c] = par ? hx : h;
                s_second[c] = par ? h : hx;
            }
            F t[CPLN][4];
#pragma unroll
            for (int l = 0; l < 4; ++l) {
                const V first = *reinterpret_cast<const V*>(row + l * 16 * CPLN + off_first);
                const V second = *reinterpret_cast<const V*>(row + l * 16 * CPLN + off_second);
#pragma unroll
                for (int c = 0; c < CPLN; ++c) {
                    const F u = first.v[2 * c] + first.v[2 * c + 1] * x;
                    const F v = second.v[2 * c] + second.v[2 * c + 1] * x;
                    t[c][l] = u * s_first[c] + v * s_second[c];
                }
            }
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const F y = (F)Yd[q];
#pragma unroll
                for (int c = 0; c < CPLN; ++c) acc[q][c] += t[c][lm_l(q)] * y;
            }
        }
        // add up the lanes of the row that hold the same channels (they took alternate edges)
#pragma unroll
        for (int q = 0; q < 16; ++q)
#pragma unroll
            for (int c = 0; c < CPLN; ++c) acc[q][c] = row_sum_strided<CL>(acc[q][c]);
        if (live && e_sub == 0) {
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const F cd = (F)p.cdiag[q];
#pragma unroll
                for (int c = 0; c < CPLN; ++c)
                    if (kc + c < K) {
                        F* o = a.out + ((size_t)i * 16 + q) * K + kc + c;
                        *o = acc[q][c] * cd;
                    }
            }
        }
    }
}

// ---------------------------------------------------------------------------
template <typename F, int CH, int CL, int BT>
__global__ __launch_bounds__(BT) void k_slice_bwd(const SliceParams<F> p)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const F* lds = reinterpret_cast<const F*>(smem);
    const AggParams<F>& a = p.a;
    constexpr int CPLN = CH / CL, EPR = 16 / CL;
    const BlockSlot slot_of_block = block_slot(p.units_per_die, p.slot_lines, p.num_units);
    const int slice = slot_of_block.slice, K = a.K;
    if ((long)slice * CH >= K) return;                      // a block without a slot
    const int W = p.W, R = a.spl_nodes - 1;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int sub = lane & 15, e_sub = sub / CL, cs = sub % CL;
    const int kc = slice * CH + cs * CPLN;
    const int rot = slice_rotates<F>() ? (e_sub & 3) : 0;
    int poff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) poff[i] = ((i + rot) & 3) * CH;
    const int wave_tasks = (a.num_nodes + 3) / 4;
    __shared__ int task_counter;
    double* fpart = p.fpart + (size_t)slice * p.E * 3;

    if (threadIdx.x == 0) task_counter = 0;
    copy_slice_to_lds(p.tabS + (size_t)slice * R * W, smem, (size_t)R * W * sizeof(F));
    __syncthreads();
    for (int task = slot_of_block.group + p.receiver_groups * next_block_task(&task_counter); task < wave_tasks;
         task = slot_of_block.group + p.receiver_groups * next_block_task(&task_counter)) {
        const int slot = task * 4 + (lane >> 4);
        const bool live = slot < a.num_nodes;
        const int i = live ? p.order[slot] : 0;
        int e0 = 0, e1 = 0;
        if (live) { e0 = a.first_neigh[i]; e1 = a.first_neigh[i + 1]; }
        F d[16][CPLN];
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const F cd = (F)p.cdiag[q];
#pragma unroll
            for (int c = 0; c < CPLN; ++c)
                d[q][c] = (live && kc + c < K) ? a.d_out[((size_t)i * 16 + q) * K + kc + c] * cd : F(0);
        }
        // the lanes of a row iterate together so that the cross-lane sums below see all CL partners
        const int iters = (e1 - e0 + EPR - 1) / EPR;
        EdgeGeo nx = {1.0, 0.0, 0.0, 1.0, 0};
        {
            const int ef = e0 + e_sub;
            if (ef < e1) nx = load_edge(a, ef);
        }
        for (int it = 0; it < iters; ++it) {
            const int e = e0 + it * EPR + e_sub;
            bool on = e < e1;
            const EdgeGeo cu = nx;
            nx = load_edge(a, min(e + EPR, e1 - 1));   // unconditional: a conditional load costs a register copy per value
            double fx = 0.0, fy = 0.0, fz = 0.0;
            if (on) {
                const double dx = cu.dx, dy = cu.dy, dz = cu.dz;
                const double r = cu.r;
                const int g = cu.g;
                const double inv = rsqrt_pos(dx * dx + dy * dy + dz * dz);
                const double ux = dz * inv, uy = dx * inv, uz = dy * inv;   // permuted unit vector
                const int n = spline_interval(r, a.spl_inv_h, R - 1);
                const F x = (F)(r - a.spl_h * n);
                const F* row = lds + (size_t)n * W + cs * CPLN;
                F srad = F(0), wx = F(0), wy = F(0), wz = F(0), lterm = F(0);
                F h[CPLN], mg[CPLN], Rv[CPLN][4], Rd[CPLN][4];
#pragma unroll
                for (int c = 0; c < CPLN; ++c) {
                    h[c] = a.Hsrc[(size_t)g * K + min(kc + c, K - 1)]; mg[c] = F(0);
                    // paths read in the rotated order of this lane's edge slot (see the forward kernel)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const F* rp = row + poff[i] + c;
                        const F c0 = rp[0], c1 = rp[4 * CH], c2 = rp[8 * CH], c3 = rp[12 * CH];
                        Rv[c][i] = c0 + x * (c1 + x * (c2 + x * c3));
                        Rd[c][i] = c1 + x * (F(2) * c2 + F(3) * x * c3);
                    }
                    if constexpr (slice_rotates<F>()) { unrotate4(Rv[c], rot); unrotate4(Rd[c], rot); }
                }
                // One order l at a time: its harmonics are formed, used for all channels of the lane and
                // dropped; the fence keeps the next order's harmonics from being formed early (all 16
                // with their derivatives would hold 128 registers).
                double vx = ux, vy = uy, vz = uz;
                static_for<0, 4>([&](auto lc) {
                    constexpr int l = decltype(lc)::value;
                    F Yl[2 * l + 1], g0[2 * l + 1], g1[2 * l + 1], g2[2 * l + 1];
                    static_for<0, 2 * l + 1>([&](auto mc) {
                        constexpr int m = decltype(mc)::value;
                        double y, a0, a1, a2;
                        ylm_g<l * l + m>(vx, vy, vz, y, a0, a1, a2);
                        Yl[m] = (F)y; g0[m] = (F)a0; g1[m] = (F)a1; g2[m] = (F)a2;
                    });
#pragma unroll
                    for (int c = 0; c < CPLN; ++c) {
                        F ul = F(0), v0 = F(0), v1 = F(0), v2 = F(0);
#pragma unroll
                        for (int m = 0; m < 2 * l + 1; ++m) {
                            const F dd = d[l * l + m][c];
                            ul += dd * Yl[m];
                            v0 += dd * g0[m]; v1 += dd * g1[m]; v2 += dd * g2[m];
                        }
                        const F Rh = Rv[c][l] * h[c];
                        srad += Rd[c][l] * h[c] * ul;
                        wx += Rh * v0; wy += Rh * v1; wz += Rh * v2;
                        lterm += Rh * ul * F(l);
                        mg[c] += Rv[c][l] * ul;
                    }
                    order_l(srad, wx, wy, wz, lterm, vx, vy, vz);
#pragma unroll
                    for (int c = 0; c < CPLN; ++c) pin_value(mg[c]);
                });
                if (a.msg) {
#pragma unroll
                    for (int c = 0; c < CPLN; ++c)
                        if (kc + c < K) a.msg[(size_t)e * K + kc + c] = mg[c];
                }
                // gradient with respect to the edge vector: (w - u (l-weighted sum)) / |v|, axes unpermuted;
                // radial part along xyz / r with the caller's r (mace.cpp:256-264, 558-566)
                const double sr = (double)srad, lt = (double)lterm;
                const double ir = rcp_pos(r);
                fx = -(dx * ir * sr + ((double)wy - uy * lt) * inv);   // original x is permuted axis 1
                fy = -(dy * ir * sr + ((double)wz - uz * lt) * inv);   // original y is permuted axis 2
                fz = -(dz * ir * sr + ((double)wx - ux * lt) * inv);   // original z is permuted axis 0
            }
            // channels of the slice are spread over CL adjacent lanes: add their partial forces
            if constexpr (CL >= 2) { fx += lane_xor1(fx); fy += lane_xor1(fy); fz += lane_xor1(fz); }
            if constexpr (CL >= 4) { fx += lane_xor2(fx); fy += lane_xor2(fy); fz += lane_xor2(fz); }
            if constexpr (CL >= 8) { fx += half_mirror(fx); fy += half_mirror(fy); fz += half_mirror(fz); }
            if (on && cs == 0) {
                fpart[3 * (size_t)e] = fx; fpart[3 * (size_t)e + 1] = fy; fpart[3 * (size_t)e + 2] = fz;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Adjoint kernel, one lane per edge.  A 16-lane row serves one receiver and takes 16 of its edges at a time;
// every lane holds all CH channels of the slice for its edge (CH * sizeof(F) = 32 bytes: one sender-row load, two
// 16-byte LDS reads per coefficient).  The direction, the harmonics and their gradient are formed once per
// (edge, slice) instead of once per (edge, channel): for every harmonic the lane first sums over its channels,
//     P = sum_c d[lm][c] h[c] R_l[c],   Q = sum_c d[lm][c] h[c] R'_l[c],
// and only then multiplies with Y_lm and its gradient.  No lane talks to another one.  The receiver's adjoint
// rows d[16][CH] (times the coupling constant) are staged per wavefront in the LDS left free by the table slice
// and read back as broadcasts, one harmonic at a time.  tabS rows here are [4 coefficients][4 paths][CH] padded to
// W elements with W * sizeof(F) = 16 (mod 32), so that the rows of 16 edges spread over the banks.
template <typename F, int CH, int BT, int RL, bool MSG, bool CARRY, bool WHOLE>
__global__ __launch_bounds__(BT) void k_slice_bwd_edge(const SliceParams<F> p)
{
    static_assert(CH * sizeof(F) == 32, "a lane moves its channels as two 16-byte words");
    extern __shared__ __align__(16) unsigned char smem[];
    using V = Vec<F, CH>;
    const F* lds = reinterpret_cast<const F*>(smem);
    const AggParams<F>& a = p.a;
    const BlockSlot slot_of_block = block_slot(p.units_per_die, p.slot_lines, p.num_units);
    const int slice = slot_of_block.slice, K = a.K;
    if ((long)slice * CH >= K) return;                      // a block without a slot
    const int W = p.W, R = a.spl_nodes - 1;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    constexpr int ROWS = 64 / RL;                            // receivers a wavefront works on at a time
    const int row = lane / RL, sub = lane % RL;
    const int kc = slice * CH;
    // all channels of the slice exist (WHOLE: of every slice) and rows of K elements keep its 32-byte pieces on
    // 16-byte addresses: only then are they moved as vectors
    const bool whole = WHOLE || (kc + CH <= K && (K * sizeof(F)) % 16 == 0);
    // staged adjoint rows of the wavefront's receivers, [harmonic][receiver][CH]: the receivers' reads of one
    // harmonic (same instruction, one 32-byte piece each) cover contiguous memory
    F* dstage = reinterpret_cast<F*>(smem + (size_t)R * W * sizeof(F)) + ((size_t)wave * 16 * ROWS + row) * CH;
    const int wave_tasks = (a.num_nodes + ROWS - 1) / ROWS;
    __shared__ int task_counter;
    double* fpart = p.fpart + (size_t)slice * p.E * 3;

    if (threadIdx.x == 0) task_counter = 0;
    copy_slice_to_lds(p.tabS + (size_t)slice * R * W, smem, (size_t)R * W * sizeof(F));
    __syncthreads();
    for (int task = slot_of_block.group + p.receiver_groups * next_block_task(&task_counter); task < wave_tasks;
         task = slot_of_block.group + p.receiver_groups * next_block_task(&task_counter)) {
        const int slot = task * ROWS + row;
        const bool live = slot < a.num_nodes;
        const int i = live ? p.order[slot] : 0;
        int e0 = 0, e1 = 0;
        if (live) { e0 = a.first_neigh[i]; e1 = a.first_neigh[i + 1]; }
        // the lanes of the row bring the receiver's adjoint rows, one harmonic each per round
        wave_lds_sync();                                       // the previous task's reads are done
#pragma unroll
        for (int lm = sub; lm < 16; lm += RL) {
            V v;
#pragma unroll
            for (int c = 0; c < CH; ++c) v.v[c] = F(0);
            if (live) {
                const F* src = a.d_out + ((size_t)i * 16 + lm) * K + kc;
                if (whole) v = *reinterpret_cast<const V*>(src);
                else {
#pragma unroll
                    for (int c = 0; c < CH; ++c) if (kc + c < K) v.v[c] = src[c];
                }
            }
            const F cd = (F)p.cdiag[lm];
#pragma unroll
            for (int c = 0; c < CH; ++c) v.v[c] *= cd;
            *reinterpret_cast<V*>(dstage + lm * ROWS * CH) = v;
        }
        wave_lds_sync();
        const int iters = (e1 - e0 + RL - 1) / RL;
        auto sender_row = [&](int g) {
            V h;
            const F* src = a.Hsrc + (size_t)g * K + kc;
            if (whole) h = *reinterpret_cast<const V*>(src);
            else {
#pragma unroll
                for (int c = 0; c < CH; ++c) h.v[c] = src[min(c, K - 1 - kc)];
            }
            return h;
        };
        // Loads and stores share one in-order counter: a wait for a load that was requested after a store also waits
        // for the store to be acknowledged.  So everything the next iteration needs early is requested before this
        // iteration's stores: the next edge one iteration ahead (nx, copied into cu before the stores), the sender's
        // row and the partial forces an earlier stage left for the edge right before the stores, into the
        // registers the finished edge has just given up.
        EdgeGeo cu = {1.0, 0.0, 0.0, 1.0, 0}, nx = cu;
        V h;
#pragma unroll
        for (int c = 0; c < CH; ++c) h.v[c] = F(0);
        double f0 = 0.0, f1 = 0.0, f2 = 0.0;
        if (e0 + sub < e1) {
            const int ef = e0 + sub;
            cu = load_edge(a, ef);
            if constexpr (CARRY) { f0 = fpart[3 * (size_t)ef]; f1 = fpart[3 * (size_t)ef + 1]; f2 = fpart[3 * (size_t)ef + 2]; }
            h = sender_row(cu.g);
        }
        // nothing outstanding on entry: the waits inside the loop are then counted along the loop alone (merged with a
        // way in that has loads in flight and no stores, they would assume fewer operations behind a load than the loop
        // has, and wait for its stores)
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        for (int it = 0; it < iters; ++it) {
            const int e = e0 + it * RL + sub;
            const int en = min(e + RL, e1 - 1);
            nx = load_edge(a, en);   // unconditional: a conditional load costs a register copy per value
            if (e >= e1) continue;
            const double dx = cu.dx, dy = cu.dy, dz = cu.dz, r = cu.r;
            const double inv = rsqrt_pos(dx * dx + dy * dy + dz * dz);
            const double ux = dz * inv, uy = dx * inv, uz = dy * inv;   // permuted unit vector
            const int n = spline_interval(r, a.spl_inv_h, R - 1);
            const F x = (F)(r - a.spl_h * n);
            const F* rowp = lds + (size_t)n * W;
            auto piece = [&](int q, int l) { return *reinterpret_cast<const V*>(rowp + (q * 4 + l) * CH); };
            F srad = F(0), wx = F(0), wy = F(0), wz = F(0), lterm = F(0);
            F mg[CH];
#pragma unroll
            for (int c = 0; c < CH; ++c) mg[c] = F(0);
            double vx = ux, vy = uy, vz = uz;
            // one order l at a time (the fence keeps the harmonics of the next order from being formed early)
            static_for<0, 4>([&](auto lc) {
                constexpr int l = decltype(lc)::value;
                F ul[CH];
#pragma unroll
                for (int c = 0; c < CH; ++c) ul[c] = F(0);
                F py = F(0);
                // sender row times radial value / derivative once per order, not once per harmonic
                F Rv[CH], hv[CH], hd[CH];
                {
                    const V c0 = piece(0, l), c1 = piece(1, l), c2 = piece(2, l), c3 = piece(3, l);
#pragma unroll
                    for (int c = 0; c < CH; ++c) {
                        Rv[c] = c0.v[c] + x * (c1.v[c] + x * (c2.v[c] + x * c3.v[c]));
                        hv[c] = h.v[c] * Rv[c];
                        hd[c] = h.v[c] * (c1.v[c] + x * (F(2) * c2.v[c] + F(3) * x * c3.v[c]));
                    }
                }
                static_for<0, 2 * l + 1>([&](auto mc) {
                    constexpr int lm = l * l + decltype(mc)::value;
                    double y, g0, g1, g2;
                    ylm_g<lm>(vx, vy, vz, y, g0, g1, g2);
                    const V dd = *reinterpret_cast<const V*>(dstage + lm * ROWS * CH);
                    const F yf = (F)y;
                    F P = F(0), Q = F(0);
#pragma unroll
                    for (int c = 0; c < CH; ++c) {
                        P += dd.v[c] * hv[c];
                        Q += dd.v[c] * hd[c];
                        ul[c] += dd.v[c] * yf;
                    }
                    srad += Q * yf;
                    wx += P * (F)g0; wy += P * (F)g1; wz += P * (F)g2;
                    py += P * yf;
                });
                lterm += py * F(l);
#pragma unroll
                for (int c = 0; c < CH; ++c) mg[c] += Rv[c] * ul[c];
                order_l(srad, wx, wy, wz, lterm, vx, vy, vz);
#pragma unroll
                for (int c = 0; c < CH; ++c) pin_value(mg[c]);
            });
            // gradient with respect to the edge vector: (w - u (l-weighted sum)) / |v|, axes unpermuted;
            // radial part along xyz / r with the caller's r (mace.cpp:256-264, 558-566)
            const double sr = (double)srad, lt = (double)lterm;
            const double ir = rcp_pos(r);
            const bool carried = CARRY && e < p.fpart_carry;    // edges past fpart_carry hold nothing yet (read, not used)
            const double res0 = (carried ? f0 : 0.0) - (dx * ir * sr + ((double)wy - uy * lt) * inv);   // original x is permuted axis 1
            const double res1 = (carried ? f1 : 0.0) - (dy * ir * sr + ((double)wz - uz * lt) * inv);   // original y is permuted axis 2
            const double res2 = (carried ? f2 : 0.0) - (dz * ir * sr + ((double)wx - ux * lt) * inv);   // original z is permuted axis 0
            // the next edge (this very edge again after the last one: not used), then the stores
            take_edge(cu, nx);
            h = sender_row(cu.g);
            if constexpr (CARRY) { f0 = fpart[3 * (size_t)en]; f1 = fpart[3 * (size_t)en + 1]; f2 = fpart[3 * (size_t)en + 2]; }
            if constexpr (MSG) {
                F* dstm = a.msg + (size_t)e * K + kc;
                if (whole) {
                    V m;
#pragma unroll
                    for (int c = 0; c < CH; ++c) m.v[c] = mg[c];
                    *reinterpret_cast<V*>(dstm) = m;
                } else {
#pragma unroll
                    for (int c = 0; c < CH; ++c) if (kc + c < K) dstm[c] = mg[c];
                }
            }
            fpart[3 * (size_t)e] = res0; fpart[3 * (size_t)e + 1] = res1; fpart[3 * (size_t)e + 2] = res2;
        }
    }
}

__global__ void k_fpart_reduce(long n3, long stride3, int nslices, const double* fpart, double* forces, int accumulate,
                               double* copy, const int* guard)
{
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n3) return;
    double s = accumulate ? forces[t] : 0.0;
    for (int q = 0; q < nslices; ++q) s += fpart[(size_t)q * stride3 + t];
    // a skipped evaluation (inputs failed their checks) left nothing in fpart: its forces say so
    if (guard && *guard) s = __builtin_nan("");
    forces[t] = s;
    if (copy) copy[t] = s;
}

template <typename F, int CH, int CL, int BT, bool BWD>
hipError_t launch_slice_cfg(const SliceParams<F>& p, hipStream_t s)
{
    const int S = (p.a.K + CH - 1) / CH;
    const size_t lds = (size_t)(p.a.spl_nodes - 1) * p.W * sizeof(F);
    const int waves_per_block = BT / 64;
    // one block per CU (the slice fills most of its LDS); receiver groups share a slice
    int RG = p.num_cus / S;
    if (RG < 1) RG = 1;
    const long tasks_per_slice = ((long)p.a.num_nodes + 3) / 4;
    if ((long)RG * waves_per_block > tasks_per_slice) RG = (int)((tasks_per_slice + waves_per_block - 1) / waves_per_block);
    SliceParams<F> q = p;
    unsigned blocks = 0;
    place_blocks(q, S, RG, blocks);
    dim3 grid(blocks);
    void (*kern)(const SliceParams<F>) = nullptr;
    if constexpr (BWD) kern = k_slice_bwd<F, CH, CL, BT>;
    else kern = k_slice_fwd<F, CH, CL, BT>;
    if (lds > 64 * 1024) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
    }
    hipLaunchKernelGGL(kern, grid, dim3(BT), lds, s, q);
    return hipGetLastError();
}

// Four lanes per edge and twelve wavefronts per block measured best for both directions and both
// precisions: the kernels wait on dependent LDS reads and arithmetic chains, and a third wavefront
// per SIMD (168 registers each) hides more of that than wider per-lane work does.
template <typename F, int CH, bool BWD>
hipError_t launch_slice_t(const SliceParams<F>& p, hipStream_t s)
{
    if constexpr (CH % 4 == 0 && !BWD && sizeof(F) == 8 && CH == 4) return launch_slice_cfg<F, CH, 4, 1024, BWD>(p, s);
    else if constexpr (CH % 4 == 0) return launch_slice_cfg<F, CH, 4, 768, BWD>(p, s);
    else return launch_slice_cfg<F, CH, 2, 512, BWD>(p, s);
}

}  // namespace

template <typename F, int BT>
static hipError_t launch_slice_fwd_halves(const SliceParams<F>& p, hipStream_t s)
{
    constexpr int CH = 32 / (int)sizeof(F);
    const int S = (p.a.K + CH - 1) / CH;
    const size_t lds = (size_t)(p.a.spl_nodes - 1) * 512;
    int RG = p.num_cus / S;
    if (RG < 1) RG = 1;
    const long tasks_per_slice = ((long)p.a.num_nodes + 3) / 4;
    if ((long)RG * (BT / 64) > tasks_per_slice) RG = (int)((tasks_per_slice + BT / 64 - 1) / (BT / 64));
    auto kern = k_slice_fwd_halves<F, BT>;
    if (lds > 64 * 1024) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
    }
    SliceParams<F> q = p;
    unsigned blocks = 0;
    place_blocks(q, S, RG, blocks);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(BT), lds, s, q);
    return hipGetLastError();
}

template <typename F>
hipError_t launch_slice_fwd(const SliceParams<F>& p, hipStream_t s)
{
    if (p.a.num_nodes <= 0) return hipSuccess;
    if (p.tabF) return launch_slice_fwd_halves<F, 1024>(p, s);
    switch (p.CH) {
    case 2: return launch_slice_t<F, 2, false>(p, s);
    case 4: return launch_slice_t<F, 4, false>(p, s);
    case 8: return launch_slice_t<F, 8, false>(p, s);
    default: return hipErrorInvalidValue;
    }
}
// threads per block of the lane-per-edge adjoint kernel: three wavefronts per SIMD, up to 168 registers each (four
// per SIMD would need the table rows without their padding to fit the LDS, and plain 512-byte rows put every lane's
// piece on the same banks: twice the time)
template <typename F> constexpr int kEdgeBlock = 768;
template <typename F, int BT, int RL, bool MSG, bool CARRY, bool WHOLE>
static hipError_t launch_slice_bwd_edge_cfg(const SliceParams<F>& p, hipStream_t s)
{
    constexpr int CH = 32 / (int)sizeof(F), ROWS = 64 / RL;
    const int S = (p.a.K + CH - 1) / CH;
    const size_t lds = (size_t)(p.a.spl_nodes - 1) * p.W * sizeof(F) + (size_t)(BT / 64) * ROWS * 512;
    int RG = p.num_cus / S;
    if (RG < 1) RG = 1;
    const long tasks_per_slice = ((long)p.a.num_nodes + ROWS - 1) / ROWS;
    if ((long)RG * (BT / 64) > tasks_per_slice) RG = (int)((tasks_per_slice + BT / 64 - 1) / (BT / 64));
    auto kern = k_slice_bwd_edge<F, CH, BT, RL, MSG, CARRY, WHOLE>;
    if (lds > 64 * 1024) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
    }
    SliceParams<F> q = p;
    unsigned blocks = 0;
    place_blocks(q, S, RG, blocks);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(BT), lds, s, q);
    return hipGetLastError();
}
// Twelve wavefronts per block and sixteen lanes per receiver measured best (eight lanes per receiver fill the
// lanes better, 95 % against 80 % at 38 neighbours, but the staged adjoint rows of twice as many receivers leave
// room for six wavefronts only: 163 / 138 us against 154 / 114 us for the two adjoint stages of the 3 000-atom
// benchmark in double precision; eight wavefronts with sixteen lanes run like twelve).
template <typename F>
static hipError_t launch_slice_bwd_edge(const SliceParams<F>& p, hipStream_t s)
{
    // with or without messages and carried forces, every slice complete or not: compiled apart, so that the loop
    // body has no branches (a wait for a load counts the memory operations requested after it; where paths merge
    // it assumes the shorter one, and would wait for stores of the longer)
    constexpr int CH = 32 / (int)sizeof(F);
    const int variant = (p.a.msg ? 4 : 0) + (p.fpart_carry > 0 ? 2 : 0) + (p.a.K % CH == 0 ? 1 : 0);
    constexpr int BT = kEdgeBlock<F>;
    switch (variant) {
    case 0: return launch_slice_bwd_edge_cfg<F, BT, 16, false, false, false>(p, s);
    case 1: return launch_slice_bwd_edge_cfg<F, BT, 16, false, false, true>(p, s);
    case 2: return launch_slice_bwd_edge_cfg<F, BT, 16, false, true, false>(p, s);
    case 3: return launch_slice_bwd_edge_cfg<F, BT, 16, false, true, true>(p, s);
    case 4: return launch_slice_bwd_edge_cfg<F, BT, 16, true, false, false>(p, s);
    case 5: return launch_slice_bwd_edge_cfg<F, BT, 16, true, false, true>(p, s);
    case 6: return launch_slice_bwd_edge_cfg<F, BT, 16, true, true, false>(p, s);
    default: return launch_slice_bwd_edge_cfg<F, BT, 16, true, true, true>(p, s);
    }
}
template <typename F> int slice_edge_row_elements()
{
    // [4][4][CH] with CH * sizeof(F) = 32: 512 bytes, plus 16 so that consecutive rows start four banks apart
    // (pieces permuted by the row index inside unpadded rows conflicted more: 56 % against 42 % of the LDS cycles)
    return (512 + 16) / (int)sizeof(F);
}
template int slice_edge_row_elements<double>();
template int slice_edge_row_elements<float>();
template <typename F> size_t slice_edge_lds_bytes(int spl_nodes)
{
    return (size_t)(spl_nodes - 1) * slice_edge_row_elements<F>() * sizeof(F) + (size_t)(kEdgeBlock<F> / 64) * 4 * 512;
}
template size_t slice_edge_lds_bytes<double>(int);
template size_t slice_edge_lds_bytes<float>(int);

template <typename F>
hipError_t launch_slice_bwd(const SliceParams<F>& p, hipStream_t s)
{
    if (p.a.num_nodes <= 0) return hipSuccess;
    if (p.edge_lanes) return launch_slice_bwd_edge<F>(p, s);
    switch (p.CH) {
    case 2: return launch_slice_t<F, 2, true>(p, s);
    case 4: return launch_slice_t<F, 4, true>(p, s);
    case 8: return launch_slice_t<F, 8, true>(p, s);
    default: return hipErrorInvalidValue;
    }
}
template <typename F>
int slice_row_elements(int CH)
{
    int W = 16 * CH;
    if (slice_rotates<F>()) return (W * (int)sizeof(F)) % 128 == 0 ? W : 0;
    const int step = 16 / (int)sizeof(F);
    while (((W * (int)sizeof(F) / 4) / 4) % 2 == 0) W += step;   // rows start on different 16-byte bank groups
    return W;
}
template int slice_row_elements<double>(int);
template int slice_row_elements<float>(int);
template hipError_t launch_slice_fwd<double>(const SliceParams<double>&, hipStream_t);
template hipError_t launch_slice_fwd<float>(const SliceParams<float>&, hipStream_t);
template hipError_t launch_slice_bwd<double>(const SliceParams<double>&, hipStream_t);
template hipError_t launch_slice_bwd<float>(const SliceParams<float>&, hipStream_t);

hipError_t launch_fpart_reduce(long edges, long E, int nslices, const double* fpart, double* forces, int accumulate,
                               double* copy, hipStream_t s, const int* guard)
{
    const long n3 = 3 * edges;
    if (n3 <= 0 || edges > E) return n3 <= 0 ? hipSuccess : hipErrorInvalidValue;
    hipLaunchKernelGGL(k_fpart_reduce, dim3((unsigned)((n3 + 255) / 256)), dim3(256), 0, s, n3, 3 * E, nslices, fpart,
                       forces, accumulate, copy, guard);
    return hipGetLastError();
}

}  // namespace smx
