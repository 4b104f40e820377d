// Full neighbour list on the device in the canonical order of this library:
// receivers ascending; within a receiver senders ascending; several periodic
// images of one sender ordered by the index of their image shift (the caller
// lists the shifts in lexicographic order of their integer triples).
//
// The arithmetic that decides membership and fills xyz and r is spelled out
// with round-to-nearest intrinsics (no fused multiply-add), in the order
//     image = x_j + shift;  d = image - x_i;  r2 = (d0*d0 + d1*d1) + d2*d2
// so that the list is bit-identical to the host builder
// (symmetrix_amd/neighbors.py), whatever the compiler would contract.
#include "smx_kernels.hpp"

namespace smx {

namespace {

struct Cand {
    double d0, d1, d2, r2;
};
__device__ __forceinline__ Cand displacement(const double* pos, int i, int j, const double* sv)
{
    Cand c;
    c.d0 = __dsub_rn(__dadd_rn(pos[3 * (size_t)j], sv[0]), pos[3 * (size_t)i]);
    c.d1 = __dsub_rn(__dadd_rn(pos[3 * (size_t)j + 1], sv[1]), pos[3 * (size_t)i + 1]);
    c.d2 = __dsub_rn(__dadd_rn(pos[3 * (size_t)j + 2], sv[2]), pos[3 * (size_t)i + 2]);
    c.r2 = __dadd_rn(__dadd_rn(__dmul_rn(c.d0, c.d0), __dmul_rn(c.d1, c.d1)), __dmul_rn(c.d2, c.d2));
    return c;
}

__device__ __forceinline__ int bin_of(double x, double lo, double inv_bs, int nb)
{
    return min(max((int)floor((x - lo) * inv_bs), 0), nb - 1);
}

// per-block minima and maxima of the coordinates: part[block][6]
__global__ __launch_bounds__(256) void k_nl_bbox(const double* pos, int N, double* part)
{
    __shared__ double red[6][256];
    double lo[3] = {1e300, 1e300, 1e300}, hi[3] = {-1e300, -1e300, -1e300};
    for (int i = blockIdx.x * 256 + threadIdx.x; i < N; i += gridDim.x * 256)
        for (int k = 0; k < 3; ++k) {
            const double v = pos[3 * (size_t)i + k];
            lo[k] = fmin(lo[k], v); hi[k] = fmax(hi[k], v);
        }
    for (int k = 0; k < 3; ++k) { red[k][threadIdx.x] = lo[k]; red[3 + k][threadIdx.x] = hi[k]; }
    __syncthreads();
    for (int off = 128; off >= 1; off >>= 1) {
        if ((int)threadIdx.x < off)
            for (int k = 0; k < 3; ++k) {
                red[k][threadIdx.x] = fmin(red[k][threadIdx.x], red[k][threadIdx.x + off]);
                red[3 + k][threadIdx.x] = fmax(red[3 + k][threadIdx.x], red[3 + k][threadIdx.x + off]);
            }
        __syncthreads();
    }
    if (threadIdx.x < 6) part[blockIdx.x * 6 + threadIdx.x] = red[threadIdx.x][0];
}

__global__ void k_nl_bin_count(const double* pos, int N, NlGrid g, int* atom_bin, int* bin_count)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N) return;
    const int b0 = bin_of(pos[3 * (size_t)i], g.lo[0], g.inv_bs[0], g.nb[0]);
    const int b1 = bin_of(pos[3 * (size_t)i + 1], g.lo[1], g.inv_bs[1], g.nb[1]);
    const int b2 = bin_of(pos[3 * (size_t)i + 2], g.lo[2], g.inv_bs[2], g.nb[2]);
    const int b = (b0 * g.nb[1] + b1) * g.nb[2] + b2;
    atom_bin[i] = b;
    atomicAdd(&bin_count[b], 1);
}
__global__ void k_nl_bin_fill(int N, const int* atom_bin, const int* bin_start, int* bin_cursor, int* bin_atoms)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N) return;
    const int b = atom_bin[i];
    bin_atoms[bin_start[b] + atomicAdd(&bin_cursor[b], 1)] = i;
}

// One thread per receiver walks every image shift and the bins that the cutoff sphere of the shifted
// receiver can touch.  FILL = false counts, FILL = true writes the keys sender * num_shifts + shift index
// (in whatever order the bins deliver them: k_nl_sort orders them).
template <bool FILL>
__global__ void k_nl_search(const double* pos, int N, NlGrid g, const int* bin_start, const int* bin_atoms,
                            int num_shifts, const double* shift_vec, int zero_shift, double r_cut, double r2cut,
                            int* count, const int* first, long long* keys)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N) return;
    const double xi[3] = {pos[3 * (size_t)i], pos[3 * (size_t)i + 1], pos[3 * (size_t)i + 2]};
    const double reach = r_cut * (1.0 + 1e-9) + 1e-12;
    int c = 0;
    long long* out = FILL ? keys + first[i] : nullptr;
    for (int s = 0; s < num_shifts; ++s) {
        const double* sv = shift_vec + 3 * s;
        int blo[3], bhi[3];
        bool empty = false;
        for (int k = 0; k < 3; ++k) {
            const double q = xi[k] - sv[k];   // senders within reach of q see the receiver through shift s
            if (q + reach < g.lo[k] || q - reach > g.hi[k]) { empty = true; break; }
            blo[k] = bin_of(q - reach, g.lo[k], g.inv_bs[k], g.nb[k]);
            bhi[k] = bin_of(q + reach, g.lo[k], g.inv_bs[k], g.nb[k]);
        }
        if (empty) continue;
        for (int b0 = blo[0]; b0 <= bhi[0]; ++b0)
            for (int b1 = blo[1]; b1 <= bhi[1]; ++b1)
                for (int b2 = blo[2]; b2 <= bhi[2]; ++b2) {
                    const int b = (b0 * g.nb[1] + b1) * g.nb[2] + b2;
                    for (int t = bin_start[b]; t < bin_start[b + 1]; ++t) {
                        const int j = bin_atoms[t];
                        if (j == i && s == zero_shift) continue;
                        const Cand cd = displacement(pos, i, j, sv);
                        if (cd.r2 < r2cut) {
                            if (FILL) out[c] = (long long)j * num_shifts + s;
                            ++c;
                        }
                    }
                }
    }
    if (!FILL) count[i] = c;
}

// One wavefront per receiver: rank of every key among the receiver's keys (they are distinct); the keys are
// rewritten in ascending order, which is the canonical edge order of the receiver.
__global__ __launch_bounds__(256) void k_nl_sort(int N, const int* cfirst, const long long* keys, long long* sorted)
{
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (i >= N) return;
    const int e0 = cfirst[i], n = cfirst[i + 1] - e0;
    for (int a = lane; a < n; a += 64) {
        const long long key = keys[e0 + a];
        int rank = 0;
        for (int b = 0; b < n; ++b) rank += keys[e0 + b] < key ? 1 : 0;
        sorted[(size_t)e0 + rank] = key;
    }
}

// One wavefront per receiver walks its sorted candidates with the current positions and keeps those inside
// the cutoff, in order.  EMIT = false counts; EMIT = true writes the edge arrays at first[i] + (number kept before).
template <bool EMIT>
__global__ __launch_bounds__(256) void k_nl_filter(const double* pos, const int* types, int N, const int* cfirst,
                                                   const long long* sorted, int num_shifts, const double* shift_vec,
                                                   const int* shift_int, double r2cut, int* count, const int* first,
                                                   int* neigh_indices, int* neigh_types, int* neigh_shift, double* xyz,
                                                   double* r)
{
    const int i = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (i >= N) return;
    const int c0 = cfirst[i], n = cfirst[i + 1] - c0;
    int kept = 0;
    const size_t e0 = EMIT ? (size_t)first[i] : 0;
    for (int a0 = 0; a0 < n; a0 += 64) {
        const int a = a0 + lane;
        bool pass = false;
        int j = 0, s = 0;
        Cand cd{};
        if (a < n) {
            const long long key = sorted[(size_t)c0 + a];
            j = (int)(key / num_shifts); s = (int)(key % num_shifts);
            cd = displacement(pos, i, j, shift_vec + 3 * s);
            pass = cd.r2 < r2cut;
        }
        const unsigned long long mask = __ballot(pass);
        if (EMIT && pass) {
            const size_t e = e0 + kept + __popcll(mask & ((1ull << lane) - 1ull));
            neigh_indices[e] = j;
            neigh_types[e] = types ? types[j] : 0;
            neigh_shift[3 * e] = shift_int[3 * s]; neigh_shift[3 * e + 1] = shift_int[3 * s + 1];
            neigh_shift[3 * e + 2] = shift_int[3 * s + 2];
            xyz[3 * e] = cd.d0; xyz[3 * e + 1] = cd.d1; xyz[3 * e + 2] = cd.d2;
            r[e] = __dsqrt_rn(cd.r2);
        }
        kept += __popcll(mask);
    }
    if (!EMIT && lane == 0) count[i] = kept;
}

}  // namespace

hipError_t launch_nl_bbox(const double* pos, int N, double* part, int nblocks, hipStream_t s)
{
    hipLaunchKernelGGL(k_nl_bbox, dim3(nblocks), dim3(256), 0, s, pos, N, part);
    return hipGetLastError();
}
hipError_t launch_nl_bins(const double* pos, int N, const NlGrid& g, int* atom_bin, int* bin_count, hipStream_t s)
{
    if (N > 0) hipLaunchKernelGGL(k_nl_bin_count, dim3((N + 255) / 256), dim3(256), 0, s, pos, N, g, atom_bin, bin_count);
    return hipGetLastError();
}
hipError_t launch_nl_bin_fill(int N, const int* atom_bin, const int* bin_start, int* bin_cursor, int* bin_atoms,
                              hipStream_t s)
{
    if (N > 0) hipLaunchKernelGGL(k_nl_bin_fill, dim3((N + 255) / 256), dim3(256), 0, s, N, atom_bin, bin_start, bin_cursor, bin_atoms);
    return hipGetLastError();
}
hipError_t launch_nl_search(bool fill, const double* pos, int N, const NlGrid& g, const int* bin_start,
                            const int* bin_atoms, int num_shifts, const double* shift_vec, int zero_shift,
                            double r_cut, int* count, const int* first, long long* keys, hipStream_t s)
{
    if (N <= 0) return hipSuccess;
    const double r2cut = r_cut * r_cut;
    if (fill)
        hipLaunchKernelGGL(k_nl_search<true>, dim3((N + 63) / 64), dim3(64), 0, s, pos, N, g, bin_start, bin_atoms,
                           num_shifts, shift_vec, zero_shift, r_cut, r2cut, count, first, keys);
    else
        hipLaunchKernelGGL(k_nl_search<false>, dim3((N + 63) / 64), dim3(64), 0, s, pos, N, g, bin_start, bin_atoms,
                           num_shifts, shift_vec, zero_shift, r_cut, r2cut, count, first, keys);
    return hipGetLastError();
}
hipError_t launch_nl_sort(int N, const int* cfirst, const long long* keys, long long* sorted, hipStream_t s)
{
    if (N > 0) hipLaunchKernelGGL(k_nl_sort, dim3((N + 3) / 4), dim3(256), 0, s, N, cfirst, keys, sorted);
    return hipGetLastError();
}
hipError_t launch_nl_filter(bool emit, const double* pos, const int* types, int N, const int* cfirst,
                            const long long* sorted, int num_shifts, const double* shift_vec, const int* shift_int,
                            double r_cut, int* count, const int* first, int* neigh_indices, int* neigh_types,
                            int* neigh_shift, double* xyz, double* r, hipStream_t s)
{
    if (N <= 0) return hipSuccess;
    const double r2cut = r_cut * r_cut;
    if (emit)
        hipLaunchKernelGGL(k_nl_filter<true>, dim3((N + 3) / 4), dim3(256), 0, s, pos, types, N, cfirst, sorted, num_shifts,
                           shift_vec, shift_int, r2cut, count, first, neigh_indices, neigh_types, neigh_shift, xyz, r);
    else
        hipLaunchKernelGGL(k_nl_filter<false>, dim3((N + 3) / 4), dim3(256), 0, s, pos, types, N, cfirst, sorted, num_shifts,
                           shift_vec, shift_int, r2cut, count, first, neigh_indices, neigh_types, neigh_shift, xyz, r);
    return hipGetLastError();
}

}  // namespace smx
